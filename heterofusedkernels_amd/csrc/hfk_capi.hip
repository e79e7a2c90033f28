// libhfk_hip.so: gfx950 kernels and the extern "C" entry points of include/hfk.h.
//
// Launch shape: grids are 1-D, workgroups of 256 lanes, each workgroup walking
// work items bid, bid + grid, ... (a grid-stride loop with a hard upper bound, so
// every wave terminates). The grid is capped at CUs * workgroups-per-CU, which on
// MI355X (256 CUs, 8 XCDs) both fills every XCD evenly -- workgroups are handed
// to XCDs round-robin, and a work item's neighbours bid+-1 sit on other XCDs while
// the item itself streams one contiguous span, so no XCD's L2 sees another's lines
// -- and lets a caller bound the grid (the `workgroups` argument). PCIe-bound
// launches default to a small grid: the link needs no more, and whatever a grid
// keeps in flight beyond the link's bandwidth-delay product queues in the memory
// fabric in front of every other kernel's traffic (a memory-bound kernel on another
// stream runs up to 5x slower beside an oversized swap). A swap that must share the
// GPU says so (HFK_SWAP_BESIDE_COMPUTE: 8-16 workgroups, paced toward the host) or
// goes through hfk_swap_blocks_staged (HBM-only kernel + DMA copies).
#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>
#include <vector>
#include <cctype>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <type_traits>

#include "hfk.h"
#include "hfk_bodies.h"
#include "hfk_plan.h"

namespace {

using hfk::BlockCopyArgs;
using hfk::DuplexCopyArgs;
using hfk::FlatGatherArgs;
using hfk::TransposeArgs;
using hfk::kWorkgroupLanes;
using hfk::vec16;

// One body, four kernel names: the block-copy body serves the swap, the multi-plane
// block gather, the scatter out of a staging buffer and wide-row gathers, and a
// profile should say which one ran.
enum class Role { kSwapBlocks, kGatherBlocks, kGatherRows, kScatterBlocks };

// The same three, restricted by the run filter to one share of a table that is split between the
// copy engines and the compute units (hfk_swap_blocks_auto).
template <int UNROLL, int NT>
__global__ __launch_bounds__(256) void swap_short_runs_kernel(const BlockCopyArgs<int64_t> a) {
    hfk::block_copy_body<int64_t, UNROLL, NT, true>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

template <int UNROLL, int NT>
__global__ __launch_bounds__(256) void gather_long_runs_kernel(const BlockCopyArgs<int64_t> a) {
    hfk::block_copy_body<int64_t, UNROLL, NT, true, false>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

template <int UNROLL, int NT>
__global__ __launch_bounds__(256) void scatter_long_runs_kernel(const BlockCopyArgs<int64_t> a) {
    hfk::block_copy_body<int64_t, UNROLL, NT, true, false>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

// The same three again, handed the list of their pairs (hfk::kListedPairs): what hfk_swap_blocks_auto launches
// when it has room for the lists, so that no workgroup is started for a pair another mover takes.
template <int UNROLL, int NT>
__global__ __launch_bounds__(256) void swap_listed_pairs_kernel(const BlockCopyArgs<int64_t> a) {
    hfk::block_copy_body<int64_t, UNROLL, NT, false, true, true>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

template <int UNROLL, int NT>
__global__ __launch_bounds__(256) void gather_listed_pairs_kernel(const BlockCopyArgs<int64_t> a) {
    hfk::block_copy_body<int64_t, UNROLL, NT, false, false, true>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

template <int UNROLL, int NT>
__global__ __launch_bounds__(256) void scatter_listed_pairs_kernel(const BlockCopyArgs<int64_t> a) {
    hfk::block_copy_body<int64_t, UNROLL, NT, false, false, true>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

template <int UNROLL, int NT>
__global__ __launch_bounds__(256) void swap_blocks_kernel(const BlockCopyArgs<int64_t> a) {
    hfk::block_copy_body<int64_t, UNROLL, NT>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

template <int UNROLL, int NT>
__global__ __launch_bounds__(256) void gather_blocks_kernel(const BlockCopyArgs<int64_t> a) {
    hfk::block_copy_body<int64_t, UNROLL, NT, false, false>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

template <int UNROLL, int NT>
__global__ __launch_bounds__(256) void scatter_blocks_kernel(const BlockCopyArgs<int64_t> a) {
    hfk::block_copy_body<int64_t, UNROLL, NT, false, false>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

template <typename IdT, int UNROLL, int NT>
__global__ __launch_bounds__(256) void gather_rows_wide_kernel(const BlockCopyArgs<IdT> a) {
    hfk::block_copy_body<IdT, UNROLL, NT, false, false>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

template <int UNROLL, int NT>
__global__ __launch_bounds__(256) void swap_blocks_duplex_kernel(const DuplexCopyArgs a) {
    hfk::duplex_copy_body<UNROLL, NT>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

template <typename V, typename IdT, typename IndexT, int UNROLL, int NT>
__global__ __launch_bounds__(256) void flat_gather_kernel(const FlatGatherArgs<IdT> a) {
    hfk::flat_gather_body<V, IdT, IndexT, UNROLL, NT>(a, blockIdx.x, gridDim.x, threadIdx.x);
}

// The transfer kernels keep the layer-address table in LDS (see LayerTableInMemory): 512 layers, 4 KiB.
constexpr uint32_t kLayerTableLdsEntries = 512;

struct LayerTableInLds {
    const uint64_t* table;   // points into LDS; after inlining the reads are ds_read_b64
    __device__ uint64_t operator()(uint32_t l) const { return table[l]; }
};

template <typename V, int UNROLL, int NT, bool TO_PACKED, bool MIRROR = false>
__device__ void transpose_with_layer_table(const TransposeArgs& a) {
    __shared__ uint64_t layer_table[kLayerTableLdsEntries];
    if (a.L <= kLayerTableLdsEntries) {   // uniform over the grid
        for (uint32_t l = threadIdx.x; l < a.L; l += 256) layer_table[l] = hfk::table_entry(a.layer_ptrs, l);
        __syncthreads();
        hfk::transpose_body<V, UNROLL, NT, TO_PACKED, MIRROR>(a, blockIdx.x, gridDim.x, threadIdx.x,
                                                              LayerTableInLds{layer_table});
    } else {
        hfk::transpose_body<V, UNROLL, NT, TO_PACKED, MIRROR>(a, blockIdx.x, gridDim.x, threadIdx.x);
    }
}

// Packed [T,L,H,D] blocks -> per-layer [H,T,D] caches (the reference's direction) ...
template <typename V, int UNROLL, int NT>
__global__ __launch_bounds__(256) void transpose_kernel(const TransposeArgs a) {
    transpose_with_layer_table<V, UNROLL, NT, false>(a);
}

// The same, also writing every unit it reads to a second copy of the packed blocks (a.mirror): the staged
// single-block transfer in one kernel.
template <typename V, int UNROLL, int NT>
__global__ __launch_bounds__(256) void transpose_and_stage_kernel(const TransposeArgs a) {
    transpose_with_layer_table<V, UNROLL, NT, false, true>(a);
}

// ... and back: per-layer caches -> packed blocks.
template <typename V, int UNROLL, int NT>
__global__ __launch_bounds__(256) void transpose_to_packed_kernel(const TransposeArgs a) {
    transpose_with_layer_table<V, UNROLL, NT, true>(a);
}

// The same toward the packed side, tiled through LDS (see transpose_tile_load): 1 KiB runs on both sides.
template <int U, int NT>
__global__ __launch_bounds__(256) void transpose_to_packed_tiled_kernel(const TransposeArgs a) {
    __shared__ uint64_t layer_table[kLayerTableLdsEntries];
    __shared__ vec16 tile[64 * 4 * U];
    for (uint32_t l = threadIdx.x; l < a.L; l += 256) layer_table[l] = hfk::table_entry(a.layer_ptrs, l);
    __syncthreads();
    const LayerTableInLds layer_address{layer_table};
    hfk::Pacer pacer(a.pace_q8, blockIdx.x, gridDim.x);
    for (uint64_t w = blockIdx.x; w < a.n_work; w += gridDim.x) {
        hfk::TransposeTile it;
        if (!hfk::transpose_tile_item(a, w, it)) continue;   // uniform over the workgroup
        pacer.wait_turn();
        hfk::transpose_tile_load<U, NT>(a, it, threadIdx.x, layer_address, tile);
        __syncthreads();
        hfk::transpose_tile_store<U, NT>(a, it, threadIdx.x, tile);
        __syncthreads();
    }
}

// The two lists of a split table (see hfk::fill_pair_lists, which states the result), by one workgroup in three
// passes over the table, 256 pairs at a time, each pass a scan with a value carried from batch to batch. No
// pass looks further than a pair's neighbour, so the cost does not depend on how long the runs are or on the
// threshold. short_list doubles as the scratch of the first two passes: the third reads an entry before any
// lane of its batch writes, and a pair's place in the short list is never behind the pair.
//   1, forward:  where the run a pair belongs to starts (the last pair at or before it whose predecessor's id
//                is not its own less one), into short_list[j];
//   2, backward: where the next run starts (the first such pair after it, or n), hence the run's length, hence
//                whether the pair is in a long run, into short_list[j];
//   3, forward:  both lists by a running count of the pairs in long runs; what is left of either list is -1.
__global__ __launch_bounds__(256) void pair_lists_kernel(const int64_t* ids, uint32_t stride, uint32_t n, uint32_t min_run,
                                                         int64_t* long_list, int64_t* short_list) {
    __shared__ uint32_t scan[256];
    __shared__ uint32_t carried;
    const uint32_t tid = threadIdx.x;
    constexpr uint32_t kNone = 0xffffffffu;
    if (tid == 0) carried = 0;           // pass 1: start of the run that reaches into this batch
    __syncthreads();
    for (uint32_t base = 0; base < n; base += 256) {
        const uint32_t j = base + tid;
        const bool starts = j < n && (j == 0 || hfk::table_entry(ids, (uint64_t)(j - 1) * stride) + 1 !=
                                                    hfk::table_entry(ids, (uint64_t)j * stride));
        scan[tid] = starts ? j : 0u;
        __syncthreads();
        for (uint32_t step = 1; step < 256; step <<= 1) {     // inclusive maximum over the lanes up to this one
            const uint32_t other = tid >= step ? scan[tid - step] : 0u;
            __syncthreads();
            if (other > scan[tid]) scan[tid] = other;
            __syncthreads();
        }
        const uint32_t start = scan[tid] > carried ? scan[tid] : carried;
        if (j < n) short_list[j] = (int64_t)start;
        __syncthreads();
        if (tid == 255) carried = start;
        __syncthreads();
    }
    if (tid == 0) carried = n;           // pass 2: where the first run after this batch starts
    __syncthreads();
    for (uint32_t base = ((n - 1) / 256) * 256;; base -= 256) {
        const uint32_t j = base + tid;
        const uint32_t start = j < n ? (uint32_t)short_list[j] : 0u;
        scan[tid] = (j < n && start == j) ? j : kNone;
        __syncthreads();
        for (uint32_t step = 1; step < 256; step <<= 1) {     // inclusive minimum over the lanes from this one on
            const uint32_t other = tid + step < 256 ? scan[tid + step] : kNone;
            __syncthreads();
            if (other < scan[tid]) scan[tid] = other;
            __syncthreads();
        }
        uint32_t next = tid < 255 ? scan[tid + 1] : kNone;    // the first start after this pair
        if (carried < next) next = carried;
        const uint32_t first_start = scan[0] < carried ? scan[0] : carried;
        __syncthreads();
        if (j < n) short_list[j] = (next - start >= min_run) ? 1 : 0;
        if (tid == 0) carried = first_start;
        __syncthreads();
        if (base == 0) break;
    }
    if (tid == 0) carried = 0;           // pass 3: pairs in long runs before this batch
    __syncthreads();
    for (uint32_t base = 0; base < n; base += 256) {
        const uint32_t j = base + tid;
        const uint32_t is_long = j < n && short_list[j] != 0 ? 1u : 0u;
        scan[tid] = is_long;
        __syncthreads();
        for (uint32_t step = 1; step < 256; step <<= 1) {     // inclusive sum over the lanes up to this one
            const uint32_t add = tid >= step ? scan[tid - step] : 0u;
            __syncthreads();
            scan[tid] += add;
            __syncthreads();
        }
        if (j < n) {
            const uint32_t long_before = carried + scan[tid] - is_long;    // pairs in long runs among 0 .. j - 1
            if (is_long) long_list[long_before] = (int64_t)j;
            else short_list[j - long_before] = (int64_t)j;
        }
        __syncthreads();
        if (tid == 255) carried += scan[255];
        __syncthreads();
    }
    const uint32_t n_long = carried;
    for (uint32_t i = n_long + tid; i < n; i += 256) long_list[i] = -1;
    for (uint32_t i = n - n_long + tid; i < n; i += 256) short_list[i] = -1;
}

// ---- tuning state ---------------------------------------------------------
// Defaults are the measured best on MI355X:
//  * HBM-bound launches (gathers, the staged swap's kernel): ONE 16-byte vector per lane, i.e. 4 KiB
//    per workgroup, one workgroup per chunk, non-temporal loads and stores. A compute unit holds 8
//    such workgroups (32 KiB in flight per unit, 8 MiB on the chip), and the finer the chunks, the
//    more evenly the traffic spreads: 6.28-6.36 TB/s on 32 KiB blocks where 8 vectors per lane
//    reach 5.5-6.0, 6.5-6.6 TB/s on 72 KiB and 16 KiB blocks (with more in flight per lane the best
//    rate needs the resident workgroups bounded to about 48 KiB per unit, HFK_KNOB_HBM_LDS_BYTES,
//    and stays below this one). A grid-stride loop over fewer workgroups loses 5-10 %, so the grid
//    bound is high enough to stay inactive (CUs x 65536 workgroups).
//  * non-temporal accesses: +15-20 % over plain ones (the data is touched once).
//  * PCIe-bound swaps about which nothing is known are flat from 16 to 128 workgroups (55.4-56.0
//    GB/s out, 57.0-57.4 in); what grows with the grid is the harm to kernels on other streams (a
//    memory-bound neighbour runs 2.3-3x slower beside 16 workgroups, 4-5.7x beside 64), so such a
//    swap defaults to 16. For the same reason the duplex swap defaults to 32 workgroups (98.2 GB/s
//    summed against 99.1 at 128, neighbours 1.1-1.6x slower instead of 2.8-2.9x), a block-table
//    transfer out of host memory to 24 and one into host memory to 32 (see launch_transpose).
//
// Every knob has a process-wide value (hfk_set_tuning) and, per thread, an optional override that
// lasts from hfk_thread_tuning_begin to hfk_thread_tuning_end: a caller that wants a launch shape
// of its own for a few calls changes nothing another thread can see.
constexpr int kKnobCount = 21;
std::atomic<int64_t> g_knob[kKnobCount] = {
    1,       // HFK_KNOB_UNROLL
    3,       // HFK_KNOB_NONTEMPORAL
    65536,   // HFK_KNOB_WORKGROUPS_PER_CU
    16,      // HFK_KNOB_SWAP_WORKGROUPS
    1,       // HFK_KNOB_DUPLEX_UNROLL
    8,       // HFK_KNOB_SWAP_UNROLL
    0,       // HFK_KNOB_SWAP_PACE_MBPS
    -1,      // HFK_KNOB_LINK_MBPS
    32,      // HFK_KNOB_DUPLEX_WORKGROUPS
    0,       // HFK_KNOB_THROUGHPUT_PACE_PERMILLE
    0,       // HFK_KNOB_HBM_LDS_BYTES
    4,       // HFK_KNOB_PACED_UNROLL
    6,       // HFK_KNOB_PACED_WORKGROUPS
    0,       // HFK_KNOB_PACE_REPORT
    890,     // HFK_KNOB_DUPLEX_PACE_PERMILLE
    0,       // HFK_KNOB_TRANSFER_PACE_PERMILLE
    8,       // HFK_KNOB_TRANSFER_UNROLL
    0,       // HFK_KNOB_CHECK_HOST_COLUMN
    1,       // HFK_KNOB_TRANSFER_TILED
    1,       // HFK_KNOB_ADAPTIVE_PACE
    0,       // HFK_KNOB_FUSED_COPY_ENGINE
};

struct ThreadTuning {
    uint32_t mask = 0;                 // bit k: this thread overrides knob k
    int64_t value[kKnobCount] = {};
};
thread_local ThreadTuning t_tuning;

int64_t knob_value(int k) {
    return ((t_tuning.mask >> k) & 1u) != 0 ? t_tuning.value[k] : g_knob[k].load(std::memory_order_relaxed);
}

bool is_unroll(int64_t v) { return v == 1 || v == 2 || v == 4 || v == 8 || v == 16; }

bool knob_value_valid(int k, int64_t v) {
    switch (k) {
        case HFK_KNOB_UNROLL:
        case HFK_KNOB_DUPLEX_UNROLL:
        case HFK_KNOB_SWAP_UNROLL:
        case HFK_KNOB_PACED_UNROLL: return is_unroll(v);
        case HFK_KNOB_NONTEMPORAL: return v >= 0 && v <= 3;
        case HFK_KNOB_WORKGROUPS_PER_CU: return v >= 1 && v <= 65536;
        case HFK_KNOB_SWAP_WORKGROUPS:
        case HFK_KNOB_DUPLEX_WORKGROUPS:
        case HFK_KNOB_PACED_WORKGROUPS: return v >= 1 && v <= (1 << 20);
        case HFK_KNOB_SWAP_PACE_MBPS: return v >= 0 && v <= 1000000;
        case HFK_KNOB_LINK_MBPS: return v >= -1 && v <= 1000000;
        case HFK_KNOB_THROUGHPUT_PACE_PERMILLE: return v >= 0 && v <= 2000;
        case HFK_KNOB_HBM_LDS_BYTES: return v >= 0 && v <= 65536;
        case HFK_KNOB_PACE_REPORT: return (v & 7) == 0;   // an address of 64-bit words, or 0
        case HFK_KNOB_DUPLEX_PACE_PERMILLE:
        case HFK_KNOB_TRANSFER_PACE_PERMILLE: return v >= 0 && v <= 2000;
        case HFK_KNOB_TRANSFER_UNROLL: return v == 2 || v == 8;
        case HFK_KNOB_CHECK_HOST_COLUMN:
        case HFK_KNOB_TRANSFER_TILED:
        case HFK_KNOB_ADAPTIVE_PACE:
        case HFK_KNOB_FUSED_COPY_ENGINE: return v == 0 || v == 1;
        default: return false;
    }
}

constexpr uint32_t kBesideDuplexWorkgroups = 16;
constexpr int kBesideDuplexUnroll = 2;
constexpr uint32_t kBesideTransferWorkgroups = 16;
constexpr uint32_t kTransferToHostWorkgroups = 32;
constexpr uint32_t kShortTransferToHostWorkgroups = 64;     // under 128 MiB
constexpr uint64_t kShortTransferBytes = 128ull << 20;
constexpr uint32_t kShorterTransferToHostWorkgroups = 128;  // under 64 MiB
constexpr uint64_t kShorterTransferBytes = 64ull << 20;
constexpr uint32_t kTransferFromHostWorkgroups = 24;
// One block out of host memory, 4 / 8 / 32 / 64 MiB. The rate over the grid is not smooth: the direct transfer gives
// 53.2 / 55.3 / 57.0 / 57.3 GB/s on 32 workgroups (24: 0.3 below) and 50.2 / 52.2 / 53.8 / 54.2 on 48-56; the
// variant that fills the staging buffer as well gives 52.9 / 55.0 / 56.9 / 57.2 on 64 (48-72 within 0.3) and
// 49.1 / 52.1 / 54.4 / 55.0 on 24. Each sits in the middle of its plateau.
constexpr uint32_t kSingleBlockTransferWorkgroups = 32;
constexpr uint32_t kSingleBlockStagedTransferWorkgroups = 64;
constexpr uint32_t kHostGatherWorkgroups = 64;
constexpr uint64_t kLongHostGatherBytes = 4ull << 20;
constexpr uint64_t kAskTableSideBytes = 64ull << 10;
// The duplex swap wants little in flight per workgroup: one vector per lane and direction
// (unroll 8 loses 6 %). 32 workgroups reach 98.1-98.4 GB/s summed for 16, 32 and 72 KiB
// blocks; 40-64 dip to 89-94, 96-192 are a flat 98-99.

// Launch shapes of a swap whose host side the caller has named. What a host-facing launch keeps in
// flight beyond the link's bandwidth-delay product (about 64 KiB toward the host, 128 KiB from it)
// does not make it faster; it queues in the memory fabric in front of every other kernel's traffic.
// The gentlest shape that still fills the link is the finest one: ONE 16-byte vector per lane (4 KiB
// per workgroup iteration) and just enough workgroups. Measured on MI355X with 32 KiB blocks, as
// own rate / slowdown of a 1 GiB device copy / of a bf16 8192^3 GEMM on another stream:
//  * toward the host, paced (workgroups x vectors per lane):
//      12 x 1 at 0.90 of the link: 56.4 GB/s / 1.05x / 2.2x      16 x 4 at 0.90: 55.9 / 2.9x / 4.3x
//      16 x 1 at 0.90:             56.6 GB/s / 1.08x / 2.7x
//      12 x 1 at 0.84:             52.8 GB/s / 1.05x / 1.64x     8 x 4 at 0.84: 52.2 / 1.64x / 1.75x
//    (8 x 1 cannot hold the pace: 42.9 GB/s; unpaced, small grids are erratic: 38-48 GB/s);
//  * from the host, unpaced (pacing changes nothing there):
//      24 x 1: 55.9 GB/s / 1.30x / 1.58x     40 x 1: 57.4 / 1.95x / 1.59x     16 x 4: 57.4 / 3.4x / 1.58x
//    the copy's slowdown follows what is in flight, the GEMM's (1.5-1.6x) is what any resident kernel
//    costs it (one wavefront that only sleeps: 1.50x).
// Toward the host, throughput mode: unpaced by default, 96 vectors per lane in flight over the grid
// (12 workgroups x 8 for blocks of 32 KiB and more, see hfk::to_host_shape) with non-temporal loads
// and PLAIN stores: 56.6-56.7 GB/s on every kind of block table (55.9 on a slower host), 0.899 of
// the link's raw rate and 99 % of what hipMemcpy reaches, against 55.9-56.2 with non-temporal stores (which reach the link as
// 1.4 % more write requests than the payload has lines; plain ones go through the L2, which hands the
// link whole lines). It is the fast shape, not the gentle one: a device copy / SDPA / GEMM on another
// stream runs 5.9x / 2.9x / 4.0x slower meanwhile.
// Paced (HFK_KNOB_THROUGHPUT_PACE_PERMILLE != 0: HFK_KNOB_PACED_WORKGROUPS x HFK_KNOB_PACED_UNROLL
// with non-temporal stores) the same swap is gentler, 1.35x / 1.32x / 2.5x at 0.89 of the link on
// 6 x 4, and was the default until its rate turned out to follow the machine: a paced launch holds
// its schedule to 0.01 % (ran / allotted ticks in its pace report, on every machine tried), so it
// delivers its offered rate times whatever that machine's 100 MHz counter really runs at, and 0.89
// was 55.9 GB/s on one box, 55.5 on a second and 54.9 on a third, while the link's knee (0.905: 13 %
// of the turns begin late, against 2 % at 0.89) leaves no room to offer more. An unpaced launch
// depends on no clock. Measured while pacing was the default, over eight address patterns
// (consecutive, strided, descending, runs of 8, random; 12 launches each):
//   0.90: 16 x 1 53.2-56.5 GB/s by pattern, single launches down to 52.6; 6 x 4 56.4-56.6, single
//         launches down to 50.7 and one benchmark run at 49.8; 32 x 1 55.6-56.6;
//   0.89: every shape within 55.5-56.0 on every pattern; 6 x 4 56.0 on all eight.
// A swap that should be gentle says so (HFK_SWAP_BESIDE_COMPUTE) and gets the fine shape at 0.84,
// which it holds on every pattern (52.3-52.8 GB/s; 1.05x / 1.08x / 1.6x).
// Share of the link's raw rate offered to host writes when pacing. 256-byte transaction payloads
// cap the link at 0.90 of raw (56.8 of 63.0 GB/s measured, reached only by a paced grid); from 0.92
// on throughput collapses to 0.84 and the neighbours' slowdown doubles. The closer to the cap, the
// longer the fabric's queues: a GEMM beside the 12 x 1 swap runs 1.64x slower at 0.84
// (hfk::kBesidePaceShareOfLink), 1.93x at 0.88, 2.2x at 0.90 (1.5-1.6x is what any resident kernel
// costs this GEMM).
using hfk::kLongSwapBytes;
constexpr double kPaceShareOfLink = hfk::kBesidePaceShareOfLink;

constexpr int kMaxDevices = 64;
std::atomic<int> g_cu_count[kMaxDevices];

int current_cu_count(int* out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev >= 0 && dev < kMaxDevices) {
        int c = g_cu_count[dev].load(std::memory_order_relaxed);
        if (c > 0) {
            *out = c;
            return 0;
        }
    }
    int cus = 0;
    e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e != hipSuccess) return (int)e;
    if (cus <= 0) cus = 1;
    if (dev >= 0 && dev < kMaxDevices) g_cu_count[dev].store(cus, std::memory_order_relaxed);
    *out = cus;
    return 0;
}

// Ticks per second of the counter the pacer reads (wall_clock64): 100 MHz on MI355X; asked of the
// runtime once per device rather than assumed, and assumed where the runtime does not say.
std::atomic<int> g_wall_clock_khz[kMaxDevices];

double pacer_ticks_per_second() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) {
        (void)hipGetLastError();
        return 1e8;
    }
    int khz = g_wall_clock_khz[dev].load(std::memory_order_relaxed);
    if (khz == 0) {
        if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || khz <= 0) {
            (void)hipGetLastError();
            khz = 100000;
        }
        g_wall_clock_khz[dev].store(khz, std::memory_order_relaxed);
    }
    return khz * 1e3;
}

// The pacer's interval for work items of `item_bytes` on `grid` workgroups at `pace_mbps`, in 1/256 ticks.
uint32_t pace_interval_q8(double item_bytes, uint32_t grid, uint32_t pace_mbps) {
    const double q8 = item_bytes * grid / ((double)pace_mbps * 1e6) * pacer_ticks_per_second() * 256.0 + 0.5;
    return q8 < 4294967295.0 ? (uint32_t)q8 : 0xffffffffu;   // absurdly low rates: the wait's spin limit rules
}

int pick_grid(uint32_t n_work, uint32_t workgroups, uint32_t* grid) {
    uint32_t cap = workgroups;
    if (cap == 0) {
        int cus = 0;
        int rc = current_cu_count(&cus);
        if (rc != 0) return rc;
        cap = (uint32_t)cus * (uint32_t)knob_value(HFK_KNOB_WORKGROUPS_PER_CU);
    }
    *grid = n_work < cap ? n_work : cap;
    return 0;
}

int finish_launch() {
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? HFK_OK : (int)e;
}

// Raw PCIe rate of a device's link in MB/s (lanes x GT/s x line encoding), from sysfs; 0 if unknown.
std::atomic<int> g_link_mbps[kMaxDevices];   // 0 = not read yet, -1 = unknown

// One sysfs attribute of a PCI device as text ("" when unreadable).
void read_pci_attribute(const char* bdf, const char* name, char* out, size_t out_size) {
    out[0] = 0;
    char path[160];
    std::snprintf(path, sizeof(path), "/sys/bus/pci/devices/%s/%s", bdf, name);
    if (FILE* f = std::fopen(path, "r")) {
        if (std::fgets(out, (int)out_size, f) == nullptr) out[0] = 0;
        std::fclose(f);
    }
}

// The link's rate as trained at its best: a link that idles in a low-power speed, or that is read
// while it retrains, reports less in current_link_* than it delivers under load, and a pace derived
// from that would throttle every paced swap for the life of the process. A pace that is too high
// degrades gracefully (the launch behaves like an unpaced one), one that is too low does not, so the
// larger of the current and the maximum rate is used. HFK_KNOB_LINK_MBPS overrides both.
int read_link_mbps(int dev) {
    char bdf[32] = {0};
    if (hipDeviceGetPCIBusId(bdf, (int)sizeof(bdf), dev) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    for (char* c = bdf; *c; ++c) *c = (char)std::tolower((unsigned char)*c);
    char speed[64], width[64];
    read_pci_attribute(bdf, "current_link_speed", speed, sizeof(speed));
    read_pci_attribute(bdf, "current_link_width", width, sizeof(width));
    const int now = hfk::link_mbps_from_sysfs(speed, width);
    read_pci_attribute(bdf, "max_link_speed", speed, sizeof(speed));
    read_pci_attribute(bdf, "max_link_width", width, sizeof(width));
    const int best = hfk::link_mbps_from_sysfs(speed, width);
    return now > best ? now : best;
}

int current_link_mbps() {
    const int64_t forced = knob_value(HFK_KNOB_LINK_MBPS);
    if (forced >= 0) return (int)forced;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) {
        (void)hipGetLastError();
        return 0;
    }
    if (dev < 0 || dev >= kMaxDevices) return 0;
    int v = g_link_mbps[dev].load(std::memory_order_relaxed);
    if (v == 0) {
        v = read_link_mbps(dev);
        g_link_mbps[dev].store(v, std::memory_order_relaxed);
    }
    return v > 0 ? v : 0;
}

// The eight words behind a pace that is set between launches (hfk::pace_factor): one set per device, in the
// library's device image like the staging array below, zero until the first paced launch has settled.
static __device__ __align__(32) uint32_t pace_state_words[8];
std::atomic<void*> g_pace_state_ptr[kMaxDevices];

int pace_state(uint32_t** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return HFK_ERR_TOO_LARGE;
    void* ptr = g_pace_state_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(pace_state_words));   // `dev` is current: its copy of the words
        if (e != hipSuccess) return (int)e;
        if (ptr == nullptr) return (int)hipErrorInvalidSymbol;
        g_pace_state_ptr[dev].store(ptr, std::memory_order_release);
    }
    *out = static_cast<uint32_t*>(ptr);
    return HFK_OK;
}

// ---- block copy -----------------------------------------------------------
template <Role ROLE, typename IdT, int UNROLL, int NT>
void launch_block_copy_one(const BlockCopyArgs<IdT>& a, uint32_t grid, uint32_t lds, hipStream_t s) {
    if constexpr (std::is_same<IdT, int64_t>::value && ROLE != Role::kGatherRows) {
        if (a.run_mode == hfk::kListedPairs) {
            if constexpr (ROLE == Role::kSwapBlocks) {
                hipLaunchKernelGGL((swap_listed_pairs_kernel<UNROLL, NT>), dim3(grid), dim3(256), lds, s, a);
            } else if constexpr (ROLE == Role::kGatherBlocks) {
                hipLaunchKernelGGL((gather_listed_pairs_kernel<UNROLL, NT != 0 ? 3 : 0>), dim3(grid), dim3(256), lds, s, a);
            } else {
                hipLaunchKernelGGL((scatter_listed_pairs_kernel<UNROLL, NT != 0 ? 3 : 0>), dim3(grid), dim3(256), lds, s, a);
            }
            return;
        }
        if (a.run_mode != hfk::kAllPairs) {   // a split table: non-temporal or plain, nothing in between
            constexpr int SNT = NT != 0 ? 3 : 0;
            if constexpr (ROLE == Role::kSwapBlocks) {
                hipLaunchKernelGGL((swap_short_runs_kernel<UNROLL, SNT>), dim3(grid), dim3(256), lds, s, a);
            } else if constexpr (ROLE == Role::kGatherBlocks) {
                hipLaunchKernelGGL((gather_long_runs_kernel<UNROLL, SNT>), dim3(grid), dim3(256), lds, s, a);
            } else {
                hipLaunchKernelGGL((scatter_long_runs_kernel<UNROLL, SNT>), dim3(grid), dim3(256), lds, s, a);
            }
            return;
        }
    }
    if constexpr (ROLE == Role::kSwapBlocks) {
        hipLaunchKernelGGL((swap_blocks_kernel<UNROLL, NT>), dim3(grid), dim3(256), lds, s, a);
    } else if constexpr (ROLE == Role::kGatherBlocks) {
        hipLaunchKernelGGL((gather_blocks_kernel<UNROLL, NT>), dim3(grid), dim3(256), lds, s, a);
    } else if constexpr (ROLE == Role::kScatterBlocks) {
        hipLaunchKernelGGL((scatter_blocks_kernel<UNROLL, NT>), dim3(grid), dim3(256), lds, s, a);
    } else {
        hipLaunchKernelGGL((gather_rows_wide_kernel<IdT, UNROLL, NT>), dim3(grid), dim3(256), lds, s, a);
    }
}

template <Role ROLE, typename IdT, int UNROLL>
void launch_block_copy_nt(const BlockCopyArgs<IdT>& a, uint32_t grid, int nt, uint32_t lds, hipStream_t s) {
    switch (nt & 3) {
        case 0: launch_block_copy_one<ROLE, IdT, UNROLL, 0>(a, grid, lds, s); break;
        case 1: launch_block_copy_one<ROLE, IdT, UNROLL, 1>(a, grid, lds, s); break;
        case 2: launch_block_copy_one<ROLE, IdT, UNROLL, 2>(a, grid, lds, s); break;
        default: launch_block_copy_one<ROLE, IdT, UNROLL, 3>(a, grid, lds, s); break;
    }
}

template <Role ROLE, typename IdT>
int launch_block_copy(BlockCopyArgs<IdT> a, uint32_t workgroups, hipStream_t s, int preferred_unroll = 0,
                      uint32_t pace_mbps = 0, bool plain_stores = false, bool pace_between_launches = false) {
    int unroll = 1;
    if (preferred_unroll == 0) preferred_unroll = (int)knob_value(HFK_KNOB_UNROLL);
    // Everything but the swap runs one workgroup per chunk and wants whole chunks.
    int rc = hfk::plan_block_copy<IdT>(a, preferred_unroll, &unroll, ROLE != Role::kSwapBlocks);
    if (rc != 0) return rc;
    uint32_t grid = 0;
    rc = pick_grid(a.n_work, workgroups, &grid);
    if (rc != 0) return rc;
    if (pace_mbps != 0) {
        // bytes per work item (average over a block) * workgroups / rate
        a.pace_q8 = pace_interval_q8((double)a.block_bytes / a.chunks_per_block, grid, pace_mbps);
        a.pace_report = reinterpret_cast<uint64_t*>((uintptr_t)knob_value(HFK_KNOB_PACE_REPORT));
        if (pace_between_launches) {
            rc = pace_state(&a.pace_state);
            if (rc != 0) return rc;
        }
    }
    const int nt = (int)knob_value(HFK_KNOB_NONTEMPORAL) & (plain_stores ? 1 : 3);
    // HBM-bound launches may ask for LDS they never touch: it bounds how many workgroups a compute
    // unit holds at a time (HFK_KNOB_HBM_LDS_BYTES).
    const uint32_t lds = ROLE == Role::kSwapBlocks ? 0u : (uint32_t)knob_value(HFK_KNOB_HBM_LDS_BYTES);
    switch (unroll) {
        case 1: launch_block_copy_nt<ROLE, IdT, 1>(a, grid, nt, lds, s); break;
        case 2: launch_block_copy_nt<ROLE, IdT, 2>(a, grid, nt, lds, s); break;
        case 4: launch_block_copy_nt<ROLE, IdT, 4>(a, grid, nt, lds, s); break;
        case 8: launch_block_copy_nt<ROLE, IdT, 8>(a, grid, nt, lds, s); break;
        default: launch_block_copy_nt<ROLE, IdT, 16>(a, grid, nt, lds, s); break;
    }
    return finish_launch();
}

template <int UNROLL>
void launch_duplex_nt(const DuplexCopyArgs& a, uint32_t grid, int nt, hipStream_t s) {
    if (nt & 3) hipLaunchKernelGGL((swap_blocks_duplex_kernel<UNROLL, 3>), dim3(grid), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((swap_blocks_duplex_kernel<UNROLL, 0>), dim3(grid), dim3(256), 0, s, a);
}

// ---- flat gather ----------------------------------------------------------
template <typename V, typename IdT, typename IndexT, int UNROLL>
void launch_flat_gather_u(const FlatGatherArgs<IdT>& a, uint32_t grid, int nt, hipStream_t s) {
    if (nt & 3) {
        hipLaunchKernelGGL((flat_gather_kernel<V, IdT, IndexT, UNROLL, 3>), dim3(grid), dim3(256), 0, s, a);
    } else {
        hipLaunchKernelGGL((flat_gather_kernel<V, IdT, IndexT, UNROLL, 0>), dim3(grid), dim3(256), 0, s, a);
    }
}

template <typename V, typename IdT, typename IndexT>
void launch_flat_gather_v(const FlatGatherArgs<IdT>& a, uint32_t grid, int nt, int unroll, hipStream_t s) {
    if (unroll == hfk::kFlatUnrollHost) launch_flat_gather_u<V, IdT, IndexT, hfk::kFlatUnrollHost>(a, grid, nt, s);
    else launch_flat_gather_u<V, IdT, IndexT, hfk::kFlatUnrollDevice>(a, grid, nt, s);
}

template <typename IdT>
int launch_flat_gather(uint64_t table, uint64_t dst, const IdT* ids, uint64_t n_ids, uint64_t row_bytes,
                       uint64_t row_limit, uint32_t workgroups, bool table_in_host, hipStream_t s) {
    FlatGatherArgs<IdT> a;
    hfk::FlatGatherPlan p;
    const int unroll = table_in_host ? hfk::kFlatUnrollHost : hfk::kFlatUnrollDevice;
    int rc = hfk::plan_flat_gather<IdT>(a, p, table, dst, ids, n_ids, row_bytes, row_limit, unroll);
    if (rc != 0) return rc;
    uint32_t grid = 0;
    rc = pick_grid(a.n_work, workgroups, &grid);
    if (rc != 0) return rc;
    const int nt = (int)knob_value(HFK_KNOB_NONTEMPORAL);
    if (p.unit == 16u) {
        if (p.index32) launch_flat_gather_v<vec16, IdT, uint32_t>(a, grid, nt, unroll, s);
        else launch_flat_gather_v<vec16, IdT, uint64_t>(a, grid, nt, unroll, s);
    } else if (p.unit == 4u) {
        if (p.index32) launch_flat_gather_v<uint32_t, IdT, uint32_t>(a, grid, nt, unroll, s);
        else launch_flat_gather_v<uint32_t, IdT, uint64_t>(a, grid, nt, unroll, s);
    } else {
        if (p.index32) launch_flat_gather_v<uint8_t, IdT, uint32_t>(a, grid, nt, unroll, s);
        else launch_flat_gather_v<uint8_t, IdT, uint64_t>(a, grid, nt, unroll, s);
    }
    return finish_launch();
}

template <typename IdT>
int gather_rows_typed(const void* table, void* dst, const IdT* ids, uint64_t n_ids, uint64_t row_bytes,
                      uint64_t table_rows, uint32_t workgroups, bool table_in_host, hipStream_t s) {
    const uint64_t limit = table_rows ? table_rows : hfk::kUnchecked;
    if (row_bytes >= hfk::kWideRowBytes) {
        BlockCopyArgs<IdT> a;
        int rc = hfk::plan_wide_gather<IdT>(a, table, dst, ids, n_ids, row_bytes, limit);
        if (rc != 0) return rc;
        return launch_block_copy<Role::kGatherRows, IdT>(a, workgroups, s);
    }
    return launch_flat_gather<IdT>((uint64_t)(uintptr_t)table, (uint64_t)(uintptr_t)dst, ids, n_ids, row_bytes,
                                   limit, workgroups, table_in_host, s);
}

// ---- transpose ------------------------------------------------------------
template <typename V, int U, int NT>
void launch_transpose_nt(const TransposeArgs& a, uint32_t grid, bool to_packed, hipStream_t s) {
    if (to_packed) {
        hipLaunchKernelGGL((transpose_to_packed_kernel<V, U, NT>), dim3(grid), dim3(256), 0, s, a);
    } else if (a.mirror != 0) {
        if constexpr (U == hfk::kTransposeUnroll) {   // the one shape the staged op launches
            hipLaunchKernelGGL((transpose_and_stage_kernel<V, U, NT>), dim3(grid), dim3(256), 0, s, a);
        }
    } else {
        hipLaunchKernelGGL((transpose_kernel<V, U, NT>), dim3(grid), dim3(256), 0, s, a);
    }
}

template <typename V, int U>
void launch_transpose_u(const TransposeArgs& a, uint32_t grid, int nt, bool to_packed, hipStream_t s) {
    switch (nt & 3) {
        case 0: launch_transpose_nt<V, U, 0>(a, grid, to_packed, s); break;
        case 1: launch_transpose_nt<V, U, 1>(a, grid, to_packed, s); break;
        case 2: launch_transpose_nt<V, U, 2>(a, grid, to_packed, s); break;
        default: launch_transpose_nt<V, U, 3>(a, grid, to_packed, s); break;
    }
}

template <typename V>
void launch_transpose_v(const TransposeArgs& a, uint32_t grid, int nt, bool to_packed, int unroll, hipStream_t s) {
    switch (unroll) {
        case hfk::kTransposeUnroll: launch_transpose_u<V, hfk::kTransposeUnroll>(a, grid, nt, to_packed, s); break;
        default: launch_transpose_u<V, hfk::kTransposeUnrollToHost>(a, grid, nt, to_packed, s); break;
    }
}
// The tiled kernel stores plainly (through the L2, which hands the link whole lines); `nt_loads` picks its loads.
template <int U>
void launch_transpose_tiled_u(const TransposeArgs& a, uint32_t grid, bool nt_loads, hipStream_t s) {
    if (nt_loads) hipLaunchKernelGGL((transpose_to_packed_tiled_kernel<U, 1>), dim3(grid), dim3(256), 0, s, a);
    else hipLaunchKernelGGL((transpose_to_packed_tiled_kernel<U, 0>), dim3(grid), dim3(256), 0, s, a);
}

void launch_transpose_tiled(const TransposeArgs& a, uint32_t grid, bool nt_loads, int U, hipStream_t s) {
    switch (U) {
        case 8: launch_transpose_tiled_u<8>(a, grid, nt_loads, s); break;
        case 4: launch_transpose_tiled_u<4>(a, grid, nt_loads, s); break;
        case 2: launch_transpose_tiled_u<2>(a, grid, nt_loads, s); break;
        default: launch_transpose_tiled_u<1>(a, grid, nt_loads, s); break;
    }
}

// Where an address lives: 1 = host memory (pinned, device-mapped), 0 = device memory, -1 = the
// runtime does not know the pointer.
int memory_side(const void* p) {
    hipPointerAttribute_t attr;
    if (hipPointerGetAttributes(&attr, p) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
    if (attr.type == hipMemoryTypeHost) return 1;
    if (attr.type == hipMemoryTypeDevice) return 0;
    return -1;
}

// A transfer toward the host that is over in a millisecond wants to be over sooner rather than gentler.
uint32_t transfer_to_host_workgroups(uint64_t bytes) {
    return bytes < kShorterTransferBytes ? kShorterTransferToHostWorkgroups
           : bytes < kShortTransferBytes ? kShortTransferToHostWorkgroups
                                         : kTransferToHostWorkgroups;
}

// `packed_side` is what the caller knows about the packed pool (1 host memory, 0 device memory);
// kAskRuntime: the runtime is asked where it lives.
constexpr int kAskRuntime = -2;
int launch_transpose(const void* dev_layer_ptrs, const void* packed, const int64_t* pairs, uint64_t n_pairs,
                     uint64_t packed_stride, uint64_t layered_stride, uint64_t packed_blocks,
                     uint64_t layered_blocks, uint32_t T, uint32_t L, uint32_t H, uint32_t D, uint32_t elem_bytes,
                     bool to_packed, int packed_side, uint32_t workgroups, hipStream_t s,
                     bool beside_compute = false, void* mirror = nullptr) {
    if (dev_layer_ptrs == nullptr || packed == nullptr) return HFK_ERR_NULL_POINTER;
    if (mirror != nullptr && to_packed) return HFK_ERR_BAD_FLAGS;
    // With the packed side in host memory the PCIe link is the bound and a small grid does; an
    // unknown pointer gets the small grid too. Measured on the reference's four shapes, 8 blocks per
    // launch: host -> device (two units per lane) 56.0-57.0 GB/s on 16 workgroups, 57.1-57.6 on 24-36,
    // 54.1-54.6 on 48-56 (a dip that repeats), 56.6-57.5 on 80-96.
    // Device -> host, row by row (eight units per lane): 53.2-54.0 GB/s on 32 or more workgroups,
    // whatever the store kind, against 55.3-56.9 when the rows are 256 bytes or longer: a wavefront
    // load that fetches eight 128-byte rows from eight places makes the same kernel 2-3 GB/s slower
    // on the link, although HBM serves either pattern five times faster than the link drains it (the
    // link then takes 2 % more 64-byte write requests than the payload has lines, against 1.4 %; no
    // difference in address translation: 0.05 % of the lookups miss either way). Through LDS tiles
    // (1 KiB runs on both sides) with plain stores: 56.5-56.6 GB/s on 32 workgroups for transfers of
    // 256 MiB and more (55.4 with non-temporal stores, 56.1 on 64 workgroups); short transfers want
    // more workgroups to be over sooner (32 MiB: 54.2 on 32, 55.3 on 64, 55.8 on 128; 64 MiB: 55.4, 55.6, 55.6).
    // Pacing does not pay: at 0.895 of the link 55.3-55.9 on the long shapes and 50-52 on the short.
    const int side = packed_side == kAskRuntime ? memory_side(packed) : packed_side;
    const int unroll = to_packed && side != 0 ? (int)knob_value(HFK_KNOB_TRANSFER_UNROLL) : hfk::kTransposeUnroll;
    TransposeArgs a;
    uint32_t unit = 16;
    int rc = hfk::plan_transpose(a, &unit, dev_layer_ptrs, packed, pairs, n_pairs, packed_stride, layered_stride,
                                 packed_blocks, layered_blocks, T, L, H, D, elem_bytes, unroll, mirror);
    if (rc != 0) return rc;
    if (a.n_work == 0) return HFK_OK;  // nothing to move
    int tiled_unroll = 0;
    if (to_packed && side != 0 && knob_value(HFK_KNOB_TRANSFER_TILED) != 0) {
        tiled_unroll = hfk::plan_transpose_tiles(a, unit, kLayerTableLdsEntries);
    }
    if (workgroups == 0 && side != 0) {
        // One block (the reference's op: 4-64 MiB, over in 0.1-1.2 ms) is sized for speed alone; a
        // block table may run for many milliseconds beside other kernels and gets the smaller grid.
        workgroups = pairs == nullptr ? (mirror != nullptr ? kSingleBlockStagedTransferWorkgroups : kSingleBlockTransferWorkgroups)
                     : beside_compute ? kBesideTransferWorkgroups
                     : to_packed      ? transfer_to_host_workgroups((uint64_t)a.total_units * unit * n_pairs)
                                      : kTransferFromHostWorkgroups;
    }
    uint32_t grid = 0;
    rc = pick_grid(a.n_work, workgroups, &grid);
    if (rc != 0) return rc;
    if (to_packed && side != 0 && knob_value(HFK_KNOB_TRANSFER_PACE_PERMILLE) != 0) {
        const uint32_t pace_mbps = (uint32_t)(knob_value(HFK_KNOB_TRANSFER_PACE_PERMILLE) / 1000.0 * current_link_mbps());
        if (pace_mbps != 0) a.pace_q8 = pace_interval_q8((double)a.total_units * unit / a.chunks_per_block, grid, pace_mbps);
    }
    const int nt = (int)knob_value(HFK_KNOB_NONTEMPORAL);
    if (tiled_unroll != 0) launch_transpose_tiled(a, grid, (nt & 1) != 0, tiled_unroll, s);
    else if (unit == 16u) launch_transpose_v<vec16>(a, grid, nt, to_packed, unroll, s);
    else if (unit == 4u) launch_transpose_v<uint32_t>(a, grid, nt, to_packed, unroll, s);
    else launch_transpose_v<uint8_t>(a, grid, nt, to_packed, unroll, s);
    return finish_launch();
}

// Launch shape of a block-table swap, from what the caller says about it (`flags`) and how many bytes
// it moves (`bytes`; for a table split by run length, the share this launch moves).
constexpr uint32_t kSwapFlagMask = HFK_SWAP_DST_HOST | HFK_SWAP_SRC_HOST | HFK_SWAP_BESIDE_COMPUTE;

int launch_swap(const BlockCopyArgs<int64_t>& a, uint32_t flags, uint32_t workgroups, uint64_t bytes, hipStream_t s) {
    // Toward the host the link accepts the most when it is offered what it can take (offering 1.5-2x
    // its rate lowers what it accepts to 47-49 GB/s). A swap that shares the GPU is paced at 0.84 of the
    // raw rate; one that owns it runs unpaced on the shape that offers just enough (hfk::to_host_shape)
    // unless pacing is switched on for it; should the link's rate be unknown a paced launch degrades
    // to an unpaced one. A paced launch starts its workgroups staggered over one interval and ends
    // behind its schedule, and the plain stores of the long unpaced shape only pay once the launch
    // lasts (2 MiB: 50.5 us on 16 x 8 with non-temporal stores, 53.9 on 12 x 8 with plain ones; 32 MiB:
    // 619 against 624 us; from 64 MiB on the plain-store shape wins, 256 MiB: 4816 against 4767 us), so
    // a short throughput-mode swap runs as one about which nothing is known: the shape that saturates
    // the link either way (16 workgroups x 8 vectors per lane: 55.4-56.0 GB/s out, 57.0-57.4 in).
    // Without a usable pace (no host side named, or the link's rate unknown) a beside-compute swap gets
    // a small unpaced grid (49.8 GB/s toward the host).
    const bool wants_pace = (flags & HFK_SWAP_DST_HOST) != 0;
    const hfk::SwapTuning tuning{(uint32_t)knob_value(HFK_KNOB_SWAP_WORKGROUPS),
                                 (int)knob_value(HFK_KNOB_SWAP_UNROLL),
                                 (uint32_t)knob_value(HFK_KNOB_PACED_WORKGROUPS),
                                 (int)knob_value(HFK_KNOB_PACED_UNROLL),
                                 (uint32_t)knob_value(HFK_KNOB_THROUGHPUT_PACE_PERMILLE),
                                 (uint32_t)knob_value(HFK_KNOB_SWAP_PACE_MBPS)};
    const hfk::SwapShape shape =
        hfk::choose_swap_shape(flags, bytes, a.block_bytes, wants_pace ? (uint32_t)current_link_mbps() : 0u, workgroups, tuning);
    // A paced throughput-mode swap lets the launches before it set its pace (hfk::pace_factor); the beside-compute
    // pace is meant to stay well under the link's limit and stays fixed.
    const bool between = shape.pace_mbps != 0 && (flags & HFK_SWAP_BESIDE_COMPUTE) == 0 &&
                         knob_value(HFK_KNOB_ADAPTIVE_PACE) != 0;
    return launch_block_copy<Role::kSwapBlocks, int64_t>(a, shape.workgroups, s, shape.unroll, shape.pace_mbps,
                                                         shape.plain_stores, between);
}

// ---- staged swap: HBM-only kernel + DMA copies ----------------------------
// What the PCIe leg of a staged (or split) swap needs to know.
struct HostLeg {
    void* const* host_plane_addrs;   // host array of n_planes host addresses
    const int64_t* host_block_ids;   // host array of n_blocks slots
    uint32_t n_planes;
    uint64_t n_blocks;
    uint64_t block_bytes;
    uint64_t host_block_stride;
    void* staging;                   // [n_planes][n_blocks][block_bytes] in device memory, or, when compact,
    bool to_host;
    bool compact = false;            // [n_planes][stage_plane_blocks][block_bytes]: the long runs only, in table order
    uint64_t stage_plane_blocks = 0;
};

int check_host_leg(const HostLeg& h, uint64_t host_blocks) {
    if (h.host_plane_addrs == nullptr || h.host_block_ids == nullptr) return HFK_ERR_NULL_POINTER;
    if (h.host_block_stride < h.block_bytes) return HFK_ERR_BAD_SIZE;
    for (uint32_t p = 0; p < h.n_planes; ++p) {
        if (h.host_plane_addrs[p] == nullptr) return HFK_ERR_NULL_POINTER;
    }
    for (uint64_t i = 0; i < h.n_blocks; ++i) {  // nothing is enqueued unless every host slot is valid
        if (h.host_block_ids[i] < 0 || (host_blocks != 0 && (uint64_t)h.host_block_ids[i] >= host_blocks)) {
            return HFK_ERR_OUT_OF_RANGE;
        }
    }
    return HFK_OK;
}

// The PCIe leg: one copy per run of at least `min_run` consecutive host slots. A run of k slots is
// k * block_bytes contiguous bytes in every plane. Planes that are evenly spaced on the host (a
// pool [planes][blocks][...], the usual case) are moved together by ONE 2-D copy per run (rows =
// planes), which the DMA engines execute at their full rate (57 GB/s measured, against 53 for one
// copy per plane); a plane that does not line up gets its own copy. Host blocks with a padded
// stride use a 2-D copy per plane (rows = blocks). All copies go to `s`: dealing the runs to two
// streams gains nothing (same-direction copies are executed one after the other: 45.1 GB/s either
// way for 111 runs of 2-14 MiB; a copy costs its engine about 9.5 us before the first byte moves).
int copy_host_runs(const HostLeg& h, uint64_t min_run, hipStream_t s) {
    const uint64_t stage_pitch = (h.compact ? h.stage_plane_blocks : h.n_blocks) * h.block_bytes;
    uint64_t staged_before = 0;      // pairs in long runs before the current run (compact staging: its first slot)
    hipError_t e = hipSuccess;
    // Copies `run_bytes` at host_off / stage_off for planes [p0, p0 + count), which are evenly spaced
    // by `pitch` bytes on the host (count == 1: a plain copy).
    auto copy_plane_group = [&](uint32_t p0, uint32_t count, int64_t pitch, uint64_t host_off, uint64_t stage_off,
                                uint64_t run_bytes) -> hipError_t {
        hipStream_t cs = s;
        char* hp = static_cast<char*>(h.host_plane_addrs[p0]) + host_off;
        char* d = static_cast<char*>(h.staging) + (uint64_t)p0 * stage_pitch + stage_off;
        if (count == 1) {
            return h.to_host ? hipMemcpyAsync(hp, d, run_bytes, hipMemcpyDeviceToHost, cs)
                             : hipMemcpyAsync(d, hp, run_bytes, hipMemcpyHostToDevice, cs);
        }
        return h.to_host
                   ? hipMemcpy2DAsync(hp, (size_t)pitch, d, stage_pitch, run_bytes, count, hipMemcpyDeviceToHost, cs)
                   : hipMemcpy2DAsync(d, stage_pitch, hp, (size_t)pitch, run_bytes, count, hipMemcpyHostToDevice, cs);
    };
    hfk::for_each_host_run(h.host_block_ids, h.n_blocks, [&](uint64_t first, uint64_t len) {
        if (len < min_run || e != hipSuccess) return;
        hipStream_t cs = s;
        const uint64_t host_off = (uint64_t)h.host_block_ids[first] * h.host_block_stride;
        const uint64_t stage_off = (h.compact ? staged_before : first) * h.block_bytes;
        staged_before += len;
        const uint64_t run_bytes = len * h.block_bytes;
        if (h.host_block_stride == h.block_bytes) {
            // maximal groups of evenly spaced planes: one 2-D copy each
            uint32_t p0 = 0;
            while (p0 < h.n_planes && e == hipSuccess) {
                uint32_t count = 1;
                int64_t pitch = 0;
                if (p0 + 1 < h.n_planes) {
                    pitch = static_cast<char*>(h.host_plane_addrs[p0 + 1]) - static_cast<char*>(h.host_plane_addrs[p0]);
                    if (pitch >= (int64_t)run_bytes) {
                        count = 2;
                        while (p0 + count < h.n_planes &&
                               static_cast<char*>(h.host_plane_addrs[p0 + count]) -
                                       static_cast<char*>(h.host_plane_addrs[p0 + count - 1]) == pitch) {
                            ++count;
                        }
                    }
                }
                e = copy_plane_group(p0, count, pitch, host_off, stage_off, run_bytes);
                p0 += count;
            }
        } else {
            for (uint32_t p = 0; p < h.n_planes && e == hipSuccess; ++p) {
                char* hp = static_cast<char*>(h.host_plane_addrs[p]) + host_off;
                char* d = static_cast<char*>(h.staging) + (uint64_t)p * stage_pitch + stage_off;
                e = h.to_host ? hipMemcpy2DAsync(hp, h.host_block_stride, d, h.block_bytes, h.block_bytes, len,
                                                 hipMemcpyDeviceToHost, cs)
                              : hipMemcpy2DAsync(d, h.block_bytes, hp, h.host_block_stride, h.block_bytes, len,
                                                 hipMemcpyHostToDevice, cs);
            }
        }
    });
    return e == hipSuccess ? HFK_OK : (int)e;
}

int staged_swap(const void* dev_plane_ptrs, void* const* host_plane_addrs, const int64_t* dev_block_ids,
                const int64_t* host_block_ids, uint32_t n_planes, uint64_t n_blocks, uint64_t block_bytes,
                uint64_t dev_block_stride, uint64_t host_block_stride, uint64_t dev_blocks, uint64_t host_blocks,
                void* staging, int to_host, uint32_t workgroups, hipStream_t s) {
    const HostLeg leg{host_plane_addrs, host_block_ids, n_planes, n_blocks, block_bytes, host_block_stride, staging,
                      to_host != 0};
    BlockCopyArgs<int64_t> a;
    int rc = hfk::plan_stage_blocks(a, dev_plane_ptrs, staging, dev_block_ids, n_planes, n_blocks, block_bytes,
                                    dev_block_stride, dev_blocks, to_host != 0);
    if (rc != 0) return rc;
    rc = check_host_leg(leg, host_blocks);
    if (rc != 0) return rc;
    if (to_host) {
        rc = launch_block_copy<Role::kGatherBlocks, int64_t>(a, workgroups, s);
        if (rc != 0) return rc;
        return copy_host_runs(leg, 1, s);
    }
    rc = copy_host_runs(leg, 1, s);
    if (rc != 0) return rc;
    return launch_block_copy<Role::kScatterBlocks, int64_t>(a, workgroups, s);
}

// ---- staging owned by the library, for callers that may not allocate ------
// One array per device the library is loaded on, held until the process ends. In host code the
// array's name stands for the symbol, not for device memory: the address kernels and copies use
// is asked of the runtime once per device and kept.
constexpr uint64_t kStaticStagingBytes = HFK_STATIC_STAGING_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticStagingBytes];
std::atomic<void*> g_scratch_ptr[kMaxDevices];

int static_staging(void** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return HFK_ERR_TOO_LARGE;
    void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        // `dev` is current: the address returned is that of this device's copy of the array.
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (ptr == nullptr) return (int)hipErrorInvalidSymbol;
        g_scratch_ptr[dev].store(ptr, std::memory_order_release);   // racing threads store the same address
    }
    *out = ptr;
    return HFK_OK;
}

// Every static call on a device shares that device's array, and two that overlap in time corrupt each
// other's blocks without either noticing. Calls on one stream are ordered by the stream. For calls on
// different streams the library remembers, per device, the stream of the last static call and an event
// recorded behind it: a call that arrives on another stream while that event is still pending is
// refused (HFK_ERR_STAGING_BUSY) instead of racing. A stream under capture is left alone (an event
// recorded there belongs to the graph): callers that replay graphs order them themselves.
struct StaticUse {
    std::mutex lock;
    hipEvent_t done = nullptr;     // created on the device's first static call, never destroyed
    hipStream_t last_stream = nullptr;
    bool pending = false;          // `done` was recorded and not yet seen complete
};
StaticUse g_static_use[kMaxDevices];

// Before a static call enqueues anything. `*guarded` tells static_release whether to record.
int static_acquire(hipStream_t s, int* dev_out, bool* guarded) {
    *guarded = false;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return HFK_ERR_TOO_LARGE;
    *dev_out = dev;
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(s, &capture) != hipSuccess) {
        (void)hipGetLastError();
        return HFK_OK;
    }
    if (capture != hipStreamCaptureStatusNone) return HFK_OK;
    StaticUse& u = g_static_use[dev];
    std::lock_guard<std::mutex> hold(u.lock);
    if (u.done == nullptr) {
        e = hipEventCreateWithFlags(&u.done, hipEventDisableTiming);
        if (e != hipSuccess) return (int)e;
    }
    if (u.pending && u.last_stream != s) {
        e = hipEventQuery(u.done);
        if (e == hipErrorNotReady) {
            (void)hipGetLastError();
            return HFK_ERR_STAGING_BUSY;
        }
        if (e != hipSuccess) return (int)e;
        u.pending = false;
    }
    *guarded = true;
    return HFK_OK;
}

void static_release(hipStream_t s, int dev, bool guarded) {
    if (!guarded) return;
    StaticUse& u = g_static_use[dev];
    std::lock_guard<std::mutex> hold(u.lock);
    if (hipEventRecord(u.done, s) == hipSuccess) {
        u.last_stream = s;
        u.pending = true;
    } else {
        (void)hipGetLastError();
    }
}

// A run of host slots is worth a DMA copy when one copy of it moves at least this much.
constexpr uint64_t kDmaRunBytes = 16ull << 20;
constexpr uint64_t kDmaRunBytesBesideCompute = 4ull << 20;
// Longest run threshold the kernels' run filter is asked to evaluate (it reads up to twice as many
// table entries per pair); a larger threshold means "never stage".
constexpr uint64_t kMaxRunFilter = 1024;

// Number of leading planes that one 2-D copy covers (planes evenly spaced on the host).
uint64_t evenly_spaced_planes(const HostLeg& h) {
    if (h.n_planes < 2) return 1;
    const int64_t pitch = static_cast<char*>(h.host_plane_addrs[1]) - static_cast<char*>(h.host_plane_addrs[0]);
    if (pitch < (int64_t)h.block_bytes) return 1;
    uint64_t count = 2;
    while (count < h.n_planes && static_cast<char*>(h.host_plane_addrs[count]) -
                                         static_cast<char*>(h.host_plane_addrs[count - 1]) == pitch) {
        ++count;
    }
    return count;
}

}  // namespace

extern "C" {

int hfk_version(void) { return HFK_VERSION_MAJOR * 1000 + HFK_VERSION_MINOR; }

const char* hfk_status_string(int status) {
    switch (status) {
        case HFK_OK: return "ok";
        case HFK_ERR_NULL_POINTER: return "hfk: required pointer argument is NULL";
        case HFK_ERR_BAD_SIZE: return "hfk: size or stride is zero or inconsistent";
        case HFK_ERR_TOO_LARGE: return "hfk: count exceeds what one launch can index";
        case HFK_ERR_BAD_KNOB: return "hfk: unknown tuning knob or value out of range";
        case HFK_ERR_OUT_OF_RANGE: return "hfk: host-side index outside the declared range";
        case HFK_ERR_BAD_FLAGS: return "hfk: unknown flag bits";
        case HFK_ERR_STAGING_TOO_SMALL:
            return "hfk: transfer exceeds the library's static staging buffer (HFK_STATIC_STAGING_BYTES)";
        case HFK_ERR_STAGING_BUSY:
            return "hfk: the library's static staging buffer is still in use by a call on another stream";
        case HFK_ERR_TABLE_MISMATCH: return "hfk: host_block_ids differs from the host column of block_pairs";
        default: break;
    }
    if (status > 0) return hipGetErrorString((hipError_t)status);
    return "hfk: unknown status";
}

int hfk_gather_rows(const void* table, void* dst, const void* ids, int ids_are_i64, uint64_t n_ids,
                    uint64_t row_bytes, uint64_t table_rows, uint32_t flags, uint32_t workgroups,
                    hfk_stream_t stream) {
    if (flags != 0 && flags != HFK_SWAP_SRC_HOST && flags != HFK_SWAP_SRC_DEVICE) return HFK_ERR_BAD_FLAGS;
    if (n_ids == 0) return HFK_OK;
    if (table == nullptr || dst == nullptr || ids == nullptr) return HFK_ERR_NULL_POINTER;
    if (row_bytes == 0) return HFK_ERR_BAD_SIZE;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // Where the table lives shapes the launch. A caller that does not say is answered by the runtime,
    // which takes about 5 us of the calling thread, so it is asked only when the answer can matter
    // (a gather of less than 64 KiB is over before either shape could differ).
    const bool table_in_host = flags == HFK_SWAP_SRC_HOST ||
                               (flags == 0 && n_ids * row_bytes >= kAskTableSideBytes && memory_side(table) == 1);
    if (workgroups == 0 && table_in_host && n_ids * row_bytes > kLongHostGatherBytes) {
        // A table in host memory (the reference's embedding case) is read over the PCIe link: 64
        // workgroups already run it at the link's rate (55-57 GB/s for 1 KiB rows), and every further
        // one only slows kernels on other streams. Gathers of a few MiB keep one workgroup per chunk
        // (they are over in tens of microseconds and a cap would only add a partly filled second round).
        workgroups = kHostGatherWorkgroups;
    }
    if (ids_are_i64) {
        return gather_rows_typed<int64_t>(table, dst, static_cast<const int64_t*>(ids), n_ids, row_bytes,
                                          table_rows, workgroups, table_in_host, s);
    }
    return gather_rows_typed<int32_t>(table, dst, static_cast<const int32_t*>(ids), n_ids, row_bytes,
                                      table_rows, workgroups, table_in_host, s);
}

int hfk_multi_layer_block_transfer(const void* dev_layer_ptrs, const void* src_block, uint32_t T,
                                   uint32_t L, uint32_t H, uint32_t D, uint32_t elem_bytes, uint32_t flags,
                                   uint32_t workgroups, hfk_stream_t stream) {
    if (flags != 0 && flags != HFK_SWAP_SRC_HOST && flags != HFK_SWAP_SRC_DEVICE) return HFK_ERR_BAD_FLAGS;
    const int side = flags == HFK_SWAP_SRC_HOST ? 1 : flags == HFK_SWAP_SRC_DEVICE ? 0 : kAskRuntime;
    return launch_transpose(dev_layer_ptrs, src_block, nullptr, 1, 0, 0, 0, 0, T, L, H, D, elem_bytes, false, side,
                            workgroups, static_cast<hipStream_t>(stream));
}

int hfk_fused_memcpy_multi_layer_block_transfer(const void* dev_layer_ptrs, const void* host_block,
                                                void* staging, uint32_t T, uint32_t L, uint32_t H,
                                                uint32_t D, uint32_t elem_bytes, uint32_t workgroups,
                                                hfk_stream_t stream) {
    if (dev_layer_ptrs == nullptr || host_block == nullptr || staging == nullptr) return HFK_ERR_NULL_POINTER;
    if (elem_bytes == 0) return HFK_ERR_BAD_SIZE;
    const uint64_t bytes = (uint64_t)T * L * H * D * elem_bytes;
    if (bytes == 0) return HFK_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    // A block in pinned, device-mapped host memory is read over the link once, by the kernel of the direct
    // transfer, which writes every unit to its layer and to the staging buffer as well: the staging copy costs
    // HBM writes the link-bound kernel has room for, and the call takes what the direct transfer takes (4 MiB:
    // 80 us) instead of a copy and then a kernel (93 us: a block this short costs the copy engines 10 us before
    // its first byte). A block the device cannot address (pageable memory), or HFK_KNOB_FUSED_COPY_ENGINE, takes
    // the copy and the kernel.
    if (knob_value(HFK_KNOB_FUSED_COPY_ENGINE) == 0) {
        void* mapped = nullptr;
        if (hipHostGetDevicePointer(&mapped, const_cast<void*>(host_block), 0) == hipSuccess && mapped != nullptr) {
            return launch_transpose(dev_layer_ptrs, mapped, nullptr, 1, 0, 0, 0, 0, T, L, H, D, elem_bytes, false, 1,
                                    workgroups, s, false, staging);
        }
        (void)hipGetLastError();
    }
    hipError_t e = hipMemcpyAsync(staging, host_block, bytes, hipMemcpyHostToDevice, s);
    if (e != hipSuccess) return (int)e;
    return launch_transpose(dev_layer_ptrs, staging, nullptr, 1, 0, 0, 0, 0, T, L, H, D, elem_bytes, false, 0,
                            workgroups, s);
}

int hfk_multi_layer_block_table_transfer(const void* dev_layer_ptrs, uint64_t dev_block_stride,
                                         void* packed_blocks, uint64_t packed_block_stride,
                                         const int64_t* block_pairs, uint64_t n_pairs, uint64_t n_packed_blocks,
                                         uint64_t n_dev_blocks, uint32_t T, uint32_t L, uint32_t H, uint32_t D,
                                         uint32_t elem_bytes, int to_packed, uint32_t flags, uint32_t workgroups,
                                         hfk_stream_t stream) {
    // What the caller says about the packed pool: the source on the way to the device, the destination back.
    const uint32_t host_flag = to_packed ? HFK_SWAP_DST_HOST : HFK_SWAP_SRC_HOST;
    const uint32_t device_flag = to_packed ? HFK_SWAP_DST_DEVICE : HFK_SWAP_SRC_DEVICE;
    if ((flags & ~(HFK_SWAP_BESIDE_COMPUTE | host_flag | device_flag)) != 0) return HFK_ERR_BAD_FLAGS;
    if ((flags & host_flag) != 0 && (flags & device_flag) != 0) return HFK_ERR_BAD_FLAGS;
    if (n_pairs == 0) return HFK_OK;
    if (block_pairs == nullptr) return HFK_ERR_NULL_POINTER;
    const int side = (flags & host_flag) != 0 ? 1 : (flags & device_flag) != 0 ? 0 : kAskRuntime;
    return launch_transpose(dev_layer_ptrs, packed_blocks, block_pairs, n_pairs, packed_block_stride,
                            dev_block_stride, n_packed_blocks, n_dev_blocks, T, L, H, D, elem_bytes, to_packed != 0,
                            side, workgroups, static_cast<hipStream_t>(stream), (flags & HFK_SWAP_BESIDE_COMPUTE) != 0);
}

int hfk_swap_blocks(const void* dst_plane_ptrs, const void* src_plane_ptrs, const int64_t* block_pairs,
                    uint32_t n_planes, uint64_t n_pairs, uint64_t block_bytes, uint64_t src_block_stride,
                    uint64_t dst_block_stride, uint64_t src_blocks, uint64_t dst_blocks, uint32_t flags,
                    uint32_t workgroups, hfk_stream_t stream) {
    if ((flags & ~kSwapFlagMask) != 0) return HFK_ERR_BAD_FLAGS;
    if (n_planes == 0 || n_pairs == 0) return HFK_OK;
    BlockCopyArgs<int64_t> a;
    int rc = hfk::plan_swap_blocks(a, dst_plane_ptrs, src_plane_ptrs, block_pairs, n_planes, n_pairs, block_bytes,
                                   src_block_stride, dst_block_stride, src_blocks, dst_blocks);
    if (rc != 0) return rc;
    return launch_swap(a, flags, workgroups, (uint64_t)n_planes * n_pairs * block_bytes,
                       static_cast<hipStream_t>(stream));
}

int hfk_swap_blocks_duplex(const hfk_block_move* out_move, const hfk_block_move* in_move, uint32_t n_planes,
                           uint64_t block_bytes, uint32_t flags, uint32_t workgroups, hfk_stream_t stream) {
    if ((flags & ~(uint32_t)HFK_SWAP_BESIDE_COMPUTE) != 0) return HFK_ERR_BAD_FLAGS;
    DuplexCopyArgs a;
    int unroll = 1;
    if (block_bytes == 0) return HFK_ERR_BAD_SIZE;
    const bool beside = (flags & HFK_SWAP_BESIDE_COMPUTE) != 0;
    // Beside compute: half the workgroups, two vectors per lane and direction, paced (97-98 GB/s summed
    // on 16 workgroups where one vector per lane leaves them latency-bound at 64).
    int rc = hfk::plan_duplex(a, out_move, in_move, n_planes, block_bytes,
                              beside ? kBesideDuplexUnroll : (int)knob_value(HFK_KNOB_DUPLEX_UNROLL), &unroll);
    if (rc != 0) return rc;
    if (a.n_work == 0) return HFK_OK;
    if (workgroups == 0) {
        workgroups = beside ? kBesideDuplexWorkgroups : (uint32_t)knob_value(HFK_KNOB_DUPLEX_WORKGROUPS);
    }
    uint32_t grid = 0;
    rc = pick_grid(a.n_work, workgroups, &grid);
    if (rc != 0) return rc;
    const uint64_t out_bytes = out_move ? (uint64_t)n_planes * out_move->n_pairs * block_bytes : 0;
    if (a.first.n_work != 0 && (beside || out_bytes >= kLongSwapBytes)) {
        // Every iteration moves one chunk toward the host (and one from it): offer the link what the
        // paced one-way swap offers it in the same mode.
        uint32_t pace_mbps = 0;
        if (beside) {
            pace_mbps = (uint32_t)knob_value(HFK_KNOB_SWAP_PACE_MBPS);
            if (pace_mbps == 0) pace_mbps = (uint32_t)(kPaceShareOfLink * current_link_mbps());
        } else {
            pace_mbps = (uint32_t)(knob_value(HFK_KNOB_DUPLEX_PACE_PERMILLE) / 1000.0 * current_link_mbps());
        }
        if (pace_mbps != 0) {
            a.pace_q8 = pace_interval_q8((double)block_bytes / a.first.chunks_per_block, grid, pace_mbps);
            }
    }
    const int nt = (int)knob_value(HFK_KNOB_NONTEMPORAL);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (unroll) {
        case 1: launch_duplex_nt<1>(a, grid, nt, s); break;
        case 2: launch_duplex_nt<2>(a, grid, nt, s); break;
        case 4: launch_duplex_nt<4>(a, grid, nt, s); break;
        case 8: launch_duplex_nt<8>(a, grid, nt, s); break;
        default: launch_duplex_nt<16>(a, grid, nt, s); break;
    }
    return finish_launch();
}

int hfk_swap_blocks_staged(const void* dev_plane_ptrs, void* const* host_plane_addrs, const int64_t* dev_block_ids,
                           const int64_t* host_block_ids, uint32_t n_planes, uint64_t n_blocks, uint64_t block_bytes,
                           uint64_t dev_block_stride, uint64_t host_block_stride, uint64_t dev_blocks,
                           uint64_t host_blocks, void* staging, int to_host, uint32_t workgroups,
                           hfk_stream_t stream) {
    if (n_planes == 0 || n_blocks == 0) return HFK_OK;
    return staged_swap(dev_plane_ptrs, host_plane_addrs, dev_block_ids, host_block_ids, n_planes, n_blocks, block_bytes,
                       dev_block_stride, host_block_stride, dev_blocks, host_blocks, staging, to_host, workgroups,
                       static_cast<hipStream_t>(stream));
}

int hfk_swap_blocks_staged_static(const void* dev_plane_ptrs, void* const* host_plane_addrs,
                                  const int64_t* dev_block_ids, const int64_t* host_block_ids, uint32_t n_planes,
                                  uint64_t n_blocks, uint64_t block_bytes, uint64_t dev_block_stride,
                                  uint64_t host_block_stride, uint64_t dev_blocks, uint64_t host_blocks, int to_host,
                                  uint32_t workgroups, hfk_stream_t stream) {
    if (n_planes == 0 || n_blocks == 0) return HFK_OK;
    // n_planes * n_blocks * block_bytes <= kStaticStagingBytes, without overflowing on the way
    if (block_bytes == 0) return HFK_ERR_BAD_SIZE;
    if (block_bytes > kStaticStagingBytes || n_blocks > kStaticStagingBytes / block_bytes ||
        (uint64_t)n_planes > kStaticStagingBytes / (n_blocks * block_bytes)) {
        return HFK_ERR_STAGING_TOO_SMALL;
    }
    void* staging = nullptr;
    int rc = static_staging(&staging);
    if (rc != 0) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    int dev = 0;
    bool guarded = false;
    rc = static_acquire(s, &dev, &guarded);
    if (rc != 0) return rc;
    rc = staged_swap(dev_plane_ptrs, host_plane_addrs, dev_block_ids, host_block_ids, n_planes, n_blocks, block_bytes,
                     dev_block_stride, host_block_stride, dev_blocks, host_blocks, staging, to_host, workgroups, s);
    static_release(s, dev, guarded);   // also after a failure: part of the work may be enqueued
    return rc;
}

int hfk_swap_blocks_auto(const void* dev_plane_ptrs, const void* host_plane_ptrs, void* const* host_plane_addrs,
                         const int64_t* block_pairs, const int64_t* host_block_ids, uint32_t n_planes,
                         uint64_t n_pairs, uint64_t block_bytes, uint64_t dev_block_stride,
                         uint64_t host_block_stride, uint64_t dev_blocks, uint64_t host_blocks, void* staging,
                         uint64_t staging_bytes, int to_host, uint32_t min_run_blocks, uint32_t flags,
                         hfk_stream_t stream) {
    if ((flags & ~(uint32_t)HFK_SWAP_BESIDE_COMPUTE) != 0) return HFK_ERR_BAD_FLAGS;
    if (n_planes == 0 || n_pairs == 0) return HFK_OK;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool out = to_host != 0;
    if (host_block_ids != nullptr && block_pairs != nullptr && knob_value(HFK_KNOB_CHECK_HOST_COLUMN) != 0) {
        // Debugging aid: the two movers read the host column from two places; make sure they agree.
        hipError_t e = hipStreamSynchronize(s);   // whatever uploads the table on this stream has finished
        std::vector<int64_t> table;
        try {
            table.resize(2 * n_pairs);
        } catch (...) {                           // nothing may be thrown across this interface
            return HFK_ERR_TOO_LARGE;
        }
        if (e == hipSuccess) e = hipMemcpy(table.data(), block_pairs, 2 * n_pairs * sizeof(int64_t), hipMemcpyDefault);
        if (e != hipSuccess) return (int)e;
        for (uint64_t j = 0; j < n_pairs; ++j) {
            if (table[2 * j + (out ? 1 : 0)] != host_block_ids[j]) return HFK_ERR_TABLE_MISMATCH;
        }
    }
    const uint32_t side_flags = flags | (out ? HFK_SWAP_DST_HOST : HFK_SWAP_SRC_HOST);
    // The direct mover over the whole table: (src, dst) = (device, host) on the way out, (host, device) back.
    BlockCopyArgs<int64_t> direct;
    int rc = out ? hfk::plan_swap_blocks(direct, host_plane_ptrs, dev_plane_ptrs, block_pairs, n_planes, n_pairs,
                                         block_bytes, dev_block_stride, host_block_stride, dev_blocks, host_blocks)
                 : hfk::plan_swap_blocks(direct, dev_plane_ptrs, host_plane_ptrs, block_pairs, n_planes, n_pairs,
                                         block_bytes, host_block_stride, dev_block_stride, host_blocks, dev_blocks);
    if (rc != 0) return rc;
    direct.zero_skipped = out ? 1u : 0u;   // one rule for the whole table, whichever mover takes a pair
    const uint64_t total_bytes = (uint64_t)n_planes * n_pairs * block_bytes;
    // Staging the copy engines' share takes the host arrays and a buffer: one that holds the blocks of the
    // long runs and, behind them, the two lists of pairs (16 bytes per pair), or one that holds the whole
    // table ([n_planes][n_pairs] blocks).
    const bool have_arrays = staging != nullptr && host_plane_addrs != nullptr && host_block_ids != nullptr;
    const bool holds_table = have_arrays && staging_bytes / block_bytes / n_pairs >= n_planes;
    uint64_t min_run = min_run_blocks;
    uint64_t long_blocks = 0;
    if (have_arrays) {
        const HostLeg probe{host_plane_addrs, host_block_ids, n_planes, n_pairs, block_bytes, host_block_stride, staging,
                            out};
        rc = check_host_leg(probe, host_blocks);
        if (rc != 0) return rc;
        if (min_run == 0) {
            // A copy costs the DMA engines about 9.5 us before its first byte, 0.5 MiB of link time. A swap
            // that has the GPU to itself hands them only runs they move at 97 % of the link rate or better
            // (16 MiB per copy); one that shares it gives up to 12 % of its own rate (4 MiB per copy) so
            // that more of the table bypasses the compute units.
            const uint64_t run_bytes = (flags & HFK_SWAP_BESIDE_COMPUTE) != 0 ? kDmaRunBytesBesideCompute : kDmaRunBytes;
            const uint64_t planes_per_copy = host_block_stride == block_bytes ? evenly_spaced_planes(probe) : 1;
            const uint64_t per_block = block_bytes * planes_per_copy;
            min_run = (run_bytes + per_block - 1) / per_block;
        }
        if (min_run <= kMaxRunFilter) long_blocks = hfk::blocks_in_long_runs(host_block_ids, n_pairs, min_run);
    }
    // A table that is split is moved by two lists of pairs, which a one-workgroup kernel of this call writes
    // behind the staged blocks; the staging buffer then holds the long runs only, in table order. Without room
    // for the lists (tiny blocks) a buffer that holds the whole table is used with pair j in slot j and the
    // kernels sort the pairs out themselves (the run filter); a buffer that holds neither is not used.
    const bool split = long_blocks != 0 && long_blocks < n_pairs;
    bool listed = false;
    uint64_t lists_offset = 0;
    if (split && n_pairs <= 0x7fffffffu && long_blocks <= staging_bytes / block_bytes / n_planes) {
        lists_offset = (n_planes * long_blocks * block_bytes + 255u) & ~(uint64_t)255u;
        listed = lists_offset <= staging_bytes && n_pairs <= (staging_bytes - lists_offset) / (2 * sizeof(int64_t));
    }
    if (long_blocks != 0 && !listed && !holds_table) long_blocks = 0;   // everything goes direct
    if (long_blocks == 0) {   // nothing for the copy engines (or no staging to give them): one direct launch
        return launch_swap(direct, side_flags, 0, total_bytes, s);
    }
    HostLeg leg{host_plane_addrs, host_block_ids, n_planes, n_pairs, block_bytes, host_block_stride, staging, out};
    leg.compact = listed;
    leg.stage_plane_blocks = long_blocks;
    const int64_t* host_column = block_pairs + (out ? 1 : 0);
    const int64_t* dev_column = block_pairs + (out ? 0 : 1);
    BlockCopyArgs<int64_t> hbm;   // long runs: device planes <-> staging, the copy engines do the rest
    rc = hfk::plan_stage_blocks(hbm, dev_plane_ptrs, staging, dev_column, n_planes, listed ? long_blocks : n_pairs, block_bytes,
                                dev_block_stride, dev_blocks, out);
    if (rc != 0) return rc;
    hbm.id_stride = 2;
    if (listed) {   // both lists, computed on the device from the device's table
        int64_t* long_list = reinterpret_cast<int64_t*>(static_cast<char*>(staging) + lists_offset);
        int64_t* short_list = long_list + n_pairs;
        hipLaunchKernelGGL(pair_lists_kernel, dim3(1), dim3(256), 0, s, host_column, 2u, (uint32_t)n_pairs, (uint32_t)min_run,
                           long_list, short_list);
        rc = finish_launch();
        if (rc != 0) return rc;
        hfk::list_pairs(hbm, long_list, (uint32_t)long_blocks, (uint32_t)n_pairs);
        hfk::list_pairs(direct, short_list, (uint32_t)(n_pairs - long_blocks), (uint32_t)n_pairs);
    } else if (split) {
        hfk::filter_runs(hbm, hfk::kLongRunsOnly, host_column, (uint32_t)min_run);
        hfk::filter_runs(direct, hfk::kShortRunsOnly, host_column, (uint32_t)min_run);
    }
    if (out) {
        rc = launch_block_copy<Role::kGatherBlocks, int64_t>(hbm, 0, s);
        if (rc == 0) rc = copy_host_runs(leg, min_run, s);
    } else {
        rc = copy_host_runs(leg, min_run, s);
        if (rc == 0) rc = launch_block_copy<Role::kScatterBlocks, int64_t>(hbm, 0, s);
    }
    if (rc != 0 || !split) return rc;
    return launch_swap(direct, side_flags, 0, (n_pairs - long_blocks) * n_planes * block_bytes, s);
}

int hfk_gather_blocks(const void* dst_plane_ptrs, const void* src_plane_ptrs, const int64_t* ids,
                      uint32_t n_planes, uint64_t n_ids, uint64_t block_bytes, uint64_t src_block_stride,
                      uint64_t src_blocks, uint32_t flags, uint32_t workgroups, hfk_stream_t stream) {
    if ((flags & ~(uint32_t)(HFK_SWAP_SRC_HOST | HFK_SWAP_BESIDE_COMPUTE)) != 0) return HFK_ERR_BAD_FLAGS;
    if (n_planes == 0 || n_ids == 0) return HFK_OK;
    BlockCopyArgs<int64_t> a;
    int rc = hfk::plan_gather_blocks(a, dst_plane_ptrs, src_plane_ptrs, ids, n_planes, n_ids, block_bytes,
                                     src_block_stride, src_blocks);
    if (rc != 0) return rc;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if ((flags & HFK_SWAP_SRC_HOST) != 0) {
        // Source planes in host memory: this is a swap-in whose destinations are consecutive, and the
        // PCIe link, not HBM, sizes the launch.
        return launch_swap(a, flags, workgroups, (uint64_t)n_planes * n_ids * block_bytes, s);
    }
    return launch_block_copy<Role::kGatherBlocks, int64_t>(a, workgroups, s);
}

int hfk_pace_state(uint32_t* out8) {
    if (out8 == nullptr) return HFK_ERR_NULL_POINTER;
    uint32_t* words = nullptr;
    int rc = pace_state(&words);
    if (rc != 0) return rc;
    hipError_t e = hipMemcpy(out8, words, 8 * sizeof(uint32_t), hipMemcpyDeviceToHost);   // waits for the device
    return e == hipSuccess ? HFK_OK : (int)e;
}

int hfk_set_tuning(int knob, int64_t value) {
    if (knob < 0 || knob >= kKnobCount || !knob_value_valid(knob, value)) return HFK_ERR_BAD_KNOB;
    g_knob[knob].store(value, std::memory_order_relaxed);
    return HFK_OK;
}

int64_t hfk_get_tuning(int knob) {
    if (knob < 0 || knob >= kKnobCount) return HFK_ERR_BAD_KNOB;
    if (knob == HFK_KNOB_LINK_MBPS) return current_link_mbps();
    return knob_value(knob);
}

int hfk_thread_tuning_begin(const hfk_knob_value* overrides, uint32_t n) {
    if (n != 0 && overrides == nullptr) return HFK_ERR_NULL_POINTER;
    ThreadTuning next;
    for (uint32_t i = 0; i < n; ++i) {
        const int k = overrides[i].knob;
        if (k < 0 || k >= kKnobCount || !knob_value_valid(k, overrides[i].value)) return HFK_ERR_BAD_KNOB;
        next.mask |= 1u << k;
        next.value[k] = overrides[i].value;
    }
    t_tuning = next;   // replaces whatever this thread had; nothing is kept on a rejected list
    return HFK_OK;
}

void hfk_thread_tuning_end(void) { t_tuning = ThreadTuning{}; }

}  // extern "C"
