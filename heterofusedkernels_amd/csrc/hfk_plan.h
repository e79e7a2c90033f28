// Launch planning: turns the C-ABI arguments into kernel argument structs and
// picks the access width. Pure host arithmetic with no HIP calls, shared by the
// launchers and by the CPU index-math checker, so both walk the same geometry.
#pragma once

#include <stdint.h>
#include <stdlib.h>

#include "hfk.h"
#include "hfk_bodies.h"

namespace hfk {

constexpr uint64_t kUnchecked = 1ull << 63;  // "no bound": still rejects negative ids
constexpr uint64_t kU32Max = 0xffffffffull;

// Rows at least this wide go through the block-copy kernel (uniform id loads, no
// per-lane division); narrower rows through the flat kernel.
constexpr uint64_t kWideRowBytes = 4096;
// Units per lane of the flat row gather: one for a table in device memory (finer workgroups spread
// the traffic better: 5.98-6.08 TB/s against 5.85-5.92 with four), four for a table in host memory
// (a 1 MiB gather of 1 KiB rows over PCIe takes 22 us against 27).
constexpr int kFlatUnrollDevice = 1;
constexpr int kFlatUnrollHost = 4;
// Units per lane of the layout-converting transfer: two (one block from host memory 53-57 GB/s,
// eight blocks 57 GB/s; one unit per lane needs twice the workgroups, four gain nothing), except
// toward a packed pool in host memory, where eight hold 53.2-53.9 GB/s and two 52.2-53.2.
constexpr int kTransposeUnroll = 2;
constexpr int kTransposeUnrollToHost = 8;

// A block smaller than 256 * unroll vectors would leave lanes idle, so the unroll
// is halved until one chunk fits inside the block (down to 1).
inline int fit_unroll(uint64_t block_bytes, int unroll) {
    while (unroll > 1 && (uint64_t)kWorkgroupLanes * 16u * (uint64_t)unroll > block_bytes) {
        unroll >>= 1;
    }
    return unroll;
}

// ---- launch shape of a block-table swap -------------------------------------
// What a swap launch looks like follows from what the caller says about it (flags), how much it
// moves, and the link's rate; the rules live here, apart from the launching code, so that a CPU
// test can pin them. Workgroups x 16-byte vectors per lane, the rate offered toward the host
// (0 = unpaced), and whether the stores are plain (through the L2) or non-temporal (streamed). The
// measurements behind each shape stand beside the tunables in hfk_capi.hip.
// Toward the host, throughput mode: unpaced, plain stores, and a grid that keeps 96-128 vectors per lane
// in flight: 12 x 8 for blocks of 32 KiB and more, 32 x 4, 64 x 2 or 96 x 1 for smaller ones. Measured
// for blocks of 4 KiB to 128 KiB on random tables (256 MiB per launch): 12 x 8 56.6 GB/s, 32 x 4
// 56.5-56.6 (24 x 4 56.3-56.5, and 55.9 against 56.6 on a table of fragmented runs of 16 KiB blocks),
// 64 x 2 56.4-56.6, 96 x 1 56.5; half as much in flight 54.6-55.5, twice as much no more. A block that
// does not divide into whole chunks gets 32 x 4 (72 KiB blocks: 56.6 against 54.8 on 12 x 8), and no
// grid may be a multiple of the chunks per block when the last chunk is short: the same workgroups
// would then draw the short chunks every time (12 workgroups, chunks of 32 + 32 + 8 KiB: four of them
// idle most of the time).
constexpr int kToHostUnroll = 8;
constexpr uint32_t kToHostRaggedWorkgroups = 32;
constexpr int kToHostRaggedUnroll = 4;
inline uint32_t to_host_workgroups(int unroll) { return unroll >= 8 ? 12u : unroll == 4 ? 32u : unroll == 2 ? 64u : 96u; }
constexpr uint32_t kBesidePacedWorkgroups = 12;    // toward the host, beside compute: 12 x 1 paced at 0.84
constexpr uint32_t kFromHostWorkgroups = 40;       // from the host: 40 x 1
constexpr uint32_t kBesideFromHostWorkgroups = 24; // from the host, beside compute: 24 x 1
constexpr uint32_t kBesideWorkgroups = 8;          // beside compute, no usable pace: 8 x 4 unpaced
constexpr int kBesideUnnamedUnroll = 4;
constexpr int kFineUnroll = 1;
constexpr double kBesidePaceShareOfLink = 0.84;
// From this size on a throughput-mode swap toward the host writes through the L2 (and a paced one,
// if pacing is switched on, is paced); a shorter one is over before either could pay.
constexpr uint64_t kLongSwapBytes = 64ull << 20;

struct SwapTuning {              // what hfk_set_tuning can change
    uint32_t swap_workgroups;    // no side named
    int swap_unroll;
    uint32_t paced_workgroups;   // toward a named host side, throughput mode, when paced
    int paced_unroll;
    uint32_t throughput_pace_permille;   // 0 (default) = that swap is not paced
    uint32_t beside_pace_mbps;   // 0 = kBesidePaceShareOfLink of the link
};

struct SwapShape {
    uint32_t workgroups;
    int unroll;
    uint32_t pace_mbps;
    bool plain_stores;
};

inline SwapShape to_host_shape(uint64_t block_bytes) {
    int unroll = fit_unroll(block_bytes, kToHostUnroll);
    uint32_t grid = to_host_workgroups(unroll);
    uint64_t chunk_bytes = (uint64_t)kWorkgroupLanes * 16u * (uint64_t)unroll;
    if (block_bytes > chunk_bytes && block_bytes % chunk_bytes != 0) {
        if (unroll > kToHostRaggedUnroll) {
            unroll = kToHostRaggedUnroll;
            grid = kToHostRaggedWorkgroups;
            chunk_bytes = (uint64_t)kWorkgroupLanes * 16u * (uint64_t)unroll;
        }
        const uint64_t chunks = (block_bytes + chunk_bytes - 1) / chunk_bytes;
        if (grid % chunks == 0) ++grid;
    }
    return SwapShape{grid, unroll, 0, true};
}

// `workgroups` != 0 is the caller's own grid bound and is kept; `link_mbps` 0 = unknown; `bytes` is what
// the launch moves in all, `block_bytes` the size of one block.
inline SwapShape choose_swap_shape(uint32_t flags, uint64_t bytes, uint64_t block_bytes, uint32_t link_mbps,
                                   uint32_t workgroups, const SwapTuning& t) {
    const bool beside = (flags & HFK_SWAP_BESIDE_COMPUTE) != 0;
    if ((flags & HFK_SWAP_DST_HOST) != 0 && (beside || bytes >= kLongSwapBytes)) {
        uint32_t pace = 0;
        if (beside) pace = t.beside_pace_mbps != 0 ? t.beside_pace_mbps : (uint32_t)(kBesidePaceShareOfLink * link_mbps);
        else pace = (uint32_t)(t.throughput_pace_permille / 1000.0 * link_mbps);
        if (pace != 0) {
            // the paced throughput shape keeps paced_workgroups x paced_unroll vectors per lane in flight:
            // blocks too small for that many vectors per lane get more workgroups instead
            const int fitted = beside ? kFineUnroll : fit_unroll(block_bytes, t.paced_unroll);
            const uint32_t grid = beside ? kBesidePacedWorkgroups : t.paced_workgroups * (uint32_t)(t.paced_unroll / fitted);
            return SwapShape{workgroups ? workgroups : grid, fitted, pace, false};
        }
        if (!beside) {
            SwapShape shape = to_host_shape(block_bytes);
            if (workgroups != 0) shape.workgroups = workgroups;
            return shape;
        }
    }
    if ((flags & HFK_SWAP_SRC_HOST) != 0) {
        const uint32_t grid = beside ? kBesideFromHostWorkgroups : kFromHostWorkgroups;
        return SwapShape{workgroups ? workgroups : grid, kFineUnroll, 0, false};
    }
    if (beside) return SwapShape{workgroups ? workgroups : kBesideWorkgroups, kBesideUnnamedUnroll, 0, false};
    return SwapShape{workgroups ? workgroups : t.swap_workgroups, t.swap_unroll, 0, false};
}

// Raw rate of a PCIe link in MB/s (lanes x GT/s x line encoding / 8) from the two strings sysfs
// shows for it, e.g. "32.0 GT/s PCIe" and "16"; -1 when either does not parse. Links below
// 8 GT/s use 8b/10b encoding, faster ones 128b/130b.
inline int link_mbps_from_sysfs(const char* speed_text, const char* width_text) {
    if (speed_text == nullptr || width_text == nullptr) return -1;
    char* end = nullptr;
    const double gts = strtod(speed_text, &end);
    if (end == speed_text || !(gts > 0.0) || gts > 1024.0) return -1;
    const long width = strtol(width_text, &end, 10);
    if (end == width_text || width <= 0 || width > 32) return -1;
    const double encoding = gts >= 8.0 ? 128.0 / 130.0 : 0.8;
    return (int)(gts * 1000.0 * (double)width * encoding / 8.0);
}

// For launches with one workgroup per chunk (the HBM-bound gathers): the largest unroll of at
// least 2, not above the preferred one, that cuts the block into whole chunks; a short tail
// chunk costs such a launch a workgroup that does a fraction of the work (72 KiB blocks: 6.00 TB/s
// in 8 KiB chunks against 5.86 in chunks of 32 + 32 + 8 KiB). Falls back to fit_unroll.
inline int fit_unroll_whole_chunks(uint64_t block_bytes, int unroll) {
    for (int u = fit_unroll(block_bytes, unroll); u >= 2; u >>= 1) {
        if (block_bytes % ((uint64_t)kWorkgroupLanes * 16u * (uint64_t)u) == 0) return u;
    }
    return fit_unroll(block_bytes, unroll);
}

// Fills chunks_per_block and n_work; returns the unroll to launch with.
template <typename IdT>
inline int plan_block_copy(BlockCopyArgs<IdT>& a, int preferred_unroll, int* unroll_out,
                           bool prefer_whole_chunks = false) {
    const int unroll = prefer_whole_chunks ? fit_unroll_whole_chunks(a.block_bytes, preferred_unroll)
                                           : fit_unroll(a.block_bytes, preferred_unroll);
    const uint64_t chunk_bytes = (uint64_t)kWorkgroupLanes * 16u * (uint64_t)unroll;
    const uint64_t chunks = (a.block_bytes + chunk_bytes - 1) / chunk_bytes;
    const uint64_t tiles = (uint64_t)a.n_planes * (uint64_t)a.n_pairs;
    if (chunks > kU32Max || tiles > kU32Max || chunks * tiles > kU32Max) return HFK_ERR_TOO_LARGE;
    a.chunks_per_block = (uint32_t)chunks;
    a.n_work = (uint32_t)(chunks * tiles);
    *unroll_out = unroll;
    return HFK_OK;
}

inline uint32_t pick_unit(uint64_t alignment_bits) {
    return (alignment_bits & 15u) == 0 ? 16u : (alignment_bits & 3u) == 0 ? 4u : 1u;
}

struct FlatGatherPlan {
    uint32_t unit;       // bytes per access: 16, 4 or 1
    bool index32;        // flat indices fit 32 bits (cheap division)
};

template <typename IdT>
inline int plan_flat_gather(FlatGatherArgs<IdT>& a, FlatGatherPlan& p, uint64_t table, uint64_t dst,
                            const IdT* ids, uint64_t n_ids, uint64_t row_bytes, uint64_t row_limit, int unroll) {
    p.unit = pick_unit(table | dst | row_bytes);
    a.table = table;
    a.dst = dst;
    a.ids = ids;
    a.row_units = (uint32_t)(row_bytes / p.unit);
    a.total_units = n_ids * (uint64_t)a.row_units;
    a.row_limit = row_limit;
    const uint64_t chunk_units = (uint64_t)kWorkgroupLanes * (uint64_t)unroll;
    const uint64_t n_work = (a.total_units + chunk_units - 1) / chunk_units;
    if (n_work > kU32Max) return HFK_ERR_TOO_LARGE;
    a.n_work = (uint32_t)n_work;
    p.index32 = n_work * chunk_units <= kU32Max;
    return HFK_OK;
}

// Geometry of the layout-converting transfer over a block table (pairs == nullptr:
// the single block at the two base addresses). Returns HFK_OK with n_work == 0
// when there is nothing to move. `mirror`: a second place that receives the packed blocks as they
// are while a transfer out of the packed side reads them (TransposeArgs::mirror), or null.
inline int plan_transpose(TransposeArgs& a, uint32_t* unit_out, const void* dev_layer_ptrs, const void* packed,
                          const int64_t* pairs, uint64_t n_pairs, uint64_t packed_stride, uint64_t layered_stride,
                          uint64_t packed_blocks, uint64_t layered_blocks, uint32_t T, uint32_t L, uint32_t H,
                          uint32_t D, uint32_t elem_bytes, int unroll = kTransposeUnroll, const void* mirror = nullptr) {
    a = TransposeArgs{};
    if (dev_layer_ptrs == nullptr || packed == nullptr) return HFK_ERR_NULL_POINTER;
    if (elem_bytes == 0) return HFK_ERR_BAD_SIZE;
    if (T == 0 || L == 0 || H == 0 || D == 0 || n_pairs == 0) return HFK_OK;
    const uint64_t row_bytes = (uint64_t)D * elem_bytes;
    const uint64_t rows = (uint64_t)T * L * H;
    // The kernel indexes the units of one block with 32 bits.
    if ((uint64_t)L * H > kU32Max || rows > kU32Max || rows * row_bytes > kU32Max) return HFK_ERR_TOO_LARGE;
    const uint64_t block_bytes = rows * row_bytes;
    const uint64_t layer_block_bytes = (uint64_t)H * T * row_bytes;
    if (pairs != nullptr && (packed_stride < block_bytes || layered_stride < layer_block_bytes)) {
        return HFK_ERR_BAD_SIZE;
    }
    uint64_t align = (uint64_t)(uintptr_t)packed | (uint64_t)(uintptr_t)mirror | row_bytes;
    if (pairs != nullptr) align |= packed_stride | layered_stride;
    const uint32_t unit = pick_unit(align);
    const uint64_t row_units = row_bytes / unit;
    const uint64_t total = rows * row_units;
    const uint64_t chunk_units = (uint64_t)kWorkgroupLanes * (uint64_t)unroll;
    const uint64_t chunks = (total + chunk_units - 1) / chunk_units;
    if (n_pairs > kU32Max || chunks * n_pairs > kU32Max) return HFK_ERR_TOO_LARGE;
    a.layer_ptrs = static_cast<const uint64_t*>(dev_layer_ptrs);
    a.packed = (uint64_t)(uintptr_t)packed;
    a.pairs = pairs;
    a.packed_stride = packed_stride;
    a.layered_stride = layered_stride;
    a.packed_limit = packed_blocks ? packed_blocks : kUnchecked;
    a.layered_limit = layered_blocks ? layered_blocks : kUnchecked;
    a.n_pairs = (uint32_t)n_pairs;
    a.chunks_per_block = (uint32_t)chunks;
    a.T = T;
    a.L = L;
    a.H = H;
    a.row_units = (uint32_t)row_units;
    a.total_units = (uint32_t)total;
    a.n_work = (uint32_t)(chunks * n_pairs);
    a.mirror = (uint64_t)(uintptr_t)mirror;
    *unit_out = unit;
    return HFK_OK;
}

// Turns a planned transfer (plan_transpose, 16-byte units) into its tiled form when the geometry allows
// (see transpose_tile_load): picks the largest U of 8, 4, 2, 1 with L * H a multiple of 4 * U, sets the
// tile fields, chunks_per_block (tiles per block) and n_work. Returns U, or 0 when the transfer has to
// go the direct way (a is then unchanged). `max_layers`: what the kernel's layer table holds.
inline int plan_transpose_tiles(TransposeArgs& a, uint32_t unit, uint32_t max_layers) {
    if (unit != 16u || a.n_work == 0 || a.L > max_layers) return 0;
    const uint32_t ru = a.row_units;
    if (ru == 0 || ru > 64u || (ru & (ru - 1)) != 0) return 0;
    const uint32_t tile_tokens = 64u / ru;
    if (a.T % tile_tokens != 0) return 0;
    const uint64_t LH = (uint64_t)a.L * a.H;
    int U = 8;
    while (U >= 1 && LH % (4u * (uint32_t)U) != 0) U >>= 1;
    if (U < 1) return 0;
    const uint64_t tiles = (uint64_t)(a.T / tile_tokens) * (LH / (4u * (uint32_t)U));
    if (tiles * a.n_pairs > kU32Max) return 0;
    a.tile_tokens = tile_tokens;
    a.tile_rows = 4u * (uint32_t)U;
    a.chunks_per_block = (uint32_t)tiles;
    a.n_work = (uint32_t)(tiles * a.n_pairs);
    return U;
}

// Argument checks + struct fill for the public block-table entry points.
inline int plan_swap_blocks(BlockCopyArgs<int64_t>& a, const void* dst_plane_ptrs, const void* src_plane_ptrs,
                            const int64_t* block_pairs, uint32_t n_planes, uint64_t n_pairs,
                            uint64_t block_bytes, uint64_t src_block_stride, uint64_t dst_block_stride,
                            uint64_t src_blocks, uint64_t dst_blocks) {
    if (dst_plane_ptrs == nullptr || src_plane_ptrs == nullptr || block_pairs == nullptr) {
        return HFK_ERR_NULL_POINTER;
    }
    if (block_bytes == 0 || src_block_stride < block_bytes || dst_block_stride < block_bytes) {
        return HFK_ERR_BAD_SIZE;
    }
    if (n_pairs > kU32Max) return HFK_ERR_TOO_LARGE;
    a = BlockCopyArgs<int64_t>{};
    a.dst_planes = static_cast<const uint64_t*>(dst_plane_ptrs);
    a.src_planes = static_cast<const uint64_t*>(src_plane_ptrs);
    a.src_ids = block_pairs;
    a.dst_ids = block_pairs + 1;
    a.id_stride = 2;
    a.n_planes = n_planes;
    a.n_pairs = (uint32_t)n_pairs;
    a.block_bytes = block_bytes;
    a.src_stride = src_block_stride;
    a.dst_stride = dst_block_stride;
    a.src_limit = src_blocks ? src_blocks : kUnchecked;
    a.dst_limit = dst_blocks ? dst_blocks : kUnchecked;
    return HFK_OK;
}

// Both sides of a duplex swap share planes, block size and therefore the chunking.
inline int plan_duplex(DuplexCopyArgs& d, const hfk_block_move* out_move, const hfk_block_move* in_move,
                       uint32_t n_planes, uint64_t block_bytes, int preferred_unroll, int* unroll_out) {
    d = DuplexCopyArgs{};
    const hfk_block_move* moves[2] = {out_move, in_move};
    BlockCopyArgs<int64_t>* sides[2] = {&d.first, &d.second};
    int unroll = fit_unroll(block_bytes, preferred_unroll);
    for (int i = 0; i < 2; ++i) {
        const hfk_block_move* m = moves[i];
        if (m == nullptr || m->n_pairs == 0 || n_planes == 0) continue;  // this side has nothing to do
        int rc = plan_swap_blocks(*sides[i], m->dst_plane_ptrs, m->src_plane_ptrs, m->block_pairs, n_planes, m->n_pairs,
                                  block_bytes, m->src_block_stride, m->dst_block_stride, m->src_blocks, m->dst_blocks);
        if (rc != HFK_OK) return rc;
        int u = unroll;
        rc = plan_block_copy<int64_t>(*sides[i], unroll, &u);
        if (rc != HFK_OK) return rc;
    }
    d.n_work = d.first.n_work > d.second.n_work ? d.first.n_work : d.second.n_work;
    *unroll_out = unroll;
    return HFK_OK;
}

inline int plan_gather_blocks(BlockCopyArgs<int64_t>& a, const void* dst_plane_ptrs, const void* src_plane_ptrs,
                              const int64_t* ids, uint32_t n_planes, uint64_t n_ids, uint64_t block_bytes,
                              uint64_t src_block_stride, uint64_t src_blocks) {
    if (dst_plane_ptrs == nullptr || src_plane_ptrs == nullptr || ids == nullptr) return HFK_ERR_NULL_POINTER;
    if (block_bytes == 0 || src_block_stride < block_bytes) return HFK_ERR_BAD_SIZE;
    if (n_ids > kU32Max) return HFK_ERR_TOO_LARGE;
    a = BlockCopyArgs<int64_t>{};
    a.dst_planes = static_cast<const uint64_t*>(dst_plane_ptrs);
    a.src_planes = static_cast<const uint64_t*>(src_plane_ptrs);
    a.src_ids = ids;
    a.dst_ids = nullptr;
    a.id_stride = 1;
    a.n_planes = n_planes;
    a.n_pairs = (uint32_t)n_ids;
    a.block_bytes = block_bytes;
    a.src_stride = src_block_stride;
    a.dst_stride = block_bytes;
    a.src_limit = src_blocks ? src_blocks : kUnchecked;
    a.dst_limit = kUnchecked;
    return HFK_OK;
}

// The kernel half of a staged swap: blocks between the device planes and a
// contiguous staging buffer [n_planes][n_blocks][block_bytes] in device memory.
// to_staging: staging[p][i] = plane_p[ids[i]]  (gather);  else  plane_p[ids[i]] = staging[p][i]  (scatter).
// Pair j's blocks live in staging slot j and a plane of the staging buffer holds n_blocks slots. (A launch
// that is handed a list of pairs, list_pairs(), counts its slots by the position in the list, so a
// staging buffer that holds only the listed share of a table is planned with n_blocks = that share.)
inline int plan_stage_blocks(BlockCopyArgs<int64_t>& a, const void* dev_plane_ptrs, void* staging,
                             const int64_t* dev_block_ids, uint32_t n_planes, uint64_t n_blocks, uint64_t block_bytes,
                             uint64_t dev_block_stride, uint64_t dev_blocks, bool to_staging) {
    if (dev_plane_ptrs == nullptr || staging == nullptr || dev_block_ids == nullptr) return HFK_ERR_NULL_POINTER;
    if (block_bytes == 0 || dev_block_stride < block_bytes) return HFK_ERR_BAD_SIZE;
    if (n_blocks > kU32Max) return HFK_ERR_TOO_LARGE;
    a = BlockCopyArgs<int64_t>{};
    a.id_stride = 1;
    a.n_planes = n_planes;
    a.n_pairs = (uint32_t)n_blocks;
    a.block_bytes = block_bytes;
    const uint64_t limit = dev_blocks ? dev_blocks : kUnchecked;
    if (to_staging) {
        a.src_planes = static_cast<const uint64_t*>(dev_plane_ptrs);
        a.src_ids = dev_block_ids;
        a.src_stride = dev_block_stride;
        a.src_limit = limit;
        a.dst_base = (uint64_t)(uintptr_t)staging;
        a.dst_ids = nullptr;
        a.dst_plane_stride = n_blocks * block_bytes;
        a.dst_stride = block_bytes;
        a.dst_limit = kUnchecked;
        // The copies that follow move staging[p][i] to the host whatever ids[i] was (the ids live on the
        // device), so an entry the kernel cannot fill is zeroed rather than left holding an earlier
        // transfer's bytes.
        a.zero_skipped = 1;
    } else {
        a.dst_planes = static_cast<const uint64_t*>(dev_plane_ptrs);
        a.dst_ids = dev_block_ids;
        a.dst_stride = dev_block_stride;
        a.dst_limit = limit;
        a.src_base = (uint64_t)(uintptr_t)staging;
        a.src_ids = nullptr;
        a.src_plane_stride = n_blocks * block_bytes;
        a.src_stride = block_bytes;
        a.src_limit = kUnchecked;
    }
    return HFK_OK;
}

// Splitting one block table between two movers by the length of its runs of consecutive host slots.
// A maximal run is entries first .. first + len - 1 with ids[i + 1] == ids[i] + 1. `f(first, len)` is
// called for every maximal run in table order. The kernels classify a pair with run_length_capped()
// (hfk_bodies.h), which gives min(cap, len) for the same maximal run: "long" means len >= min_run on
// both sides.
template <typename F>
inline void for_each_host_run(const int64_t* ids, uint64_t n, F f) {
    uint64_t first = 0;
    while (first < n) {
        uint64_t len = 1;
        while (first + len < n && ids[first + len] == ids[first + len - 1] + 1) ++len;
        f(first, len);
        first += len;
    }
}

// Blocks of the table that sit in runs of at least min_run entries.
inline uint64_t blocks_in_long_runs(const int64_t* ids, uint64_t n, uint64_t min_run) {
    uint64_t total = 0;
    for_each_host_run(ids, n, [&](uint64_t, uint64_t len) {
        if (len >= min_run) total += len;
    });
    return total;
}

// The two lists a split table is moved by: long_list holds the table indices of the pairs in long runs
// (runs of at least min_run consecutive ids), short_list those of all other pairs, both in table
// order; what is left of either array (n entries each) is set to -1. The i-th pair of long_list has
// staging slot i, which is how the copy engines' leg counts its slots as it walks the runs. The
// sequential statement of what pair_lists_kernel computes in parallel.
inline void fill_pair_lists(const int64_t* ids, uint32_t stride, uint64_t n, uint64_t min_run, int64_t* long_list,
                            int64_t* short_list) {
    uint64_t n_long = 0, n_short = 0;
    uint64_t first = 0;
    while (first < n) {
        uint64_t len = 1;
        while (first + len < n && ids[(first + len) * stride] == ids[(first + len - 1) * stride] + 1) ++len;
        for (uint64_t i = 0; i < len; ++i) {
            if (len >= min_run) long_list[n_long++] = (int64_t)(first + i);
            else short_list[n_short++] = (int64_t)(first + i);
        }
        first += len;
    }
    for (uint64_t i = n_long; i < n; ++i) long_list[i] = -1;
    for (uint64_t i = n_short; i < n; ++i) short_list[i] = -1;
}

// Hands a planned block copy over a table of n_total pairs the list of the n_listed pairs it is to move
// (BlockCopyArgs::run_mode kListedPairs).
template <typename IdT>
inline void list_pairs(BlockCopyArgs<IdT>& a, const int64_t* list, uint32_t n_listed, uint32_t n_total) {
    a.run_mode = kListedPairs;
    a.run_ids = list;
    a.run_min = n_total;
    a.n_pairs = n_listed;
}

// Restricts a planned block copy to the pairs in long (or short) runs of `run_ids`
// (entry j at run_ids[j * a.id_stride], the table column that holds the host slots).
template <typename IdT>
inline void filter_runs(BlockCopyArgs<IdT>& a, RunFilter mode, const int64_t* run_ids, uint32_t min_run) {
    a.run_mode = mode;
    a.run_ids = run_ids;
    a.run_min = min_run;
}

// Wide-row gather expressed as a single-plane block copy with dst block i = i.
template <typename IdT>
inline int plan_wide_gather(BlockCopyArgs<IdT>& a, const void* table, void* dst, const IdT* ids, uint64_t n_ids,
                            uint64_t row_bytes, uint64_t row_limit) {
    if (n_ids > kU32Max) return HFK_ERR_TOO_LARGE;
    a = BlockCopyArgs<IdT>{};
    a.dst_base = (uint64_t)(uintptr_t)dst;
    a.src_base = (uint64_t)(uintptr_t)table;
    a.src_ids = ids;
    a.dst_ids = nullptr;
    a.id_stride = 1;
    a.n_planes = 1;
    a.n_pairs = (uint32_t)n_ids;
    a.block_bytes = row_bytes;
    a.src_stride = row_bytes;
    a.dst_stride = row_bytes;
    a.src_limit = row_limit;
    a.dst_limit = kUnchecked;
    return HFK_OK;
}

}  // namespace hfk
