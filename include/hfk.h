/*
 * hfk.h - C-ABI of libhfk_hip.so: KV-cache block swap, block gather and the
 * layout-converting multi-layer block transfer for AMD MI355X (gfx950).
 *
 * Every entry point
 *   - takes plain pointers and sizes (no torch types),
 *   - enqueues work on the HIP stream it is given and returns without waiting,
 *   - returns 0 on success, a negative hfk_status for a rejected argument, or a
 *     positive hipError_t reported by the HIP runtime,
 *   - never throws, owns no memory and keeps no state between calls apart from
 *     cached device properties, the values set through hfk_set_tuning() (process-wide)
 *     or hfk_thread_tuning_begin() (calling thread only), one event per device for
 *     hfk_swap_blocks_staged_static, and, on the device, the eight words of hfk_pace_state().
 *
 * "Device-visible" below means an address a kernel may dereference: device
 * memory, or pinned host memory in its mapped (hipHostGetDevicePointer) form.
 * Host memory is read and written by the kernels directly over the PCIe link.
 *
 * The library moves bytes only; element types matter solely through their size.
 */
#ifndef HFK_H
#define HFK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HFK_API __attribute__((visibility("default")))

#define HFK_VERSION_MAJOR 0
#define HFK_VERSION_MINOR 3

/* A hipStream_t passed as an opaque pointer; NULL is the null stream. */
typedef void* hfk_stream_t;

enum hfk_status {
    HFK_OK = 0,
    HFK_ERR_NULL_POINTER = -1, /* a required pointer argument is NULL            */
    HFK_ERR_BAD_SIZE = -2,     /* a size/stride is zero or inconsistent          */
    HFK_ERR_TOO_LARGE = -3,    /* a count exceeds what one launch can index      */
    HFK_ERR_BAD_KNOB = -4,     /* unknown tuning knob or value out of range      */
    HFK_ERR_OUT_OF_RANGE = -5, /* an index passed in host memory is out of range */
    HFK_ERR_BAD_FLAGS = -6,    /* a flags argument has unknown bits set            */
    HFK_ERR_STAGING_TOO_SMALL = -7, /* the transfer does not fit the library's static staging buffer */
    HFK_ERR_STAGING_BUSY = -9,  /* the library's static staging buffer is in use by a call on another stream */
    HFK_ERR_TABLE_MISMATCH = -8 /* two forms of the same block table disagree (HFK_KNOB_CHECK_HOST_COLUMN) */
};

/* HFK_VERSION_MAJOR * 1000 + HFK_VERSION_MINOR of the loaded library. */
HFK_API int hfk_version(void);

/* Static, NUL-terminated description of a value returned by any hfk_* call
 * (negative: this library's codes, positive: hipGetErrorString). */
HFK_API const char* hfk_status_string(int status);

/*
 * Row gather:  dst[i, :] = table[ids[i], :]   for i in [0, n_ids)
 *
 * Replaces the reference's gather op and kernel:
 *   pcieThrough/csrc/host/gather_torch.cpp:30-54   (host op `pciethrough::gather`)
 *   pcieThrough/csrc/kernel/gather.cpp:7-48        (`gather_kernel`)
 *   pcieThrough/csrc/kernel/gather.h:85-133        (`Gather::MteCopy::LoadStoreFunc`)
 *
 *   table       device-visible, rows of row_bytes bytes, row r at table + r*row_bytes
 *   dst         device-visible, n_ids contiguous rows
 *   ids         device-visible, int64 (ids_are_i64 != 0) or int32 indices
 *   table_rows  number of rows in table; an id outside [0, table_rows) leaves its
 *               dst row untouched. 0 disables the check (the reference never checks).
 *   flags       0, HFK_SWAP_SRC_HOST (the table is host memory) or HFK_SWAP_SRC_DEVICE (it is device
 *               memory). Where the table lives shapes the launch; with 0 the library asks the
 *               runtime (for gathers of 64 KiB and more), which costs the calling thread about 5 us
 *               per call: as much as the whole launch of a small gather. A caller that knows says so.
 *   workgroups  upper bound on workgroups launched, 0 = library default: one workgroup per chunk
 *               of output for a table in device memory; for a table in host memory a gather of
 *               more than 4 MiB runs on 64 workgroups, which saturate the PCIe link (55-57 GB/s
 *               for 1 KiB rows) and slow kernels on other streams 2x where the device-sized grid
 *               slows them 5x.
 *
 * n_ids == 0 is a successful no-op. Rows of any byte size and alignment are
 * accepted; 16-byte aligned rows take the vectorised path.
 */
HFK_API int hfk_gather_rows(const void* table, void* dst, const void* ids, int ids_are_i64,
                    uint64_t n_ids, uint64_t row_bytes, uint64_t table_rows,
                    uint32_t flags, uint32_t workgroups, hfk_stream_t stream);

/*
 * Layout-converting transfer of one KV block across all layers:
 *   layer_l[(h*T + t)*D + d] = src_block[((t*L + l)*H + h)*D + d]
 * for t<T, l<L, h<H, d<D, elements of elem_bytes bytes; layer_l is the pointer
 * stored in dev_layer_ptrs[l].
 *
 * Replaces
 *   pcieThrough/csrc/host/multi_layer_block_transfer_torch.cpp:58-80
 *       (host op `pciethrough::multi_layer_block_transfer`, incl. the tiling upload
 *        `mvTilingToDevice` :13-39, which has no counterpart here: the geometry
 *        travels as kernel arguments)
 *   pcieThrough/csrc/kernel/multi_layer_block_transfer_kernel.cpp:8-29
 *   pcieThrough/csrc/kernel/multi_layer_block_transfer_kernel.h:42-82
 *
 *   dev_layer_ptrs  device-visible array of L uint64 addresses, each a
 *                   device-visible buffer of H*T*D*elem_bytes bytes ([H,T,D])
 *   src_block       device-visible [T,L,H,D] block (pinned host memory in the
 *                   reference's use, device memory for the staged variant)
 *   flags           0, HFK_SWAP_SRC_HOST or HFK_SWAP_SRC_DEVICE: where src_block lives, if the caller
 *                   knows (with 0 the library asks the runtime, about 5 us per call)
 */
HFK_API int hfk_multi_layer_block_transfer(const void* dev_layer_ptrs, const void* src_block,
                                   uint32_t T, uint32_t L, uint32_t H, uint32_t D,
                                   uint32_t elem_bytes, uint32_t flags, uint32_t workgroups,
                                   hfk_stream_t stream);

/*
 * Staged variant: afterwards staging == host_block and the layers hold what the transfer above gives.
 * The reference copies the block into staging (a whole-block asynchronous copy) and runs its kernel on
 * staging. Here a block in pinned, device-mapped host memory is read over the link once, by the kernel,
 * which writes every unit to its layer and to staging (as fast as the direct transfer: a block of
 * 4 MiB in 80 us, where a copy followed by a kernel takes 93); a block the device cannot address
 * (pageable memory), or HFK_KNOB_FUSED_COPY_ENGINE, goes the reference's way, hipMemcpyAsync on `stream`
 * and then the kernel. The bytes are the same either way.
 *
 * Replaces pcieThrough/csrc/host/multi_layer_block_transfer_torch.cpp:82-106
 * (`pciethrough::fused_memcpy_multi_layer_block_transfer`).
 *
 *   host_block  the host address of the [T,L,H,D] block (not its mapped form)
 *   staging     device buffer of T*L*H*D*elem_bytes bytes
 */
HFK_API int hfk_fused_memcpy_multi_layer_block_transfer(const void* dev_layer_ptrs,
                                                const void* host_block, void* staging,
                                                uint32_t T, uint32_t L, uint32_t H,
                                                uint32_t D, uint32_t elem_bytes,
                                                uint32_t workgroups, hfk_stream_t stream);

/*
 * The transfer above over a block table, in either direction, all blocks and all
 * layers in one launch:
 *   for j < n_pairs, with (pb, db) = block_pairs[j]:
 *     to_packed == 0:  layer_l[db][(h*T + t)*D + d]  =  packed[pb][((t*L + l)*H + h)*D + d]
 *     to_packed != 0:  packed[pb][((t*L + l)*H + h)*D + d]  =  layer_l[db][(h*T + t)*D + d]
 * where packed[pb] starts at packed_blocks + pb * packed_block_stride and layer_l[db]
 * at dev_layer_ptrs[l] + db * dev_block_stride.
 *
 * Replaces the reference's per-block caller loop around multi_layer_block_transfer
 * (pcieThrough/tests/test_transfer_kernel.py:58-72) with one launch; the
 * to_packed direction (device caches -> packed host blocks) has no counterpart in
 * the reference, whose op is host -> device only
 * (pcieThrough/csrc/kernel/multi_layer_block_transfer_kernel.h:42-72).
 *
 *   dev_layer_ptrs   device-visible array of L uint64 addresses: block 0 of each
 *                    layer's cache [n_dev_blocks][H,T,D]
 *   packed_blocks    device-visible pool of [T,L,H,D] blocks (pinned host memory)
 *   block_pairs      device-visible int64 [n_pairs, 2] = (packed_block, dev_block)
 *   n_packed_blocks, n_dev_blocks  pool sizes; a pair outside them is skipped,
 *                    0 disables that side's check
 *   flags            any combination of HFK_SWAP_BESIDE_COMPUTE (other kernels run meanwhile and matter) and
 *                    one statement about the packed pool, which is the source when to_packed == 0 and
 *                    the destination otherwise: HFK_SWAP_SRC_HOST / HFK_SWAP_DST_HOST (host memory) or
 *                    HFK_SWAP_SRC_DEVICE / HFK_SWAP_DST_DEVICE (device memory); without one the library
 *                    asks the runtime (about 5 us per call). Only the default grid changes (packed
 *                    pool in host memory: 24 workgroups host -> device, 32 device -> host, 16 with
 *                    HFK_SWAP_BESIDE_COMPUTE), never the result.
 * Strides must be at least one block of their side. Destination blocks must be distinct.
 */
HFK_API int hfk_multi_layer_block_table_transfer(const void* dev_layer_ptrs, uint64_t dev_block_stride,
                                         void* packed_blocks, uint64_t packed_block_stride,
                                         const int64_t* block_pairs, uint64_t n_pairs,
                                         uint64_t n_packed_blocks, uint64_t n_dev_blocks,
                                         uint32_t T, uint32_t L, uint32_t H, uint32_t D,
                                         uint32_t elem_bytes, int to_packed, uint32_t flags,
                                         uint32_t workgroups, hfk_stream_t stream);

/*
 * Block-table swap, all planes (layer x K/V) in one launch:
 *   for p < n_planes, j < n_pairs:
 *     copy block_bytes bytes
 *       from src_plane_ptrs[p] + block_pairs[j][0] * src_block_stride
 *       to   dst_plane_ptrs[p] + block_pairs[j][1] * dst_block_stride
 * Direction-agnostic: swap-out passes device planes as src and mapped host planes
 * as dst, swap-in the reverse; device-to-device works the same way.
 *
 * Replaces the caller-side per-block loop of the reference,
 *   pcieThrough/tests/test_transfer_kernel.py:58-72
 * (one op call, one tiling upload and two allocations per block) with a single
 * launch. Equivalent CPU statement, per plane:
 *   dst.index_copy_(0, pairs[:,1], src.index_select(0, pairs[:,0]))
 *
 *   dst_plane_ptrs, src_plane_ptrs  device-visible arrays of n_planes uint64 addresses
 *   block_pairs   device-visible int64 [n_pairs, 2] = (src_block, dst_block)
 *   src_blocks, dst_blocks  blocks per plane on each side; a pair with an index
 *                 outside its range is skipped. 0 disables that side's check.
 *   flags         what the caller knows about the call, any combination of
 *                   HFK_SWAP_DST_HOST        the destination planes are host memory (swap-out)
 *                   HFK_SWAP_SRC_HOST        the source planes are host memory (swap-in)
 *                   HFK_SWAP_BESIDE_COMPUTE  other kernels run at the same time and matter
 *                 0 is always valid. The result never depends on flags; they select the launch
 *                 shape (grid, vectors in flight per lane, pacing). Measured on MI355X, 32 KiB
 *                 blocks, as own rate / slowdown of a 1 GiB device copy / of a bf16 8192^3 GEMM
 *                 running on another stream meanwhile:
 *                 - no flags: 16 workgroups x 8 vectors per lane, 55.4-55.7 GB/s out, 57.0-57.4 in;
 *                   the copy beside it runs 6x slower, the GEMM 4.4x / 1.6x (out / in): what a swap
 *                   holds in flight beyond the link's bandwidth-delay product queues in front of
 *                   every other kernel's traffic.
 *                 - HFK_SWAP_DST_HOST (swap-out): a swap of 64 MiB or more runs on 12 workgroups x 8
 *                   vectors per lane, unpaced, with non-temporal loads and plain stores (through the
 *                   L2, which hands the link whole lines): 56.6-56.7 GB/s on every block table (55.9
 *                   on a slower host), 99 % of what hipMemcpy reaches toward the host / 5.9x / 4.0x. This is the fast shape, not
 *                   the gentle one; the gentle one is asked for with HFK_SWAP_BESIDE_COMPUTE. (Paced
 *                   through HFK_KNOB_THROUGHPUT_PACE_PERMILLE it runs on 6 x 4 with non-temporal stores:
 *                   at 890, 55.5-56.0 GB/s / 1.35x / 2.5x.) A shorter one runs as with no flags.
 *                 - HFK_SWAP_SRC_HOST (swap-in): 40 x 1, unpaced: 57.4 GB/s / 1.95x / 1.6x.
 *                 - with HFK_SWAP_BESIDE_COMPUTE as well: out on 12 x 1 paced at 0.84: 52.8 GB/s / 1.05x /
 *                   1.64x; in on 24 x 1: 55.9 GB/s / 1.30x / 1.58x (1.55-1.6x is what any resident
 *                   kernel costs this GEMM). Name the host side: without it the launch cannot
 *                   pick these shapes (8 x 4 unpaced, 49.8 GB/s toward the host).
 *   workgroups    0 = the default of the mode chosen by flags; otherwise an upper bound on the
 *                 grid. The throughput default is sized for the PCIe link: pass a large bound
 *                 (e.g. 64 per CU) when both sides are device memory.
 * Destination blocks must be distinct (as index_copy_ requires for a
 * deterministic result); source and destination ranges must not overlap.
 */
#define HFK_SWAP_DST_HOST 1u
#define HFK_SWAP_SRC_HOST 2u
#define HFK_SWAP_BESIDE_COMPUTE 4u
#define HFK_SWAP_SRC_DEVICE 8u    /* the source is device memory: for entry points that would otherwise ask the runtime */
#define HFK_SWAP_DST_DEVICE 16u   /* the destination is device memory: likewise */
HFK_API int hfk_swap_blocks(const void* dst_plane_ptrs, const void* src_plane_ptrs,
                    const int64_t* block_pairs, uint32_t n_planes, uint64_t n_pairs,
                    uint64_t block_bytes, uint64_t src_block_stride,
                    uint64_t dst_block_stride, uint64_t src_blocks, uint64_t dst_blocks,
                    uint32_t flags, uint32_t workgroups, hfk_stream_t stream);

/*
 * One side of hfk_swap_blocks_duplex: the arguments of one hfk_swap_blocks call
 * (planes and block size are shared by both sides).
 */
typedef struct hfk_block_move {
    const void* dst_plane_ptrs;   /* device-visible array of n_planes uint64 addresses */
    const void* src_plane_ptrs;
    const int64_t* block_pairs;   /* device-visible int64 [n_pairs, 2] = (src_block, dst_block) */
    uint64_t n_pairs;
    uint64_t src_block_stride;
    uint64_t dst_block_stride;
    uint64_t src_blocks;          /* 0 = unchecked */
    uint64_t dst_blocks;          /* 0 = unchecked */
} hfk_block_move;

/*
 * Two block-table swaps in ONE launch, meant for a swap-out (device -> host) and a
 * swap-in (host -> device) of the same cache running at the same time: the PCIe link
 * is full duplex, and one kernel that keeps both directions in flight in lock step
 * moves more bytes per second than two launches on two streams (which is also a
 * valid way to call hfk_swap_blocks). Result: exactly that of
 *   hfk_swap_blocks(out_move...) and hfk_swap_blocks(in_move...)
 * run in either order. The two moves must not touch the same bytes (no block may
 * be read by one and written by the other); either move may be empty (n_pairs 0).
 * `in_move` should be the one that reads host memory.
 * flags: 0, or HFK_SWAP_BESIDE_COMPUTE (other kernels run meanwhile and matter): 16 workgroups
 * instead of 32, two vectors per lane and direction, and the launch offers the link 0.84 of its raw
 * rate in each direction (see hfk_swap_blocks). The result never depends on flags.
 *
 * No counterpart in the reference (its transfer op is host -> device only and one
 * block per call, pcieThrough/tests/test_transfer_kernel.py:58-72).
 */
HFK_API int hfk_swap_blocks_duplex(const hfk_block_move* out_move, const hfk_block_move* in_move,
                                   uint32_t n_planes, uint64_t block_bytes, uint32_t flags,
                                   uint32_t workgroups, hfk_stream_t stream);

/*
 * Staged block-table swap: the compute units never touch host memory. Blocks travel
 * between the device planes and pinned host planes through a contiguous device
 * staging buffer, the PCIe leg being plain hipMemcpyAsync copies (DMA engines):
 *   to_host != 0: staging[p][i] = dev_plane_p[dev_block_ids[i]]        (one gather kernel)
 *                 host_plane_p[host_block_ids[i]] = staging[p][i]       (copies)
 *   to_host == 0: staging[p][i] = host_plane_p[host_block_ids[i]]      (copies)
 *                 dev_plane_p[dev_block_ids[i]] = staging[p][i]         (one scatter kernel)
 * all on `stream`, in that order. One copy is issued per run of consecutive
 * host_block_ids (a 2-D copy spanning all planes when the host planes are evenly
 * spaced, else one copy per plane), so it is efficient when the host slots of a
 * transfer are (mostly) consecutive: 256 consecutive 32 KiB slots of 64 planes are
 * one 2-D copy of 64 rows of 8 MiB.
 * Result: that of hfk_swap_blocks with the same table, with one exception on the way out (a
 * device id out of range, below); staging holds the moved blocks afterwards.
 *
 * Why it exists: kernels on other streams run within a few per cent of their time alone beside
 * it (GEMM, device copy and attention kernels: 0.98-1.04x on MI355X), because the PCIe leg is
 * DMA and the kernel is short. A swap whose compute units touch host memory costs its neighbours
 * 1.06-1.3x at best (hfk_swap_blocks with HFK_SWAP_BESIDE_COMPUTE) and any long-resident kernel
 * costs a large GEMM about 1.5x whatever it does (the GEMM's workgroups want whole CUs). Use this entry
 * point when the swap overlaps compute and its host slots are mostly consecutive; hfk_swap_blocks
 * when they are scattered, when no staging buffer can be spared, or when the GPU is otherwise idle.
 *
 * Block-table generalisation of the reference's staged variant
 * (pcieThrough/csrc/host/multi_layer_block_transfer_torch.cpp:82-106: memcpy into a
 * device staging block, then a kernel that reads only HBM).
 *
 *   dev_plane_ptrs    device-visible array of n_planes uint64 device addresses
 *   host_plane_addrs  HOST array of n_planes pointers to pinned host planes (host addresses)
 *   dev_block_ids     device-visible int64[n_blocks]
 *   host_block_ids    HOST int64[n_blocks] (read before the call returns)
 *   staging           device buffer of n_planes * n_blocks * block_bytes bytes
 *   dev_blocks / host_blocks  blocks per plane; 0 = unchecked. A host id out of range
 *                     rejects the call (HFK_ERR_OUT_OF_RANGE) before anything is enqueued.
 *                     A device id out of range: on the way in the block is skipped, as
 *                     everywhere else. On the way out the ids live on the device, so the
 *                     copies cannot skip the entry; the kernel writes zeros to staging[p][i]
 *                     instead and the host slot receives zeros (hfk_swap_blocks would leave
 *                     the slot untouched). Bytes of an earlier transfer never reach the host.
 */
HFK_API int hfk_swap_blocks_staged(const void* dev_plane_ptrs, void* const* host_plane_addrs,
                                   const int64_t* dev_block_ids, const int64_t* host_block_ids,
                                   uint32_t n_planes, uint64_t n_blocks, uint64_t block_bytes,
                                   uint64_t dev_block_stride, uint64_t host_block_stride,
                                   uint64_t dev_blocks, uint64_t host_blocks, void* staging,
                                   int to_host, uint32_t workgroups, hfk_stream_t stream);

/*
 * hfk_swap_blocks_staged without the staging argument and without any allocation: the staging
 * buffer is an array of HFK_STATIC_STAGING_BYTES bytes that lives in the library's device image
 * (one copy per GPU the library is used on, held until the process ends).
 *
 * No counterpart in the reference. It is for callers that cannot allocate or cannot keep a
 * workspace alive: code that runs under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc. The call itself makes no hipMalloc / hipFree and calls no routine that does.
 *
 *   - n_planes * n_blocks * block_bytes must not exceed HFK_STATIC_STAGING_BYTES, else
 *     HFK_ERR_STAGING_TOO_SMALL and nothing is enqueued.
 *   - Every call on one GPU uses the same array: calls that overlap in time on one GPU (two
 *     streams, two threads) would race on it. Calls on one stream are ordered and safe. A call that
 *     arrives on another stream while the previous static call's work is still pending is refused
 *     with HFK_ERR_STAGING_BUSY and enqueues nothing (the library keeps one event per device for
 *     this, created on the first call: no device memory). What the library cannot see it cannot
 *     refuse: replays of a captured graph that holds a static call, and calls from other processes'
 *     copies of the library (each process has its own array), are the caller's to order.
 *   - The array is part of the library's device image: every process that loads the library holds
 *     HFK_STATIC_STAGING_BYTES of device memory on every GPU it uses, whether or not it ever calls this.
 *   - The array keeps the last call's blocks; nothing needs clearing between calls (every staging
 *     byte that reaches a destination was written by the same call first).
 *   - The first call on a device asks the runtime for that device's address of the array; make it
 *     before a graph capture begins, not inside one.
 * Everything else (arguments, order of operations, result) as hfk_swap_blocks_staged.
 */
#define HFK_STATIC_STAGING_BYTES (64ull << 20)
HFK_API int hfk_swap_blocks_staged_static(const void* dev_plane_ptrs, void* const* host_plane_addrs,
                                          const int64_t* dev_block_ids, const int64_t* host_block_ids,
                                          uint32_t n_planes, uint64_t n_blocks, uint64_t block_bytes,
                                          uint64_t dev_block_stride, uint64_t host_block_stride,
                                          uint64_t dev_blocks, uint64_t host_blocks, int to_host,
                                          uint32_t workgroups, hfk_stream_t stream);

/*
 * Block-table swap that chooses the mover per run of host slots: the selection between the direct
 * and the staged path that the reference leaves to its caller (its two ops
 * multi_layer_block_transfer / fused_memcpy_multi_layer_block_transfer,
 * pcieThrough/csrc/host/multi_layer_block_transfer_torch.cpp:58-106, and the crossover its README
 * measures, pcieThrough/tests/README.md:72-75), made per call and per run here.
 *
 *   - Runs of at least k consecutive host slots go the staged way: HBM gather/scatter kernel +
 *     one 2-D DMA copy per run. Kernels on other streams do not notice them.
 *   - Everything else goes the direct way, in one launch of the block-swap kernel that steps over
 *     the pairs the copy engines took.
 *   - With no staging buffer, no host arrays, or a buffer too small for what would be staged, the
 *     whole table goes the direct way: as hfk_swap_blocks with the host side named, except that a
 *     device id out of range zero-fills its host slot on the way out.
 * k = min_run_blocks, or when that is 0 the smallest run whose single copy moves 16 MiB, with
 * HFK_SWAP_BESIDE_COMPUTE 4 MiB. A copy costs the DMA engines about 9.5 us before its first byte, the
 * link time of 0.5 MiB: runs of 16 MiB move at 97 % of the link rate, runs of 4 MiB at 88 %, single
 * 2 MiB slots at 80 %. A swap that owns the GPU therefore keeps short runs on the compute units
 * (k = 8 for 64 evenly spaced planes of 32 KiB blocks), one that shares it pays some of its own rate to
 * keep the compute units off host memory (k = 2). min_run_blocks = 1 stages everything
 * (hfk_swap_blocks_staged), above 1024 nothing.
 *
 *   dev_plane_ptrs    device-visible array of n_planes uint64 device addresses
 *   host_plane_ptrs   device-visible array of n_planes uint64 mapped host addresses (direct mover)
 *   host_plane_addrs  HOST array of n_planes host addresses of the same planes (copy engines); may be NULL
 *   block_pairs       device-visible int64 [n_pairs, 2] = (src_block, dst_block):
 *                     (device, host) when to_host != 0, (host, device) otherwise
 *   host_block_ids    HOST int64 [n_pairs]: the host column of block_pairs, read before the call
 *                     returns; may be NULL. It must equal that column. The copy engines pick their
 *                     runs from this array, the kernels theirs from block_pairs: where the two
 *                     disagree blocks end up unmoved or moved twice, and a pair the array calls part
 *                     of a long run but the table does not is copied from a staging slot this call
 *                     never filled, so stale bytes of an earlier transfer reach the named host slot
 *                     (never anything outside the pools: both movers are range-checked). Setting
 *                     HFK_KNOB_CHECK_HOST_COLUMN makes the call compare the two first (it waits for
 *                     `stream` and reads the table back: for debugging, not for production) and
 *                     return HFK_ERR_TABLE_MISMATCH, with nothing enqueued, if they differ.
 *   dev_blocks / host_blocks  blocks per plane; 0 = unchecked. With host arrays present, a host id
 *                     out of range rejects the call (HFK_ERR_OUT_OF_RANGE) before anything is
 *                     enqueued. A device id out of range: skipped on the way in; on the way out
 *                     its host slot receives zeros, whichever mover had the pair.
 *   staging           device buffer (256-byte aligned), or NULL; staging_bytes its size.
 *                     n_planes * n_pairs * block_bytes always suffices. A smaller buffer is used when
 *                     it holds the staged share alone: n_planes * (blocks in runs of k or more) *
 *                     block_bytes, rounded up to 256, plus 16 bytes per pair for the two lists of pairs
 *                     (those in long runs, and the others) that a one-workgroup kernel of the same call
 *                     writes from block_pairs and the call's other launches are handed. A buffer with
 *                     room for both is used that way even if it could hold the whole table
 *   flags             0 or HFK_SWAP_BESIDE_COMPUTE (shape of the direct launch, see hfk_swap_blocks;
 *                     the host side is named by to_host)
 * All work is enqueued on `stream` in order. Destination blocks must be distinct.
 */
HFK_API int hfk_swap_blocks_auto(const void* dev_plane_ptrs, const void* host_plane_ptrs,
                                 void* const* host_plane_addrs, const int64_t* block_pairs,
                                 const int64_t* host_block_ids, uint32_t n_planes, uint64_t n_pairs,
                                 uint64_t block_bytes, uint64_t dev_block_stride,
                                 uint64_t host_block_stride, uint64_t dev_blocks, uint64_t host_blocks,
                                 void* staging, uint64_t staging_bytes, int to_host,
                                 uint32_t min_run_blocks, uint32_t flags, hfk_stream_t stream);

/*
 * Paged block gather over many planes in one launch:
 *   for p < n_planes, i < n_ids:
 *     dst_plane_ptrs[p][i*block_bytes ...] = src_plane_ptrs[p][ids[i]*src_block_stride ...]
 * i.e. hfk_gather_rows applied to every plane with a shared id list
 * (per plane: dst = src.index_select(0, ids)).
 * Same reference anchors as hfk_gather_rows; the plane loop is additive.
 *   flags  0 = source planes in device memory (grid of one workgroup per chunk, HBM-bound).
 *          HFK_SWAP_SRC_HOST = the source planes are host memory: the gather is then a swap-in with
 *          consecutive destinations and gets that launch shape (40 workgroups of one vector per
 *          lane); with HFK_SWAP_BESIDE_COMPUTE as well, 24. The result never depends on flags.
 */
HFK_API int hfk_gather_blocks(const void* dst_plane_ptrs, const void* src_plane_ptrs,
                      const int64_t* ids, uint32_t n_planes, uint64_t n_ids,
                      uint64_t block_bytes, uint64_t src_block_stride,
                      uint64_t src_blocks, uint32_t flags, uint32_t workgroups,
                      hfk_stream_t stream);

/*
 * Tuning knobs. Defaults are the measured best for MI355X. hfk_set_tuning changes a knob for the whole
 * process (every thread, every later call); hfk_thread_tuning_begin / _end change knobs for the calls
 * the calling thread makes in between and touch nothing another thread can see: that is the way to
 * give one call, or one engine thread, a launch shape of its own.
 */
enum hfk_knob {
    HFK_KNOB_UNROLL = 0,        /* 16-byte accesses in flight per lane of the HBM-bound launches
                                   (gathers, staged swap's kernel): 1 (default), 2, 4, 8, 16 */
    HFK_KNOB_NONTEMPORAL = 1,   /* bit0: non-temporal loads, bit1: non-temporal stores */
    HFK_KNOB_WORKGROUPS_PER_CU = 2, /* default grid bound of the gathers and the
                                       transfer = CUs * this, 1..65536 (default 65536)  */
    HFK_KNOB_SWAP_WORKGROUPS = 3,   /* default grid bound of hfk_swap_blocks           */
    HFK_KNOB_DUPLEX_UNROLL = 4,     /* like HFK_KNOB_UNROLL, for hfk_swap_blocks_duplex */
    HFK_KNOB_SWAP_UNROLL = 5,       /* like HFK_KNOB_UNROLL, for hfk_swap_blocks (throughput mode) */
    HFK_KNOB_SWAP_PACE_MBPS = 6,    /* rate a HFK_SWAP_BESIDE_COMPUTE swap offers toward the host, MB/s;
                                       0 (default) = 84 % of HFK_KNOB_LINK_MBPS               */
    HFK_KNOB_LINK_MBPS = 7,         /* raw rate of the current device's PCIe link, MB/s. Default: lanes x
                                       GT/s x line encoding, the larger of the link's current and its maximum
                                       rate as sysfs shows them (0 if unreadable: such swaps then run
                                       unpaced). Setting it overrides every device; -1 restores the default */
    HFK_KNOB_DUPLEX_WORKGROUPS = 8, /* default grid bound of hfk_swap_blocks_duplex                       */
    HFK_KNOB_THROUGHPUT_PACE_PERMILLE = 9, /* share of HFK_KNOB_LINK_MBPS, in thousandths, that a swap-out of
                                       64 MiB or more offers toward a named host side when it is not marked
                                       HFK_SWAP_BESIDE_COMPUTE. Default 0 = unpaced: 12 workgroups x 8 vectors
                                       per lane with plain stores, the fastest shape and the one whose rate does
                                       not depend on a clock; paced, HFK_KNOB_PACED_WORKGROUPS x
                                       HFK_KNOB_PACED_UNROLL vectors per lane in flight with non-temporal stores,
                                       gentler on kernels that run beside it (a device copy 1.3x slower instead of
                                       5.5x), at 98.5-99.5 % of the unpaced rate once HFK_KNOB_ADAPTIVE_PACE has
                                       had ten or so launches to settle the pace                            */
    HFK_KNOB_HBM_LDS_BYTES = 10,    /* dynamic LDS, 0..65536 bytes, that the HBM-bound launches (gathers, the
                                       staged swap's kernel) request without using it: with 160 KiB of LDS
                                       per compute unit it bounds the workgroups a unit holds at a time   */
    HFK_KNOB_PACED_UNROLL = 11,     /* like HFK_KNOB_UNROLL, for the paced throughput-mode swap toward the host */
    HFK_KNOB_PACED_WORKGROUPS = 12, /* default grid of that swap (hfk_swap_blocks with HFK_SWAP_DST_HOST alone) */
    HFK_KNOB_PACE_REPORT = 13,      /* diagnostic, default 0 = off: device-visible address of 8 x grid 64-bit
                                       words. Every workgroup b of a paced hfk_swap_blocks launch writes, when
                                       it has finished, at word 8 * b: ticks of the 100 MHz counter it ran,
                                       ticks its schedule allotted, turns taken, turns that began behind
                                       schedule, largest delay behind schedule in ticks, the pacing interval in
                                       1/256 ticks, and two zeros. ran > allotted means the launch could not
                                       hold its pace. The buffer must hold 64 bytes per workgroup launched     */
    HFK_KNOB_DUPLEX_PACE_PERMILLE = 14, /* share of HFK_KNOB_LINK_MBPS, in thousandths, that a duplex swap of 64 MiB
                                       or more toward the host offers in that direction when it is not marked
                                       HFK_SWAP_BESIDE_COMPUTE; 0 = unpaced; default 890                        */
    HFK_KNOB_TRANSFER_PACE_PERMILLE = 15, /* the same for a block-table transfer into a packed pool in host
                                       memory; 0 (default) = unpaced                                            */
    HFK_KNOB_TRANSFER_UNROLL = 16,  /* 16-byte units per lane of that transfer, 2 or 8 (default 8)              */
    HFK_KNOB_CHECK_HOST_COLUMN = 17, /* debugging aid, default 0: hfk_swap_blocks_auto first waits for its stream,
                                       reads block_pairs back and compares its host column with host_block_ids;
                                       a difference rejects the call with HFK_ERR_TABLE_MISMATCH                */
    HFK_KNOB_TRANSFER_TILED = 18,   /* 1 (default): a block-table transfer into a packed pool in host memory goes through
                                       LDS tiles where its geometry allows (1 KiB runs on both sides); 0: always
                                       row by row                                                               */
    HFK_KNOB_ADAPTIVE_PACE = 19,    /* 1 (default): a paced throughput-mode swap-out (HFK_KNOB_THROUGHPUT_PACE_PERMILLE != 0)
                                       takes its interval times a factor that the paced launches before it on this
                                       device have settled (see hfk_pace_state); 0: the interval as computed        */
    HFK_KNOB_FUSED_COPY_ENGINE = 20 /* 0 (default): hfk_fused_memcpy_multi_layer_block_transfer reads a block in pinned
                                       host memory once, by the kernel, which fills the staging buffer as well;
                                       1: hipMemcpyAsync into staging, then the kernel, as for pageable memory     */
};
/*
 * The state behind a pace that is set between launches, for the current device: eight words,
 * [0] the factor applied to the interval of the next paced throughput-mode swap-out, in 1/65536
 * (0 = none settled yet, i.e. 1.0; kept within 0.93 .. 1.04), [1]-[4] the account of a launch in
 * progress, [5] launches settled, [6] late turns per 65536 turns of the last one, [7] unused.
 * Every such launch ends by settling the factor for the next one from how many of its turns began
 * late and whether a workgroup ended behind its schedule: the pace follows what this machine's link
 * takes instead of what its nominal rate and a nominal 100 MHz say. Diagnostic: waits for the device.
 * No counterpart in the reference.
 */
HFK_API int hfk_pace_state(uint32_t* out8);

HFK_API int hfk_set_tuning(int knob, int64_t value);
HFK_API int64_t hfk_get_tuning(int knob);

/*
 * Knob values for the calling thread only. From hfk_thread_tuning_begin until hfk_thread_tuning_end
 * every hfk_* call made by this thread reads the listed knobs from `overrides` and every other knob
 * from the process-wide values; other threads see no change. A second begin replaces the first
 * (there is no nesting). A list with an unknown knob or an invalid value is rejected as a whole
 * (HFK_ERR_BAD_KNOB) and leaves the thread's overrides as they were. hfk_get_tuning shows the
 * calling thread's view. No counterpart in the reference, whose only tunable is the aivNum argument
 * of its ops (pcieThrough/csrc/host/gather_torch.cpp:32-36), passed per call.
 */
typedef struct hfk_knob_value {
    int knob;       /* enum hfk_knob */
    int64_t value;
} hfk_knob_value;
HFK_API int hfk_thread_tuning_begin(const hfk_knob_value* overrides, uint32_t n);
HFK_API void hfk_thread_tuning_end(void);

#ifdef __cplusplus
}
#endif
#endif /* HFK_H */
