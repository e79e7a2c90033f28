/*
 * hfk_oracle.c - CPU restatement of the reference's pcieThrough data movement.
 *
 * TEST INFRASTRUCTURE ONLY. This file is the checker the HIP kernels are compared
 * against; nothing that ships (the package, the torch extension, libhfk_hip.so)
 * may link, load or call it. Only tests/, the smoke check and the benchmark's CPU
 * baseline leg use it.
 *
 * The reference kernels are AscendC and cannot be compiled without the CANN
 * toolkit, so each function restates the reference's algorithm in plain C,
 * keeping the reference's own work split (per-core id / token ranges) so that a
 * mistake in reading the split would show up as a wrong result, and cites the
 * lines it follows. Paths are relative to the reference tree root.
 *
 * How each function is pinned (see tests/test_oracle.py): against the reference
 * tests' own expected-value expressions (permute-compare, row-by-row verify),
 * against closed forms (identity ids and L = H = 1 reduce to memcpy), against an
 * independent pure-Python brute force on tiny shapes, against the torch CPU
 * index_select / index_copy_ statement, and against the committed golden vectors
 * under tests/golden/.
 */
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/*
 * Row gather, dst[i,:] = table[ids[i],:].
 *
 * Follows pcieThrough/csrc/kernel/gather.h:
 *   :45-52   ids are split over `cores` blocks: base = n/cores, the first
 *            (n % cores) blocks take one more; block b starts at
 *            b*base + min(b, n % cores)
 *   :106-112 one row copy per id, source row = ids[i] * row elements
 *   :119-122 rows land contiguously at dst[(first + i) * row elements]
 * The rounds/UB buffering of :85-133 does not change which bytes move.
 * Host op: pcieThrough/csrc/host/gather_torch.cpp:30-54 (cores = min(aiv, n), :48).
 *
 * Returns 0, or -1 on bad arguments.
 */
ORACLE_API int oracle_gather_rows(const void* table, void* dst, const void* ids, int ids_are_i64,
                                  uint64_t n_ids, uint64_t row_bytes, uint32_t cores) {
    if (n_ids == 0) return 0;
    if (!table || !dst || !ids || row_bytes == 0 || cores == 0) return -1;
    if (cores > n_ids) cores = (uint32_t)n_ids; /* gather_torch.cpp:48 */
    const uint64_t base = n_ids / cores;
    const uint64_t rem = n_ids % cores;
    for (uint32_t b = 0; b < cores; ++b) {
        const uint64_t n_this = base + (b < rem ? 1 : 0);
        const uint64_t first = (uint64_t)b * base + (b < rem ? b : rem);
        for (uint64_t i = 0; i < n_this; ++i) {
            const int64_t id = ids_are_i64 ? ((const int64_t*)ids)[first + i]
                                           : (int64_t)((const int32_t*)ids)[first + i];
            memcpy((char*)dst + (first + i) * row_bytes, (const char*)table + (uint64_t)id * row_bytes,
                   row_bytes);
        }
    }
    return 0;
}

/*
 * One KV block, all layers, host layout [T,L,H,D] -> per-layer [H,T,D]:
 *   layer[l][(h*T + t)*D + d] = src[((t*L + l)*H + h)*D + d]
 *
 * Follows pcieThrough/csrc/kernel/multi_layer_block_transfer_kernel.h:
 *   :74-82  core c handles tokens [c*tokensPerCore, min(T, (c+1)*tokensPerCore))
 *   :47     a token starts at t*L*H*D in the source
 *   :60-67  for each (layer, head): source offset l*H*D + h*D inside the token,
 *           destination offset h*T*D + t*D inside the layer buffer, D elements
 * and pcieThrough/csrc/host/tiling/multi_layer_block_transfer.cpp:34
 * (tokensPerCore = ceil(T / aiv)). The inner-loop token batching (:35-46 of the
 * tiling, :78-81 of the kernel) only groups tokens and moves the same bytes.
 */
ORACLE_API int oracle_multi_layer_block_transfer(void* const* layer_ptrs, const void* src, uint32_t T,
                                                 uint32_t L, uint32_t H, uint32_t D, uint32_t elem_bytes,
                                                 uint32_t cores) {
    if (!layer_ptrs || !src || elem_bytes == 0 || cores == 0) return -1;
    const uint64_t row = (uint64_t)D * elem_bytes;
    const uint32_t tokens_per_core = (T + cores - 1) / cores;
    for (uint32_t c = 0; c < cores; ++c) {
        const uint64_t t0 = (uint64_t)c * tokens_per_core;
        uint64_t t1 = t0 + tokens_per_core;
        if (t1 > T) t1 = T;
        for (uint64_t t = t0; t < t1; ++t) {
            const char* token = (const char*)src + t * L * H * row;
            for (uint32_t l = 0; l < L; ++l) {
                char* layer = (char*)layer_ptrs[l];
                for (uint32_t h = 0; h < H; ++h) {
                    memcpy(layer + ((uint64_t)h * T + t) * row, token + ((uint64_t)l * H + h) * row, row);
                }
            }
        }
    }
    return 0;
}

/*
 * The transfer above over a block table: for each pair (packed block pb, layered
 * block db) either the reference's host -> device conversion (to_packed == 0), which
 * restates the caller loop pcieThrough/tests/test_transfer_kernel.py:58-72 (one
 * multi_layer_block_transfer per block, per-block pointer tables :42-47), or its
 * inverse (to_packed != 0): packed[pb][((t*L + l)*H + h)*D + d] = layer_l[db][(h*T + t)*D + d].
 * The inverse has no counterpart in the reference; it is pinned as the exact inverse
 * of the forward direction and by brute force.
 */
ORACLE_API int oracle_multi_layer_block_table_transfer(void* const* layer_ptrs, uint64_t layered_stride,
                                                       void* packed, uint64_t packed_stride,
                                                       const int64_t* pairs, uint64_t n_pairs, uint32_t T,
                                                       uint32_t L, uint32_t H, uint32_t D, uint32_t elem_bytes,
                                                       int to_packed, uint32_t cores) {
    if (n_pairs == 0) return 0;
    if (!layer_ptrs || !packed || !pairs || elem_bytes == 0 || cores == 0) return -1;
    void** block_layers = (void**)malloc(sizeof(void*) * (L ? L : 1));
    if (!block_layers) return -2;
    const uint64_t row = (uint64_t)D * elem_bytes;
    for (uint64_t j = 0; j < n_pairs; ++j) {
        char* pblock = (char*)packed + (uint64_t)pairs[2 * j] * packed_stride;
        for (uint32_t l = 0; l < L; ++l) {
            block_layers[l] = (char*)layer_ptrs[l] + (uint64_t)pairs[2 * j + 1] * layered_stride;
        }
        if (!to_packed) {
            int rc = oracle_multi_layer_block_transfer(block_layers, pblock, T, L, H, D, elem_bytes, cores);
            if (rc != 0) {
                free(block_layers);
                return rc;
            }
        } else {
            for (uint64_t t = 0; t < T; ++t)
                for (uint32_t l = 0; l < L; ++l)
                    for (uint32_t h = 0; h < H; ++h)
                        memcpy(pblock + ((t * L + l) * H + h) * row,
                               (const char*)block_layers[l] + ((uint64_t)h * T + t) * row, row);
        }
    }
    free(block_layers);
    return 0;
}

/*
 * Block-table swap over planes: per plane
 *   dst.index_copy_(0, pairs[:,1], src.index_select(0, pairs[:,0]))
 * i.e. first gather the source blocks into a temporary, then scatter them.
 *
 * The reference has no such op; its block table is the caller's loop
 * pcieThrough/tests/test_transfer_kernel.py:58-72 (one transfer per block),
 * which this restates for blocks of identical layout on both sides.
 */
ORACLE_API int oracle_swap_blocks(void* const* dst_planes, const void* const* src_planes,
                                  const int64_t* pairs, uint32_t n_planes, uint64_t n_pairs,
                                  uint64_t block_bytes, uint64_t src_stride, uint64_t dst_stride) {
    if (n_planes == 0 || n_pairs == 0) return 0;
    if (!dst_planes || !src_planes || !pairs || block_bytes == 0) return -1;
    char* tmp = (char*)malloc((size_t)(n_pairs * block_bytes));
    if (!tmp) return -2;
    for (uint32_t p = 0; p < n_planes; ++p) {
        for (uint64_t j = 0; j < n_pairs; ++j) { /* index_select */
            memcpy(tmp + j * block_bytes, (const char*)src_planes[p] + (uint64_t)pairs[2 * j] * src_stride,
                   block_bytes);
        }
        for (uint64_t j = 0; j < n_pairs; ++j) { /* index_copy_ */
            memcpy((char*)dst_planes[p] + (uint64_t)pairs[2 * j + 1] * dst_stride, tmp + j * block_bytes,
                   block_bytes);
        }
    }
    free(tmp);
    return 0;
}
