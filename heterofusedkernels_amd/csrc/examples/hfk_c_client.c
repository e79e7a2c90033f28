/*
 * hfk_c_client.c - a foreign runtime's view of the library: plain C99, only
 * include/hfk.h, include/hfk_managed_memory.h and the HIP runtime's C API.
 *
 * It plays the swap path of a paged KV cache end to end without Python or torch:
 *   1. pinned, device-mapped host planes from hfk_mm_alloc_pinned,
 *   2. device planes from hipMalloc, filled with a position-dependent pattern,
 *   3. swap-out of a shuffled block table (hfk_swap_blocks, device -> host),
 *   4. swap-in of those blocks to other device blocks (host -> device),
 *   5. the same blocks through the staged path (hfk_swap_blocks_staged),
 *   6. a row gather out of the host planes (hfk_gather_rows),
 * checking every byte after each step against the pattern it must hold.
 *
 * Usage: hfk_c_client [planes blocks block_bytes n_pairs]    (defaults 8 64 32768 24)
 * Exit status 0 and a final line "hfk_c_client: OK" on success.
 */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "hfk.h"
#include "hfk_managed_memory.h"

#define CHECK_HIP(call)                                                                    \
    do {                                                                                   \
        hipError_t e_ = (call);                                                            \
        if (e_ != hipSuccess) {                                                            \
            fprintf(stderr, "%s:%d %s -> %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
            return 2;                                                                      \
        }                                                                                  \
    } while (0)

#define CHECK_HFK(call)                                                                    \
    do {                                                                                   \
        int s_ = (call);                                                                   \
        if (s_ != 0) {                                                                     \
            fprintf(stderr, "%s:%d %s -> %d (%s)\n", __FILE__, __LINE__, #call, s_, hfk_status_string(s_)); \
            return 3;                                                                      \
        }                                                                                  \
    } while (0)

/* The byte every position of the device cache starts with. */
static uint8_t pattern(uint32_t plane, uint64_t block, uint64_t offset) {
    uint64_t x = ((uint64_t)plane * 1000003u + block) * 2654435761u + offset * 40503u;
    x ^= x >> 29;
    return (uint8_t)(x * 0x9E3779B97F4A7C15ull >> 56);
}

/* xorshift permutation of [0, n) */
static void shuffle(int64_t* v, uint64_t n, uint64_t seed) {
    uint64_t i, s = seed * 0x9E3779B97F4A7C15ull + 1;
    for (i = 0; i < n; ++i) v[i] = (int64_t)i;
    for (i = n; i > 1; --i) {
        uint64_t j;
        int64_t t;
        s ^= s << 13; s ^= s >> 7; s ^= s << 17;
        j = s % i;
        t = v[i - 1]; v[i - 1] = v[j]; v[j] = t;
    }
}

static int expect_block(const uint8_t* got, uint32_t plane, uint64_t src_block, uint64_t bytes, const char* what,
                        uint64_t where) {
    uint64_t o;
    for (o = 0; o < bytes; ++o) {
        if (got[o] != pattern(plane, src_block, o)) {
            fprintf(stderr, "MISMATCH %s: plane %u slot %llu byte %llu: got %u want %u\n", what, plane,
                    (unsigned long long)where, (unsigned long long)o, got[o], pattern(plane, src_block, o));
            return 1;
        }
    }
    return 0;
}

int main(int argc, char** argv) {
    uint32_t planes = argc > 1 ? (uint32_t)strtoul(argv[1], NULL, 0) : 8;
    uint64_t blocks = argc > 2 ? strtoull(argv[2], NULL, 0) : 64;
    uint64_t bb = argc > 3 ? strtoull(argv[3], NULL, 0) : 32768;
    uint64_t n = argc > 4 ? strtoull(argv[4], NULL, 0) : 24;
    uint64_t plane_bytes = blocks * bb, i, o;
    uint32_t p;
    void** dev_plane;
    void** host_plane;
    uint64_t *dev_tab_h, *host_tab_h;
    void *dev_tab, *host_tab, *pairs_d, *ids_d, *staging, *rows_d;
    int64_t *perm_a, *perm_b, *pairs_h, *host_ids;
    uint8_t* scratch;
    hipStream_t stream;
    int node = -1;

    if (planes == 0 || blocks < 4 || bb == 0 || n == 0 || 2 * n > blocks) {
        fprintf(stderr, "need planes > 0, block_bytes > 0 and 0 < 2 * n_pairs <= blocks\n");
        return 1;
    }
    printf("hfk_c_client: library %d, %u planes x %llu blocks x %llu B, %llu pairs\n", hfk_version(), planes,
           (unsigned long long)blocks, (unsigned long long)bb, (unsigned long long)n);
    fflush(stdout);

    CHECK_HIP(hipSetDevice(0));
    CHECK_HIP(hipStreamCreate(&stream));
    CHECK_HFK(hfk_mm_device_numa_node(0, &node));

    dev_plane = (void**)calloc(planes, sizeof(void*));
    host_plane = (void**)calloc(planes, sizeof(void*));
    dev_tab_h = (uint64_t*)calloc(planes, sizeof(uint64_t));
    host_tab_h = (uint64_t*)calloc(planes, sizeof(uint64_t));
    scratch = (uint8_t*)malloc(plane_bytes);
    perm_a = (int64_t*)malloc(blocks * sizeof(int64_t));
    perm_b = (int64_t*)malloc(blocks * sizeof(int64_t));
    pairs_h = (int64_t*)malloc(2 * n * sizeof(int64_t));
    host_ids = (int64_t*)malloc(n * sizeof(int64_t));
    if (!dev_plane || !host_plane || !dev_tab_h || !host_tab_h || !scratch || !perm_a || !perm_b || !pairs_h || !host_ids)
        return 1;

    /* 1 + 2: the two caches and their pointer tables */
    for (p = 0; p < planes; ++p) {
        CHECK_HFK(hfk_mm_alloc_pinned(plane_bytes, node, 0, &host_plane[p]));
        CHECK_HIP(hipMalloc(&dev_plane[p], plane_bytes));
        for (i = 0; i < blocks; ++i)
            for (o = 0; o < bb; ++o) scratch[i * bb + o] = pattern(p, i, o);
        CHECK_HIP(hipMemcpy(dev_plane[p], scratch, plane_bytes, hipMemcpyHostToDevice));
        dev_tab_h[p] = (uint64_t)(uintptr_t)dev_plane[p];
        host_tab_h[p] = (uint64_t)(uintptr_t)hfk_mm_get_device_ptr(host_plane[p]);   /* mapped address */
        if (host_tab_h[p] == 0) { fprintf(stderr, "registry does not know plane %u\n", p); return 1; }
    }
    CHECK_HIP(hipMalloc(&dev_tab, planes * sizeof(uint64_t)));
    CHECK_HIP(hipMalloc(&host_tab, planes * sizeof(uint64_t)));
    CHECK_HIP(hipMalloc(&pairs_d, 2 * n * sizeof(int64_t)));
    CHECK_HIP(hipMalloc(&ids_d, n * sizeof(int64_t)));
    CHECK_HIP(hipMalloc(&staging, planes * n * bb));
    CHECK_HIP(hipMalloc(&rows_d, n * bb));
    CHECK_HIP(hipMemcpy(dev_tab, dev_tab_h, planes * sizeof(uint64_t), hipMemcpyHostToDevice));
    CHECK_HIP(hipMemcpy(host_tab, host_tab_h, planes * sizeof(uint64_t), hipMemcpyHostToDevice));

    /* 3: swap-out, device block perm_a[i] -> host slot perm_b[i], i < n */
    shuffle(perm_a, blocks, 1);
    shuffle(perm_b, blocks, 2);
    for (i = 0; i < n; ++i) { pairs_h[2 * i] = perm_a[i]; pairs_h[2 * i + 1] = perm_b[i]; }
    CHECK_HIP(hipMemcpy(pairs_d, pairs_h, 2 * n * sizeof(int64_t), hipMemcpyHostToDevice));
    printf("step swap-out\n"); fflush(stdout);
    CHECK_HFK(hfk_swap_blocks(host_tab, dev_tab, (const int64_t*)pairs_d, planes, n, bb, bb, bb, blocks, blocks, 0, 0, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    for (p = 0; p < planes; ++p) {
        const uint8_t* h = (const uint8_t*)host_plane[p];
        for (i = 0; i < n; ++i)
            if (expect_block(h + (uint64_t)perm_b[i] * bb, p, (uint64_t)perm_a[i], bb, "swap-out", (uint64_t)perm_b[i])) return 4;
        for (i = n; i < blocks; ++i)                         /* untouched slots stay zero */
            for (o = 0; o < bb; ++o)
                if (h[(uint64_t)perm_b[i] * bb + o] != 0) { fprintf(stderr, "swap-out wrote slot %lld\n", (long long)perm_b[i]); return 4; }
    }

    /* 4: swap-in, host slot perm_b[i] -> device block perm_a[n + i] (a block not swapped out) */
    for (i = 0; i < n; ++i) { pairs_h[2 * i] = perm_b[i]; pairs_h[2 * i + 1] = perm_a[n + i]; }
    CHECK_HIP(hipMemcpy(pairs_d, pairs_h, 2 * n * sizeof(int64_t), hipMemcpyHostToDevice));
    printf("step swap-in\n"); fflush(stdout);
    CHECK_HFK(hfk_swap_blocks(dev_tab, host_tab, (const int64_t*)pairs_d, planes, n, bb, bb, bb, blocks, blocks,
                              HFK_SWAP_SRC_HOST | HFK_SWAP_BESIDE_COMPUTE, 0, stream));   /* the gentle launch shape: same bytes */
    CHECK_HIP(hipStreamSynchronize(stream));
    for (p = 0; p < planes; ++p) {
        CHECK_HIP(hipMemcpy(scratch, dev_plane[p], plane_bytes, hipMemcpyDeviceToHost));
        for (i = 0; i < blocks; ++i) {
            uint64_t blk = (uint64_t)perm_a[i];
            uint64_t holds = (i >= n && i < 2 * n) ? (uint64_t)perm_a[i - n] : blk;   /* swapped-in blocks hold their source */
            if (expect_block(scratch + blk * bb, p, holds, bb, "swap-in", blk)) return 5;
        }
    }

    /* 5: staged swap-out of the swapped-in blocks to consecutive host slots the first swap left empty */
    {
        uint64_t run = 0, best = 0, best_start = 0, start = 0;
        uint8_t* used = (uint8_t*)calloc(blocks, 1);
        if (!used) return 1;
        for (i = 0; i < n; ++i) used[perm_b[i]] = 1;
        for (i = 0; i < blocks; ++i) {
            if (used[i]) { run = 0; start = i + 1; continue; }
            if (++run > best) { best = run; best_start = start; }
        }
        free(used);
        if (best > n) best = n;
        for (i = 0; i < best; ++i) host_ids[i] = (int64_t)(best_start + i);
        for (i = 0; i < best; ++i) pairs_h[i] = perm_a[n + i];          /* device ids */
        CHECK_HIP(hipMemcpy(ids_d, pairs_h, best * sizeof(int64_t), hipMemcpyHostToDevice));
        printf("step staged swap-out (%llu consecutive host slots from %llu)\n", (unsigned long long)best,
               (unsigned long long)best_start);
        fflush(stdout);
        CHECK_HFK(hfk_swap_blocks_staged(dev_tab, host_plane, (const int64_t*)ids_d, host_ids, planes, best, bb, bb, bb,
                                         blocks, blocks, staging, 1, 0, stream));
        CHECK_HIP(hipStreamSynchronize(stream));
        for (p = 0; p < planes; ++p)
            for (i = 0; i < best; ++i)
                if (expect_block((const uint8_t*)host_plane[p] + (best_start + i) * bb, p, (uint64_t)perm_a[i], bb,
                                 "staged swap-out", best_start + i)) return 6;
    }

    /* 6: row gather straight out of host plane 0: rows = the n slots of the first swap, in reverse order */
    for (i = 0; i < n; ++i) pairs_h[i] = perm_b[n - 1 - i];
    CHECK_HIP(hipMemcpy(ids_d, pairs_h, n * sizeof(int64_t), hipMemcpyHostToDevice));
    printf("step gather\n"); fflush(stdout);
    CHECK_HFK(hfk_gather_rows((const void*)(uintptr_t)host_tab_h[0], rows_d, ids_d, 1, n, bb, blocks, HFK_SWAP_SRC_HOST, 0, stream));
    CHECK_HIP(hipStreamSynchronize(stream));
    CHECK_HIP(hipMemcpy(scratch, rows_d, n * bb, hipMemcpyDeviceToHost));
    for (i = 0; i < n; ++i)
        if (expect_block(scratch + i * bb, 0, (uint64_t)perm_a[n - 1 - i], bb, "gather", i)) return 7;

    /* an argument error is a status, not a crash */
    if (hfk_gather_rows(NULL, rows_d, ids_d, 1, n, bb, blocks, 0, 0, stream) != HFK_ERR_NULL_POINTER) {
        fprintf(stderr, "NULL table was not rejected\n");
        return 8;
    }

    for (p = 0; p < planes; ++p) {
        CHECK_HIP(hipFree(dev_plane[p]));
        CHECK_HFK(hfk_mm_free_pinned(host_plane[p]));
    }
    if (hfk_mm_record_count() != 0) { fprintf(stderr, "registry still holds records\n"); return 9; }
    CHECK_HIP(hipFree(dev_tab)); CHECK_HIP(hipFree(host_tab)); CHECK_HIP(hipFree(pairs_d));
    CHECK_HIP(hipFree(ids_d)); CHECK_HIP(hipFree(staging)); CHECK_HIP(hipFree(rows_d));
    CHECK_HIP(hipStreamDestroy(stream));
    free(dev_plane); free(host_plane); free(dev_tab_h); free(host_tab_h); free(scratch);
    free(perm_a); free(perm_b); free(pairs_h); free(host_ids);
    printf("hfk_c_client: OK\n");
    return 0;
}
