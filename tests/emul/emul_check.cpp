// CPU index-math checker for the kernel bodies (test infrastructure).
//
// Compiles the exact per-lane bodies and launch planning the GPU library uses
// (hfk_bodies.h, hfk_plan.h) for the host, walks every (workgroup, lane) pair of a
// launch sequentially, and compares the bytes with the C oracle. Buffers are sized
// exactly and the program is built with AddressSanitizer, so an out-of-range lane
// access aborts the run instead of faulting a GPU later. This never runs in the
// product; it exists so that indexing mistakes are found before a kernel is ever
// launched on hardware.
#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
#include <vector>

#include "hfk.h"
#include "hfk_bodies.h"
#include "hfk_plan.h"

extern "C" {
int oracle_gather_rows(const void* table, void* dst, const void* ids, int ids_are_i64, uint64_t n_ids,
                       uint64_t row_bytes, uint32_t cores);
int oracle_multi_layer_block_transfer(void* const* layer_ptrs, const void* src, uint32_t T, uint32_t L,
                                      uint32_t H, uint32_t D, uint32_t elem_bytes, uint32_t cores);
int oracle_multi_layer_block_table_transfer(void* const* layer_ptrs, uint64_t layered_stride, void* packed,
                                            uint64_t packed_stride, const int64_t* pairs, uint64_t n_pairs,
                                            uint32_t T, uint32_t L, uint32_t H, uint32_t D, uint32_t elem_bytes,
                                            int to_packed, uint32_t cores);
int oracle_swap_blocks(void* const* dst_planes, const void* const* src_planes, const int64_t* pairs,
                       uint32_t n_planes, uint64_t n_pairs, uint64_t block_bytes, uint64_t src_stride,
                       uint64_t dst_stride);
}

namespace {

using namespace hfk;

std::mt19937_64 rng(12345);
int g_failures = 0;
int g_cases = 0;

// Exactly-sized heap buffer (ASan red zones on both ends), optional misalignment.
struct Buf {
    uint8_t* raw = nullptr;
    uint8_t* p = nullptr;
    size_t n = 0;
    Buf(size_t bytes, size_t misalign = 0) : n(bytes) {
        raw = static_cast<uint8_t*>(std::aligned_alloc(64, ((bytes + misalign + 63) / 64) * 64 + 64));
        p = raw + misalign;
    }
    ~Buf() { std::free(raw); }
    void randomize() { for (size_t i = 0; i < n; ++i) p[i] = (uint8_t)rng(); }
    void fill(uint8_t v) { std::memset(p, v, n); }
    Buf(const Buf&) = delete;
    Buf& operator=(const Buf&) = delete;
};

void expect_equal(const uint8_t* a, const uint8_t* b, size_t n, const char* what) {
    ++g_cases;
    if (std::memcmp(a, b, n) != 0) {
        size_t i = 0;
        while (i < n && a[i] == b[i]) ++i;
        std::printf("FAIL %s: first difference at byte %zu of %zu\n", what, i, n);
        ++g_failures;
    }
}

template <typename Body, typename Args>
void walk(const Args& a, uint32_t grid, Body body) {
    for (uint32_t bid = 0; bid < grid; ++bid)
        for (uint32_t tid = 0; tid < kWorkgroupLanes; ++tid) body(a, bid, grid, tid);
}

template <typename IdT, int NT>
void run_block_copy(BlockCopyArgs<IdT> a, int preferred_unroll, uint32_t grid_cap, bool whole_chunks = false) {
    int unroll = 1;   // whole_chunks: as the launcher plans every role but the swap
    if (plan_block_copy<IdT>(a, preferred_unroll, &unroll, whole_chunks) != HFK_OK) { std::printf("plan failed\n"); ++g_failures; return; }
    const uint32_t grid = a.n_work < grid_cap ? a.n_work : grid_cap;
    if (a.run_mode == kListedPairs) {   // a launch that is handed its pairs runs the bodies built for a list
        switch (unroll) {
            case 1: walk(a, grid, block_copy_body<IdT, 1, NT, false, true, true>); break;
            case 2: walk(a, grid, block_copy_body<IdT, 2, NT, false, true, true>); break;
            case 4: walk(a, grid, block_copy_body<IdT, 4, NT, false, true, true>); break;
            case 8: walk(a, grid, block_copy_body<IdT, 8, NT, false, true, true>); break;
            default: walk(a, grid, block_copy_body<IdT, 16, NT, false, true, true>); break;
        }
        return;
    }
    if (a.run_mode != kAllPairs) {   // a split table runs the bodies built with the run filter, as the launcher does
        switch (unroll) {
            case 1: walk(a, grid, block_copy_body<IdT, 1, NT, true>); break;
            case 2: walk(a, grid, block_copy_body<IdT, 2, NT, true>); break;
            case 4: walk(a, grid, block_copy_body<IdT, 4, NT, true>); break;
            case 8: walk(a, grid, block_copy_body<IdT, 8, NT, true>); break;
            default: walk(a, grid, block_copy_body<IdT, 16, NT, true>); break;
        }
        return;
    }
    switch (unroll) {
        case 1: walk(a, grid, block_copy_body<IdT, 1, NT>); break;
        case 2: walk(a, grid, block_copy_body<IdT, 2, NT>); break;
        case 4: walk(a, grid, block_copy_body<IdT, 4, NT>); break;
        case 8: walk(a, grid, block_copy_body<IdT, 8, NT>); break;
        default: walk(a, grid, block_copy_body<IdT, 16, NT>); break;
    }
}

template <typename V, typename IdT, typename IndexT, int NT>
void walk_flat(const FlatGatherArgs<IdT>& a, uint32_t grid, int unroll) {
    if (unroll == kFlatUnrollHost) walk(a, grid, flat_gather_body<V, IdT, IndexT, kFlatUnrollHost, NT>);
    else walk(a, grid, flat_gather_body<V, IdT, IndexT, kFlatUnrollDevice, NT>);
}

template <typename IdT>
void run_flat_gather(uint64_t table, uint64_t dst, const IdT* ids, uint64_t n_ids, uint64_t row_bytes,
                     uint64_t limit, uint32_t grid_cap, bool force64) {
    for (int unroll : {kFlatUnrollDevice, kFlatUnrollHost}) {   // both launch shapes write the same bytes
        FlatGatherArgs<IdT> a;
        FlatGatherPlan p;
        if (plan_flat_gather<IdT>(a, p, table, dst, ids, n_ids, row_bytes, limit, unroll) != HFK_OK) { ++g_failures; return; }
        const uint32_t grid = a.n_work < grid_cap ? a.n_work : grid_cap;
        const bool i32 = p.index32 && !force64;
        if (p.unit == 16u) {
            if (i32) walk_flat<vec16, IdT, uint32_t, 3>(a, grid, unroll);
            else walk_flat<vec16, IdT, uint64_t, 0>(a, grid, unroll);
        } else if (p.unit == 4u) {
            if (i32) walk_flat<uint32_t, IdT, uint32_t, 0>(a, grid, unroll);
            else walk_flat<uint32_t, IdT, uint64_t, 3>(a, grid, unroll);
        } else {
            if (i32) walk_flat<uint8_t, IdT, uint32_t, 0>(a, grid, unroll);
            else walk_flat<uint8_t, IdT, uint64_t, 0>(a, grid, unroll);
        }
    }
}

// ---- swap_blocks ----------------------------------------------------------
void case_swap(uint32_t n_planes, uint32_t n_pairs, uint64_t block_bytes, uint64_t src_blocks, uint64_t dst_blocks,
               uint64_t src_pad, uint64_t dst_pad, size_t src_mis, size_t dst_mis, int unroll, uint32_t grid_cap,
               bool with_bad_pairs) {
    const uint64_t ss = block_bytes + src_pad, ds = block_bytes + dst_pad;
    std::vector<Buf*> src, dst, exp;
    std::vector<uint64_t> sp, dp;
    std::vector<void*> ep;
    std::vector<const void*> spc;
    for (uint32_t p = 0; p < n_planes; ++p) {
        src.push_back(new Buf(src_blocks * ss - src_pad, src_mis));
        dst.push_back(new Buf(dst_blocks * ds - dst_pad, dst_mis));
        exp.push_back(new Buf(dst_blocks * ds - dst_pad, dst_mis));
        src.back()->randomize();
        dst.back()->fill(0xA5);
        exp.back()->fill(0xA5);
        sp.push_back((uint64_t)(uintptr_t)src.back()->p);
        dp.push_back((uint64_t)(uintptr_t)dst.back()->p);
        ep.push_back(exp.back()->p);
        spc.push_back(src.back()->p);
    }
    // distinct destination blocks
    std::vector<int64_t> dperm(dst_blocks);
    for (uint64_t i = 0; i < dst_blocks; ++i) dperm[i] = (int64_t)i;
    std::shuffle(dperm.begin(), dperm.end(), rng);
    std::vector<int64_t> pairs, good;
    for (uint32_t j = 0; j < n_pairs; ++j) {
        int64_t s = (int64_t)(rng() % src_blocks), d = dperm[j % dst_blocks];
        bool bad = false;
        if (with_bad_pairs && j % 5 == 3) { s = (j % 2) ? -1 - (int64_t)(rng() % 7) : (int64_t)src_blocks + (int64_t)(rng() % 9); bad = true; }
        if (with_bad_pairs && j % 7 == 5) { d = (j % 2) ? (int64_t)dst_blocks : -3; bad = true; }
        pairs.push_back(s);
        pairs.push_back(d);
        if (!bad) { good.push_back(s); good.push_back(d); }
    }
    BlockCopyArgs<int64_t> a;
    int rc = plan_swap_blocks(a, dp.data(), sp.data(), pairs.data(), n_planes, n_pairs, block_bytes, ss, ds,
                              src_blocks, dst_blocks);
    if (rc != HFK_OK) { std::printf("plan_swap_blocks rc=%d\n", rc); ++g_failures; }
    else {
        run_block_copy<int64_t, 3>(a, unroll, grid_cap);
        oracle_swap_blocks(ep.data(), spc.data(), good.data(), n_planes, good.size() / 2, block_bytes, ss, ds);
        char what[160];
        std::snprintf(what, sizeof what, "swap planes=%u pairs=%u bytes=%llu pad=%llu/%llu mis=%zu/%zu unroll=%d grid=%u bad=%d",
                      n_planes, n_pairs, (unsigned long long)block_bytes, (unsigned long long)src_pad,
                      (unsigned long long)dst_pad, src_mis, dst_mis, unroll, grid_cap, (int)with_bad_pairs);
        for (uint32_t p = 0; p < n_planes; ++p) expect_equal(dst[p]->p, exp[p]->p, dst[p]->n, what);
    }
    for (auto* b : src) delete b;
    for (auto* b : dst) delete b;
    for (auto* b : exp) delete b;
}

// ---- duplex swap: two disjoint block-table copies in one launch ---------------
void case_duplex(uint32_t n_planes, uint32_t n_out, uint32_t n_in, uint64_t block_bytes, uint32_t dev_blocks,
                 uint32_t host_blocks, size_t mis, int unroll, uint32_t grid_cap, bool with_bad) {
    std::vector<Buf*> dev, host, dev_exp, host_exp;
    std::vector<uint64_t> dp, hp;
    std::vector<void*> dep, hep;
    std::vector<const void*> dsp, hsp;
    for (uint32_t p = 0; p < n_planes; ++p) {
        dev.push_back(new Buf(dev_blocks * block_bytes, mis));
        host.push_back(new Buf(host_blocks * block_bytes, mis));
        dev_exp.push_back(new Buf(dev_blocks * block_bytes, mis));
        host_exp.push_back(new Buf(host_blocks * block_bytes, mis));
        dev.back()->randomize();
        host.back()->randomize();
        std::memcpy(dev_exp.back()->p, dev.back()->p, dev.back()->n);
        std::memcpy(host_exp.back()->p, host.back()->p, host.back()->n);
        dp.push_back((uint64_t)(uintptr_t)dev.back()->p);
        hp.push_back((uint64_t)(uintptr_t)host.back()->p);
        dep.push_back(dev_exp.back()->p);
        hep.push_back(host_exp.back()->p);
        dsp.push_back(dev_exp.back()->p);
        hsp.push_back(host_exp.back()->p);
    }
    // out reads device blocks [0, n_out) of a permutation and writes host blocks [0, n_out) of another;
    // in reads host blocks after those and writes device blocks after those: disjoint by construction.
    std::vector<int64_t> dperm(dev_blocks), hperm(host_blocks);
    for (uint32_t i = 0; i < dev_blocks; ++i) dperm[i] = i;
    for (uint32_t i = 0; i < host_blocks; ++i) hperm[i] = i;
    std::shuffle(dperm.begin(), dperm.end(), rng);
    std::shuffle(hperm.begin(), hperm.end(), rng);
    std::vector<int64_t> po, pi, po_good, pi_good;
    for (uint32_t j = 0; j < n_out; ++j) {
        int64_t s = dperm[j], d = hperm[j];
        bool bad = with_bad && j % 3 == 1;
        if (bad) s = (j % 2) ? -5 : (int64_t)dev_blocks + 1;
        po.push_back(s); po.push_back(d);
        if (!bad) { po_good.push_back(s); po_good.push_back(d); }
    }
    for (uint32_t j = 0; j < n_in; ++j) {
        int64_t s = hperm[n_out + j], d = dperm[n_out + j];
        bool bad = with_bad && j % 4 == 2;
        if (bad) d = (int64_t)dev_blocks;
        pi.push_back(s); pi.push_back(d);
        if (!bad) { pi_good.push_back(s); pi_good.push_back(d); }
    }
    hfk_block_move out_move{hp.data(), dp.data(), po.data(), n_out, block_bytes, block_bytes, dev_blocks, host_blocks};
    hfk_block_move in_move{dp.data(), hp.data(), pi.data(), n_in, block_bytes, block_bytes, host_blocks, dev_blocks};
    DuplexCopyArgs a;
    int u = 1;
    int rc = plan_duplex(a, &out_move, &in_move, n_planes, block_bytes, unroll, &u);
    if (rc != HFK_OK) { ++g_failures; std::printf("plan_duplex rc=%d\n", rc); }
    else if (a.n_work > 0) {
        const uint32_t grid = a.n_work < grid_cap ? a.n_work : grid_cap;
        switch (u) {
            case 1: walk(a, grid, duplex_copy_body<1, 3>); break;
            case 2: walk(a, grid, duplex_copy_body<2, 0>); break;
            case 4: walk(a, grid, duplex_copy_body<4, 3>); break;
            case 8: walk(a, grid, duplex_copy_body<8, 3>); break;
            default: walk(a, grid, duplex_copy_body<16, 3>); break;
        }
    }
    if (!po_good.empty()) oracle_swap_blocks(hep.data(), dsp.data(), po_good.data(), n_planes, po_good.size() / 2, block_bytes, block_bytes, block_bytes);
    if (!pi_good.empty()) oracle_swap_blocks(dep.data(), hsp.data(), pi_good.data(), n_planes, pi_good.size() / 2, block_bytes, block_bytes, block_bytes);
    char what[160];
    std::snprintf(what, sizeof what, "duplex planes=%u out=%u in=%u bytes=%llu mis=%zu unroll=%d grid=%u bad=%d", n_planes, n_out,
                  n_in, (unsigned long long)block_bytes, mis, unroll, grid_cap, (int)with_bad);
    for (uint32_t p = 0; p < n_planes; ++p) {
        expect_equal(dev[p]->p, dev_exp[p]->p, dev[p]->n, what);
        expect_equal(host[p]->p, host_exp[p]->p, host[p]->n, what);
    }
    for (auto* b : dev) delete b;
    for (auto* b : host) delete b;
    for (auto* b : dev_exp) delete b;
    for (auto* b : host_exp) delete b;
}

// ---- kernel half of the staged swap: planes <-> contiguous staging buffer ------
void case_stage(uint32_t n_planes, uint32_t n_blocks, uint64_t block_bytes, uint32_t dev_blocks, uint64_t pad, bool to_staging,
                int unroll, uint32_t grid_cap, bool with_bad) {
    const uint64_t ds = block_bytes + pad;
    std::vector<Buf*> dev, dev_exp;
    std::vector<uint64_t> dp;
    Buf staging((uint64_t)n_planes * n_blocks * block_bytes), staging_exp((uint64_t)n_planes * n_blocks * block_bytes);
    staging.randomize();
    std::memcpy(staging_exp.p, staging.p, staging.n);
    for (uint32_t p = 0; p < n_planes; ++p) {
        dev.push_back(new Buf(dev_blocks * ds - pad));
        dev_exp.push_back(new Buf(dev_blocks * ds - pad));
        dev.back()->randomize();
        std::memcpy(dev_exp.back()->p, dev.back()->p, dev.back()->n);
        dp.push_back((uint64_t)(uintptr_t)dev.back()->p);
    }
    std::vector<int64_t> perm(dev_blocks), ids(n_blocks);
    for (uint32_t i = 0; i < dev_blocks; ++i) perm[i] = i;
    std::shuffle(perm.begin(), perm.end(), rng);
    for (uint32_t i = 0; i < n_blocks; ++i) {
        ids[i] = perm[i % dev_blocks];
        if (with_bad && i % 3 == 2) ids[i] = (i % 2) ? -1 : (int64_t)dev_blocks + 3;
    }
    BlockCopyArgs<int64_t> a;
    int rc = plan_stage_blocks(a, dp.data(), staging.p, ids.data(), n_planes, n_blocks, block_bytes, ds, dev_blocks, to_staging);
    if (rc != HFK_OK) { ++g_failures; std::printf("plan_stage_blocks rc=%d\n", rc); }
    else run_block_copy<int64_t, 3>(a, unroll, grid_cap);
    for (uint32_t p = 0; p < n_planes; ++p)
        for (uint32_t i = 0; i < n_blocks; ++i) {
            uint8_t* st = staging_exp.p + ((uint64_t)p * n_blocks + i) * block_bytes;
            if (ids[i] < 0 || ids[i] >= (int64_t)dev_blocks) {
                if (to_staging) std::memset(st, 0, block_bytes);   // a slot the gather cannot fill is zeroed
                continue;
            }
            uint8_t* dv = dev_exp[p]->p + (uint64_t)ids[i] * ds;
            if (to_staging) std::memcpy(st, dv, block_bytes); else std::memcpy(dv, st, block_bytes);
        }
    char what[160];
    std::snprintf(what, sizeof what, "stage planes=%u blocks=%u bytes=%llu pad=%llu to_staging=%d unroll=%d grid=%u bad=%d", n_planes,
                  n_blocks, (unsigned long long)block_bytes, (unsigned long long)pad, (int)to_staging, unroll, grid_cap, (int)with_bad);
    expect_equal(staging.p, staging_exp.p, staging.n, what);
    for (uint32_t p = 0; p < n_planes; ++p) expect_equal(dev[p]->p, dev_exp[p]->p, dev[p]->n, what);
    for (auto* b : dev) delete b;
    for (auto* b : dev_exp) delete b;
}

// ---- one block table split between two movers by run length (hfk_swap_blocks_auto) ----------
// Long runs of consecutive host slots: kernel between device planes and staging + plain copies
// (the copy engines' part, done here with memcpy per run exactly as copy_host_runs walks them);
// everything else: the direct kernel with the complementary filter.
void case_auto(uint32_t n_planes, uint32_t n_pairs, uint64_t block_bytes, uint32_t dev_blocks, uint32_t host_blocks,
               bool to_host, uint32_t min_run, int unroll, uint32_t grid_cap, bool with_bad_dev) {
    std::vector<Buf*> dev, host, dev_exp, host_exp;
    std::vector<uint64_t> dp, hp;
    for (uint32_t p = 0; p < n_planes; ++p) {
        dev.push_back(new Buf(dev_blocks * block_bytes));
        host.push_back(new Buf(host_blocks * block_bytes));
        dev_exp.push_back(new Buf(dev_blocks * block_bytes));
        host_exp.push_back(new Buf(host_blocks * block_bytes));
        dev.back()->randomize();
        host.back()->randomize();
        std::memcpy(dev_exp.back()->p, dev.back()->p, dev.back()->n);
        std::memcpy(host_exp.back()->p, host.back()->p, host.back()->n);
        dp.push_back((uint64_t)(uintptr_t)dev.back()->p);
        hp.push_back((uint64_t)(uintptr_t)host.back()->p);
    }
    // host slots: runs of random length at distinct places, in random order; device blocks distinct
    std::vector<int64_t> host_ids;
    {
        std::vector<std::pair<int64_t, int64_t>> runs;   // (start, len) cut out of 0..host_blocks-1 left to right
        int64_t at = 0;
        while (at < (int64_t)host_blocks) {
            const int64_t len = 1 + (int64_t)(rng() % 5);
            const int64_t gap = 1 + (int64_t)(rng() % 2);        // a gap keeps neighbouring runs apart
            if (at + len > (int64_t)host_blocks) break;
            runs.push_back({at, len});
            at += len + gap;
        }
        std::shuffle(runs.begin(), runs.end(), rng);
        for (auto& r : runs)
            for (int64_t i = 0; i < r.second && host_ids.size() < n_pairs; ++i) host_ids.push_back(r.first + i);
    }
    n_pairs = (uint32_t)host_ids.size();
    std::vector<int64_t> dperm(dev_blocks);
    for (uint32_t i = 0; i < dev_blocks; ++i) dperm[i] = i;
    std::shuffle(dperm.begin(), dperm.end(), rng);
    std::vector<int64_t> pairs(2 * (size_t)n_pairs), dev_ids(n_pairs);
    for (uint32_t j = 0; j < n_pairs; ++j) {
        dev_ids[j] = dperm[j % dev_blocks];
        if (with_bad_dev && j % 4 == 1) dev_ids[j] = (j % 8 == 1) ? -2 : (int64_t)dev_blocks + 1;
        pairs[2 * j] = to_host ? dev_ids[j] : host_ids[j];
        pairs[2 * j + 1] = to_host ? host_ids[j] : dev_ids[j];
    }
    // Every other case is moved by lists of pairs: a buffer that holds exactly the long runs (a slot beyond it would
    // be an access the sanitizer reports), lists from fill_pair_lists, which states what the list kernel computes.
    // The others keep a buffer for the whole table and let the kernels filter the pairs.
    static unsigned auto_cases = 0;
    const uint64_t long_blocks = blocks_in_long_runs(host_ids.data(), n_pairs, min_run);
    const bool compact = (auto_cases++ % 2 == 1) && long_blocks != 0 && long_blocks < n_pairs;
    const uint64_t plane_slots = compact ? long_blocks : n_pairs;
    Buf staging((uint64_t)n_planes * plane_slots * block_bytes);
    staging.randomize();
    std::vector<int64_t> long_list(n_pairs, 0), short_list(n_pairs, 0);
    if (compact) {
        fill_pair_lists(pairs.data() + (to_host ? 1 : 0), 2, n_pairs, min_run, long_list.data(), short_list.data());
        uint64_t listed = 0;                     // every pair is in exactly one list, each list in table order
        for (uint32_t i = 0; i < n_pairs; ++i) listed += (long_list[i] >= 0) + (short_list[i] >= 0);
        if (listed != n_pairs || long_list[long_blocks - 1] < 0 || long_list[long_blocks] != -1) {
            ++g_failures;
            std::printf("case_auto: lists name %llu of %u pairs\n", (unsigned long long)listed, n_pairs);
        }
    }
    // expected
    for (uint32_t p = 0; p < n_planes; ++p)
        for (uint32_t j = 0; j < n_pairs; ++j) {
            uint8_t* h = host_exp[p]->p + (uint64_t)host_ids[j] * block_bytes;
            const bool bad = dev_ids[j] < 0 || dev_ids[j] >= (int64_t)dev_blocks;
            if (to_host) {
                if (bad) std::memset(h, 0, block_bytes);
                else std::memcpy(h, dev[p]->p + (uint64_t)dev_ids[j] * block_bytes, block_bytes);
            } else if (!bad) {
                std::memcpy(dev_exp[p]->p + (uint64_t)dev_ids[j] * block_bytes, h, block_bytes);
            }
        }
    // the three steps, in the order the entry point enqueues them
    const int64_t* host_column = pairs.data() + (to_host ? 1 : 0);
    const int64_t* dev_column = pairs.data() + (to_host ? 0 : 1);
    BlockCopyArgs<int64_t> direct, hbm;
    int rc = to_host ? plan_swap_blocks(direct, hp.data(), dp.data(), pairs.data(), n_planes, n_pairs, block_bytes, block_bytes,
                                        block_bytes, dev_blocks, host_blocks)
                     : plan_swap_blocks(direct, dp.data(), hp.data(), pairs.data(), n_planes, n_pairs, block_bytes, block_bytes,
                                        block_bytes, host_blocks, dev_blocks);
    if (rc == HFK_OK) rc = plan_stage_blocks(hbm, dp.data(), staging.p, dev_column, n_planes, plane_slots, block_bytes, block_bytes,
                                             dev_blocks, to_host);
    if (rc != HFK_OK) { ++g_failures; std::printf("case_auto plan rc=%d\n", rc); return; }
    direct.zero_skipped = to_host ? 1u : 0u;
    hbm.id_stride = 2;
    if (compact) {
        list_pairs(hbm, long_list.data(), (uint32_t)long_blocks, n_pairs);
        list_pairs(direct, short_list.data(), (uint32_t)(n_pairs - long_blocks), n_pairs);
    } else {
        filter_runs(hbm, kLongRunsOnly, host_column, min_run);
        filter_runs(direct, kShortRunsOnly, host_column, min_run);
    }
    auto copies = [&]() {
        uint64_t staged_before = 0;      // as the copy engines' leg counts its slots
        for_each_host_run(host_ids.data(), n_pairs, [&](uint64_t first, uint64_t len) {
            if (len < min_run) return;
            const uint64_t slot = compact ? staged_before : first;
            staged_before += len;
            for (uint32_t p = 0; p < n_planes; ++p) {
                uint8_t* h = host[p]->p + (uint64_t)host_ids[first] * block_bytes;
                uint8_t* st = staging.p + ((uint64_t)p * plane_slots + slot) * block_bytes;
                if (to_host) std::memcpy(h, st, len * block_bytes); else std::memcpy(st, h, len * block_bytes);
            }
        });
    };
    if (to_host) { run_block_copy<int64_t, 3>(hbm, unroll, grid_cap, true); copies(); }
    else { copies(); run_block_copy<int64_t, 3>(hbm, unroll, grid_cap, true); }
    run_block_copy<int64_t, 3>(direct, unroll > 4 ? 4 : unroll, grid_cap > 16 ? 16 : grid_cap);
    char what[192];
    std::snprintf(what, sizeof what, "auto planes=%u pairs=%u bytes=%llu to_host=%d min_run=%u unroll=%d grid=%u bad=%d long=%llu compact=%d",
                  n_planes, n_pairs, (unsigned long long)block_bytes, (int)to_host, min_run, unroll, grid_cap, (int)with_bad_dev,
                  (unsigned long long)long_blocks, (int)compact);
    for (uint32_t p = 0; p < n_planes; ++p) {
        expect_equal(dev[p]->p, dev_exp[p]->p, dev[p]->n, what);
        expect_equal(host[p]->p, host_exp[p]->p, host[p]->n, what);
    }
    for (auto* b : dev) delete b;
    for (auto* b : host) delete b;
    for (auto* b : dev_exp) delete b;
    for (auto* b : host_exp) delete b;
}

// What the run-splitting swap does when its two copies of the host column disagree (the header documents it;
// HFK_KNOB_CHECK_HOST_COLUMN exists to catch it): the copy engines take their runs from the host array, the
// kernels theirs from the table. Here the array calls all four pairs one long run, the table calls them four
// single slots. On the way out the staging kernel therefore fills nothing, the copies send the four staging
// slots as they are to the array's slots, and the direct kernel then moves every pair to the table's slots: a
// slot both name ends up right, a slot only the array names holds what staging held before the call.
void case_auto_with_disagreeing_columns() {
    const uint64_t bb = 4096;
    const uint32_t n = 4, dev_blocks = 8, host_blocks = 40, min_run = 2;
    Buf dev(dev_blocks * bb), host(host_blocks * bb), staging(n * bb);
    dev.randomize();
    host.fill(0x11);
    staging.fill(0xEE);                                   // "an earlier transfer's bytes"
    const int64_t array_ids[n] = {10, 11, 12, 13}, table_ids[n] = {10, 20, 12, 30}, dev_ids[n] = {3, 1, 7, 5};
    std::vector<int64_t> pairs;
    for (uint32_t j = 0; j < n; ++j) { pairs.push_back(dev_ids[j]); pairs.push_back(table_ids[j]); }
    uint64_t dp[1] = {(uint64_t)(uintptr_t)dev.p}, hp[1] = {(uint64_t)(uintptr_t)host.p};
    BlockCopyArgs<int64_t> direct, hbm;
    int rc = plan_swap_blocks(direct, hp, dp, pairs.data(), 1, n, bb, bb, bb, dev_blocks, host_blocks);
    if (rc == HFK_OK) rc = plan_stage_blocks(hbm, dp, staging.p, pairs.data(), 1, n, bb, bb, dev_blocks, true);
    if (rc != HFK_OK) { ++g_failures; std::printf("disagreeing columns: plan rc=%d\n", rc); return; }
    direct.zero_skipped = 1;
    hbm.id_stride = 2;
    filter_runs(hbm, kLongRunsOnly, pairs.data() + 1, min_run);
    filter_runs(direct, kShortRunsOnly, pairs.data() + 1, min_run);
    run_block_copy<int64_t, 3>(hbm, 1, 4, true);                                     // the table has no long run: nothing staged
    for_each_host_run(array_ids, n, [&](uint64_t first, uint64_t len) {              // the array has one: four slots copied
        if (len >= min_run) std::memcpy(host.p + (uint64_t)array_ids[first] * bb, staging.p + first * bb, len * bb);
    });
    run_block_copy<int64_t, 3>(direct, 1, 4);                                        // every pair is short for the table
    Buf want(host_blocks * bb);
    want.fill(0x11);
    std::memset(want.p + 11 * bb, 0xEE, bb);              // named by the array only: stale staging bytes
    std::memset(want.p + 13 * bb, 0xEE, bb);
    for (uint32_t j = 0; j < n; ++j) std::memcpy(want.p + (uint64_t)table_ids[j] * bb, dev.p + (uint64_t)dev_ids[j] * bb, bb);
    expect_equal(host.p, want.p, host.n, "run-splitting swap with disagreeing host columns");
}

// The same disagreement when the call moves its pairs by lists (a table that is split, a buffer with room for the
// lists). The array calls pairs 0-2 one long run and pair 3 a single slot, so three staging slots are copied to the
// array's slots and the direct launch covers one position of the short list; the table has no long run at all, so
// its long list is empty (every entry -1: the staging kernel moves nothing) and its short list starts with pair 0.
// Pair 0 ends up right, pairs 1-3 are not moved, and the array's slots 11 and 12 hold what staging held before.
void case_auto_listed_with_disagreeing_columns() {
    const uint64_t bb = 4096;
    const uint32_t n = 4, dev_blocks = 8, host_blocks = 40, min_run = 2;
    Buf dev(dev_blocks * bb), host(host_blocks * bb), staging(3 * bb);
    dev.randomize();
    host.fill(0x11);
    staging.fill(0xEE);
    const int64_t array_ids[n] = {10, 11, 12, 20}, table_ids[n] = {10, 30, 12, 20}, dev_ids[n] = {3, 1, 7, 5};
    std::vector<int64_t> pairs;
    for (uint32_t j = 0; j < n; ++j) { pairs.push_back(dev_ids[j]); pairs.push_back(table_ids[j]); }
    const uint64_t long_blocks = blocks_in_long_runs(array_ids, n, min_run);            // the host's count: 3
    std::vector<int64_t> long_list(n), short_list(n);
    fill_pair_lists(pairs.data() + 1, 2, n, min_run, long_list.data(), short_list.data());   // the device's lists
    uint64_t dp[1] = {(uint64_t)(uintptr_t)dev.p}, hp[1] = {(uint64_t)(uintptr_t)host.p};
    BlockCopyArgs<int64_t> direct, hbm;
    int rc = plan_swap_blocks(direct, hp, dp, pairs.data(), 1, n, bb, bb, bb, dev_blocks, host_blocks);
    if (rc == HFK_OK) rc = plan_stage_blocks(hbm, dp, staging.p, pairs.data(), 1, long_blocks, bb, bb, dev_blocks, true);
    if (rc != HFK_OK || long_blocks != 3) { ++g_failures; std::printf("disagreeing columns, listed: plan rc=%d\n", rc); return; }
    direct.zero_skipped = 1;
    hbm.id_stride = 2;
    list_pairs(hbm, long_list.data(), (uint32_t)long_blocks, n);
    list_pairs(direct, short_list.data(), (uint32_t)(n - long_blocks), n);
    run_block_copy<int64_t, 3>(hbm, 1, 4, true);
    uint64_t staged_before = 0;
    for_each_host_run(array_ids, n, [&](uint64_t first, uint64_t len) {
        if (len < min_run) return;
        std::memcpy(host.p + (uint64_t)array_ids[first] * bb, staging.p + staged_before * bb, len * bb);
        staged_before += len;
    });
    run_block_copy<int64_t, 3>(direct, 1, 4);
    Buf want(host_blocks * bb);
    want.fill(0x11);
    std::memset(want.p + 11 * bb, 0xEE, bb);
    std::memset(want.p + 12 * bb, 0xEE, bb);
    std::memcpy(want.p + 10 * bb, dev.p + 3 * bb, bb);    // staging's stale bytes first, then pair 0 by the direct launch
    expect_equal(host.p, want.p, host.n, "run-splitting swap by lists with disagreeing host columns");
}

// ---- gather_blocks (multi-plane, shared ids) -------------------------------
void case_gather_blocks(uint32_t n_planes, uint32_t n_ids, uint64_t block_bytes, uint64_t src_blocks, int unroll,
                        uint32_t grid_cap) {
    std::vector<Buf*> src, dst, exp;
    std::vector<uint64_t> sp, dp;
    std::vector<int64_t> ids(n_ids);
    for (auto& i : ids) i = (int64_t)(rng() % src_blocks);
    for (uint32_t p = 0; p < n_planes; ++p) {
        src.push_back(new Buf(src_blocks * block_bytes));
        dst.push_back(new Buf((uint64_t)n_ids * block_bytes));
        exp.push_back(new Buf((uint64_t)n_ids * block_bytes));
        src.back()->randomize();
        dst.back()->fill(0x11);
        sp.push_back((uint64_t)(uintptr_t)src.back()->p);
        dp.push_back((uint64_t)(uintptr_t)dst.back()->p);
        oracle_gather_rows(src.back()->p, exp.back()->p, ids.data(), 1, n_ids, block_bytes, 3);
    }
    BlockCopyArgs<int64_t> a;
    int rc = plan_gather_blocks(a, dp.data(), sp.data(), ids.data(), n_planes, n_ids, block_bytes, block_bytes, src_blocks);
    if (rc != HFK_OK) { ++g_failures; std::printf("plan_gather_blocks rc=%d\n", rc); }
    else {
        run_block_copy<int64_t, 0>(a, unroll, grid_cap, true);
        char what[128];
        std::snprintf(what, sizeof what, "gather_blocks planes=%u ids=%u bytes=%llu unroll=%d grid=%u", n_planes, n_ids,
                      (unsigned long long)block_bytes, unroll, grid_cap);
        for (uint32_t p = 0; p < n_planes; ++p) expect_equal(dst[p]->p, exp[p]->p, dst[p]->n, what);
    }
    for (auto* b : src) delete b;
    for (auto* b : dst) delete b;
    for (auto* b : exp) delete b;
}

// ---- gather_rows (both the wide and the flat path, as the entry point picks) --
template <typename IdT>
void case_gather_rows(uint64_t table_rows, uint64_t n_ids, uint64_t row_bytes, size_t t_mis, size_t d_mis, int unroll,
                      uint32_t grid_cap, bool with_bad_ids, bool force64) {
    Buf table(table_rows * row_bytes, t_mis), dst(n_ids * row_bytes, d_mis), exp(n_ids * row_bytes, d_mis);
    table.randomize();
    dst.fill(0x5A);
    exp.fill(0x5A);
    std::vector<IdT> ids(n_ids);
    for (uint64_t i = 0; i < n_ids; ++i) {
        ids[i] = (IdT)(rng() % table_rows);
        if (with_bad_ids && i % 4 == 1) ids[i] = (i % 8 == 1) ? (IdT)-2 : (IdT)(table_rows + i);
    }
    for (uint64_t i = 0; i < n_ids; ++i) {  // expected: valid rows copied, invalid rows untouched
        if (ids[i] >= 0 && (uint64_t)ids[i] < table_rows)
            oracle_gather_rows(table.p, exp.p + i * row_bytes, &ids[i], sizeof(IdT) == 8, 1, row_bytes, 1);
    }
    if (row_bytes >= kWideRowBytes) {
        BlockCopyArgs<IdT> a;
        if (plan_wide_gather<IdT>(a, table.p, dst.p, ids.data(), n_ids, row_bytes, table_rows) != HFK_OK) { ++g_failures; return; }
        run_block_copy<IdT, 3>(a, unroll, grid_cap, true);
    } else {
        run_flat_gather<IdT>((uint64_t)(uintptr_t)table.p, (uint64_t)(uintptr_t)dst.p, ids.data(), n_ids, row_bytes,
                             table_rows, grid_cap, force64);
    }
    char what[160];
    std::snprintf(what, sizeof what, "gather_rows<i%zu> rows=%llu ids=%llu row_bytes=%llu mis=%zu/%zu unroll=%d grid=%u bad=%d f64=%d",
                  sizeof(IdT) * 8, (unsigned long long)table_rows, (unsigned long long)n_ids,
                  (unsigned long long)row_bytes, t_mis, d_mis, unroll, grid_cap, (int)with_bad_ids, (int)force64);
    expect_equal(dst.p, exp.p, dst.n, what);
}

// ---- transpose -------------------------------------------------------------
template <bool TO_PACKED, int UNROLL = kTransposeUnroll>
void walk_transpose(const TransposeArgs& a, uint32_t unit, uint32_t grid_cap) {
    if (a.n_work == 0) return;
    const uint32_t grid = a.n_work < grid_cap ? a.n_work : grid_cap;
    if constexpr (!TO_PACKED) {
        if (a.mirror != 0) {   // the bodies the staged op's single kernel is built from
            if (unit == 16u) walk(a, grid, transpose_body<vec16, UNROLL, 3, false, true>);
            else if (unit == 4u) walk(a, grid, transpose_body<uint32_t, UNROLL, 0, false, true>);
            else walk(a, grid, transpose_body<uint8_t, UNROLL, 0, false, true>);
            return;
        }
    }
    if (unit == 16u) walk(a, grid, transpose_body<vec16, UNROLL, 3, TO_PACKED>);
    else if (unit == 4u) walk(a, grid, transpose_body<uint32_t, UNROLL, 0, TO_PACKED>);
    else walk(a, grid, transpose_body<uint8_t, UNROLL, 0, TO_PACKED>);
}

// The tiled form toward the packed side: per tile every lane's load phase, then every lane's store phase,
// with a host array standing in for LDS: what the kernel's two barriers order.
template <int U>
void walk_transpose_tiles_u(const TransposeArgs& a, uint32_t grid) {
    std::vector<vec16> tile(64 * 4 * U);
    for (uint32_t bid = 0; bid < grid; ++bid) {
        for (uint64_t w = bid; w < a.n_work; w += grid) {
            TransposeTile it;
            if (!transpose_tile_item(a, w, it)) continue;
            for (uint32_t tid = 0; tid < kWorkgroupLanes; ++tid)
                transpose_tile_load<U, 3>(a, it, tid, LayerTableInMemory{a.layer_ptrs}, tile.data());
            for (uint32_t tid = 0; tid < kWorkgroupLanes; ++tid) transpose_tile_store<U, 3>(a, it, tid, tile.data());
        }
    }
}

int g_tiled_walks = 0;
void walk_transpose_tiles(const TransposeArgs& a, int U, uint32_t grid_cap) {
    const uint32_t grid = a.n_work < grid_cap ? a.n_work : grid_cap;
    ++g_tiled_walks;
    switch (U) {
        case 8: walk_transpose_tiles_u<8>(a, grid); break;
        case 4: walk_transpose_tiles_u<4>(a, grid); break;
        case 2: walk_transpose_tiles_u<2>(a, grid); break;
        default: walk_transpose_tiles_u<1>(a, grid); break;
    }
}

// single block, the reference's op
void case_transpose(uint32_t T, uint32_t L, uint32_t H, uint32_t D, uint32_t elem, size_t s_mis, size_t l_mis,
                    uint32_t grid_cap) {
    const uint64_t block = (uint64_t)T * L * H * D * elem, layer = (uint64_t)H * T * D * elem;
    Buf src(block, s_mis);
    src.randomize();
    std::vector<Buf*> dst, exp;
    std::vector<uint64_t> lp;
    std::vector<void*> ep;
    for (uint32_t l = 0; l < L; ++l) {
        dst.push_back(new Buf(layer, l_mis));
        exp.push_back(new Buf(layer, l_mis));
        dst.back()->fill(0xEE);
        exp.back()->fill(0xEE);
        lp.push_back((uint64_t)(uintptr_t)dst.back()->p);
        ep.push_back(exp.back()->p);
    }
    // every other case also fills a second copy of the packed block while it reads it (the staged op's single
    // kernel); its alignment alternates with the case, so that it takes part in the choice of the unit
    static unsigned cases = 0;
    const bool mirrored = cases++ % 2 == 1;
    Buf mirror(block, mirrored && cases % 4 == 0 ? 4 : 0);
    mirror.fill(0x5A);
    TransposeArgs a;
    uint32_t unit = 0;
    int rc = plan_transpose(a, &unit, lp.data(), src.p, nullptr, 1, 0, 0, 0, 0, T, L, H, D, elem, kTransposeUnroll,
                            mirrored ? mirror.p : nullptr);
    if (rc != HFK_OK) { ++g_failures; std::printf("plan_transpose rc=%d\n", rc); }
    else walk_transpose<false>(a, unit, grid_cap);
    oracle_multi_layer_block_transfer(ep.data(), src.p, T, L, H, D, elem, 3);
    char what[128];
    std::snprintf(what, sizeof what, "transpose T=%u L=%u H=%u D=%u elem=%u mis=%zu/%zu grid=%u unit=%u mirror=%d", T, L, H, D,
                  elem, s_mis, l_mis, grid_cap, unit, (int)mirrored);
    for (uint32_t l = 0; l < L; ++l) expect_equal(dst[l]->p, exp[l]->p, layer, what);
    if (mirrored) {
        expect_equal(mirror.p, src.p, block, what);
    } else {
        Buf untouched(block);
        untouched.fill(0x5A);
        expect_equal(mirror.p, untouched.p, block, what);
    }
    for (auto* b : dst) delete b;
    for (auto* b : exp) delete b;
}

// block table, both directions, padded strides, out-of-range pairs
void case_transpose_table(uint32_t T, uint32_t L, uint32_t H, uint32_t D, uint32_t elem, uint32_t packed_blocks,
                          uint32_t dev_blocks, uint32_t n_pairs, uint64_t p_pad, uint64_t l_pad, size_t p_mis,
                          size_t l_mis, bool to_packed, bool with_bad, uint32_t grid_cap) {
    const uint64_t block = (uint64_t)T * L * H * D * elem, layer_block = (uint64_t)H * T * D * elem;
    const uint64_t ps = block + p_pad, ls = layer_block + l_pad;
    Buf packed(packed_blocks * ps - p_pad, p_mis), packed_exp(packed_blocks * ps - p_pad, p_mis);
    packed.randomize();
    std::memcpy(packed_exp.p, packed.p, packed.n);
    std::vector<Buf*> lay, lay_exp;
    std::vector<uint64_t> lp;
    std::vector<void*> ep;
    for (uint32_t l = 0; l < L; ++l) {
        lay.push_back(new Buf(dev_blocks * ls - l_pad, l_mis));
        lay_exp.push_back(new Buf(dev_blocks * ls - l_pad, l_mis));
        lay.back()->randomize();
        std::memcpy(lay_exp.back()->p, lay.back()->p, lay.back()->n);
        lp.push_back((uint64_t)(uintptr_t)lay.back()->p);
        ep.push_back(lay_exp.back()->p);
    }
    // distinct destination blocks on whichever side is written
    std::vector<int64_t> pperm(packed_blocks), dperm(dev_blocks), pairs, good;
    for (uint32_t i = 0; i < packed_blocks; ++i) pperm[i] = i;
    for (uint32_t i = 0; i < dev_blocks; ++i) dperm[i] = i;
    std::shuffle(pperm.begin(), pperm.end(), rng);
    std::shuffle(dperm.begin(), dperm.end(), rng);
    for (uint32_t j = 0; j < n_pairs; ++j) {
        int64_t pb = pperm[j % packed_blocks], db = dperm[j % dev_blocks];
        bool bad = false;
        if (with_bad && j % 4 == 1) { pb = (j % 8 == 1) ? -1 : (int64_t)packed_blocks + 2; bad = true; }
        if (with_bad && j % 5 == 2) { db = (j % 2) ? (int64_t)dev_blocks : -7; bad = true; }
        pairs.push_back(pb);
        pairs.push_back(db);
        if (!bad) { good.push_back(pb); good.push_back(db); }
    }
    TransposeArgs a;
    uint32_t unit = 0;
    // toward the packed side both launch shapes exist (a pool in device memory, a pool in host memory):
    // alternate between them from case to case
    static unsigned to_packed_cases = 0;
    const bool to_host_shape = to_packed && (to_packed_cases++ % 2 == 1);
    int rc = plan_transpose(a, &unit, lp.data(), packed.p, pairs.data(), n_pairs, ps, ls, packed_blocks, dev_blocks, T,
                            L, H, D, elem, to_host_shape ? kTransposeUnrollToHost : kTransposeUnroll);
    // a pool in host memory goes through LDS tiles where the geometry allows
    const int tiled = rc == HFK_OK && to_host_shape ? plan_transpose_tiles(a, unit, 512) : 0;
    if (rc != HFK_OK) { ++g_failures; std::printf("plan_transpose(table) rc=%d\n", rc); }
    else if (tiled != 0) walk_transpose_tiles(a, tiled, grid_cap);
    else if (to_host_shape) walk_transpose<true, kTransposeUnrollToHost>(a, unit, grid_cap);
    else if (to_packed) walk_transpose<true>(a, unit, grid_cap);
    else walk_transpose<false>(a, unit, grid_cap);
    oracle_multi_layer_block_table_transfer(ep.data(), ls, packed_exp.p, ps, good.data(), good.size() / 2, T, L, H, D,
                                            elem, to_packed, 2);
    char what[192];
    std::snprintf(what, sizeof what, "transpose_table T=%u L=%u H=%u D=%u e=%u pb=%u db=%u pairs=%u pad=%llu/%llu mis=%zu/%zu "
                  "to_packed=%d bad=%d grid=%u unit=%u", T, L, H, D, elem, packed_blocks, dev_blocks, n_pairs,
                  (unsigned long long)p_pad, (unsigned long long)l_pad, p_mis, l_mis, (int)to_packed, (int)with_bad,
                  grid_cap, unit);
    expect_equal(packed.p, packed_exp.p, packed.n, what);
    for (uint32_t l = 0; l < L; ++l) expect_equal(lay[l]->p, lay_exp[l]->p, lay[l]->n, what);
    for (auto* b : lay) delete b;
    for (auto* b : lay_exp) delete b;
}

}  // namespace

// the launch shape of a swap, by flags, size and link rate: the rules as the header documents them
void case_swap_shape() {
    const SwapTuning t{16, 8, 6, 4, 0, 0};        // the defaults: a throughput-mode swap-out is not paced
    SwapTuning paced = t;
    paced.throughput_pace_permille = 890;         // ... unless the knob says so
    const uint32_t link = 63015, out = HFK_SWAP_DST_HOST, in = HFK_SWAP_SRC_HOST, beside = HFK_SWAP_BESIDE_COMPUTE;
    const uint64_t big = 512ull << 20, small = 2ull << 20;
    const uint64_t bb = 32768;
    struct { const SwapTuning* tuning; uint32_t flags; uint64_t bytes; uint32_t link; uint32_t asked;
             uint32_t wg; int unroll; uint32_t pace; bool plain; const char* what; } rows[] = {
        {&t, 0, big, link, 0, 16, 8, 0, false, "nothing known: 16 x 8 unpaced"},
        {&t, out, big, link, 0, 12, 8, 0, true, "swap-out of 64 MiB or more: 12 x 8 unpaced, plain stores"},
        {&t, out, kLongSwapBytes, link, 0, 12, 8, 0, true, "exactly 64 MiB counts as long"},
        {&t, out, kLongSwapBytes - 1, link, 0, 16, 8, 0, false, "a shorter swap-out runs as with no flags"},
        {&t, out, small, link, 0, 16, 8, 0, false, "a 2 MiB swap-out runs as with no flags"},
        {&t, out, big, 0, 0, 12, 8, 0, true, "link rate unknown: the unpaced shape needs none"},
        {&t, out | beside, small, link, 0, 12, 1, 52932, false, "beside compute: 12 x 1 paced at 0.84 whatever the size"},
        {&t, out | beside, big, 0, 0, 8, 4, 0, false, "beside compute, link unknown: 8 x 4 unpaced"},
        {&t, beside, big, link, 0, 8, 4, 0, false, "beside compute, no side named: 8 x 4 unpaced"},
        {&t, in, big, link, 0, 40, 1, 0, false, "swap-in: 40 x 1"},
        {&t, in | beside, big, link, 0, 24, 1, 0, false, "swap-in beside compute: 24 x 1"},
        {&t, in | out, big, link, 0, 12, 8, 0, true, "both sides host memory: the destination decides"},
        {&t, out, big, link, 20, 20, 8, 0, true, "the caller's grid bound is kept"},
        {&t, in, big, link, 7, 7, 1, 0, false, "the caller's grid bound is kept (swap-in)"},
        {&t, 0, big, link, 300, 300, 8, 0, false, "the caller's grid bound is kept (no flags)"},
        {&paced, out, big, link, 0, 6, 4, 56083, false, "pacing switched on: 6 x 4 at 0.89, non-temporal stores"},
        {&paced, out, kLongSwapBytes - 1, link, 0, 16, 8, 0, false, "pacing switched on, short swap: unpaced"},
        {&paced, out, big, 0, 0, 12, 8, 0, true, "pacing switched on, link unknown: the unpaced shape"},
        {&paced, out, big, link, 20, 20, 4, 56083, false, "pacing switched on, the caller's grid bound is kept"},
    };
    for (const auto& r : rows) {
        const SwapShape got = choose_swap_shape(r.flags, r.bytes, bb, r.link, r.asked, *r.tuning);
        ++g_cases;
        if (got.workgroups != r.wg || got.unroll != r.unroll || got.pace_mbps != r.pace || got.plain_stores != r.plain) {
            ++g_failures;
            std::printf("swap shape: %s: got %u x %d paced %u plain %d, want %u x %d paced %u plain %d\n", r.what,
                        got.workgroups, got.unroll, got.pace_mbps, (int)got.plain_stores, r.wg, r.unroll, r.pace, (int)r.plain);
        }
    }
    // the unpaced shape toward the host by block size: 12 x 8, 32 x 4, 64 x 2 or 96 x 1, whole chunks or 32 x 4,
    // never a grid that divides evenly into chunks of unequal size
    struct { uint64_t block; uint32_t wg; int unroll; } by_block[] = {
        {4096, 96, 1}, {8192, 64, 2}, {16384, 32, 4}, {32768, 12, 8}, {65536, 12, 8}, {131072, 12, 8},
        {73728, 32, 4},          // 72 KiB: 16 + 16 + 16 + 16 + 8
        {69632, 32, 4},          // 68 KiB
        {20480, 33, 4},          // 20 KiB = 16 + 4: two chunks, and 32 workgroups would split evenly over them
        {12288, 65, 2},          // 12 KiB = 8 + 4 on 64 x 2
        {4112, 97, 1},           // 4 KiB + 16 B
        {1024, 96, 1},           // smaller than one chunk
    };
    for (const auto& r : by_block) {
        const SwapShape got = choose_swap_shape(out, big, r.block, link, 0, t);
        ++g_cases;
        if (got.workgroups != r.wg || got.unroll != r.unroll || got.pace_mbps != 0 || !got.plain_stores) {
            ++g_failures;
            std::printf("swap shape for %llu-byte blocks: got %u x %d, want %u x %d\n", (unsigned long long)r.block,
                        got.workgroups, got.unroll, r.wg, r.unroll);
        }
    }
    // the paced throughput shape keeps 6 x 4 vectors per lane in flight whatever the block size
    struct { uint64_t block; uint32_t wg; int unroll; } paced_by_block[] = {{4096, 24, 1}, {8192, 12, 2}, {16384, 6, 4}, {73728, 6, 4}};
    for (const auto& r : paced_by_block) {
        const SwapShape got = choose_swap_shape(out, big, r.block, link, 0, paced);
        ++g_cases;
        if (got.workgroups != r.wg || got.unroll != r.unroll || got.pace_mbps != 56083 || got.plain_stores) {
            ++g_failures;
            std::printf("paced swap shape for %llu-byte blocks: got %u x %d\n", (unsigned long long)r.block, got.workgroups, got.unroll);
        }
    }
    // the factor a paced launch leaves for the next one: slower when it fell behind or many turns began late,
    // faster when few did, unchanged in between, and never outside its bounds
    struct { uint32_t factor; uint32_t late_per_65536; bool behind; int direction; } settle[] = {
        {65536, 0, true, +1}, {65536, 6554, false, +1}, {65536, 3932, false, +1}, {65536, 3000, false, 0},
        {65536, 2300, false, -1}, {65536, 655, false, -1}, {kPaceFactorMax, 65535, true, 0}, {kPaceFactorMin, 0, false, 0}};
    for (const auto& r : settle) {
        const uint32_t next = next_pace_factor(r.factor, r.late_per_65536, r.behind);
        const int direction = next > r.factor ? +1 : next < r.factor ? -1 : 0;
        ++g_cases;
        if (direction != r.direction || next < kPaceFactorMin || next > kPaceFactorMax) {
            ++g_failures;
            std::printf("next_pace_factor(%u, %u, %d) = %u\n", r.factor, r.late_per_65536, (int)r.behind, next);
        }
    }
    ++g_cases;
    if (pace_factor(nullptr) != kPaceFactorOne) { ++g_failures; std::printf("pace_factor(nullptr)\n"); }
    SwapTuning forced = t;
    forced.beside_pace_mbps = 1;      // an explicit pace (the test of the bounded wait uses 1 MB/s)
    const SwapShape s1 = choose_swap_shape(out | beside, small, bb, 0, 0, forced);
    ++g_cases;
    if (s1.workgroups != 12 || s1.unroll != 1 || s1.pace_mbps != 1) { ++g_failures; std::printf("swap shape: explicit pace\n"); }
}

// the PCIe link-rate parser on the strings sysfs shows
void case_link_rate() {
    struct { const char* speed; const char* width; int want; } rows[] = {
        {"32.0 GT/s PCIe\n", "16\n", 63015},      // Gen5 x16: 32 * 16 * 128/130 / 8 GB/s
        {"16.0 GT/s PCIe", "16", 31507},           // Gen4 x16
        {"8.0 GT/s PCIe", "8", 7876},              // Gen3 x8
        {"5.0 GT/s PCIe", "16", 8000},             // Gen2: 8b/10b encoding
        {"2.5 GT/s PCIe", "1", 250},
        {"64.0 GT/s PCIe", "16", 126030},
        {"Unknown", "16", -1}, {"", "16", -1}, {"32.0 GT/s PCIe", "", -1}, {"32.0 GT/s PCIe", "0", -1},
        {"32.0 GT/s PCIe", "64", -1}, {"-8.0 GT/s", "16", -1}, {nullptr, "16", -1}, {"32.0 GT/s", nullptr, -1},
    };
    for (const auto& r : rows) {
        ++g_cases;
        const int got = link_mbps_from_sysfs(r.speed, r.width);
        if (got != r.want) {
            std::printf("FAIL link rate '%s' x '%s': got %d, want %d\n", r.speed ? r.speed : "(null)",
                        r.width ? r.width : "(null)", got, r.want);
            ++g_failures;
        }
    }
}

int main() {
    case_link_rate();
    case_swap_shape();
    // swap: aligned fast path, every unroll, grid smaller and larger than the work
    for (int unroll : {1, 2, 4, 8, 16})
        for (uint32_t grid : {1u, 7u, 4096u}) {
            case_swap(3, 9, 32768, 16, 12, 0, 0, 0, 0, unroll, grid, false);
            case_swap(2, 5, 73728, 8, 8, 0, 0, 0, 0, unroll, grid, false);   // MLA block: 4.5 chunks at unroll 4
            case_swap(2, 6, 16384, 10, 9, 0, 0, 0, 0, unroll, grid, true);   // fp8 block + out-of-range pairs
        }
    // swap: blocks one vector short of / past a whole number of chunks
    for (int unroll : {1, 2, 4, 8, 16}) {
        const uint64_t chunk = 4096ull * unroll;
        case_swap(2, 3, chunk - 16, 5, 5, 0, 0, 0, 0, unroll, 4, false);
        case_swap(2, 3, chunk + 16, 5, 5, 0, 0, 0, 0, unroll, 4, false);
        case_swap(1, 3, 2 * chunk - 16, 4, 4, 0, 0, 0, 0, unroll, 100, false);
        case_swap(1, 3, 2 * chunk + 4080, 4, 4, 16, 16, 0, 0, unroll, 100, true);
    }
    // swap: padded strides, tails that are not a whole chunk, tiny blocks
    case_swap(2, 7, 4096 + 48, 9, 9, 16, 32, 0, 0, 8, 5, false);
    case_swap(1, 4, 16, 6, 6, 0, 0, 0, 0, 8, 3, false);
    case_swap(2, 4, 272, 6, 7, 16, 0, 0, 0, 4, 64, true);
    // swap: 4-byte and 1-byte paths (size or base not 16-byte aligned)
    case_swap(2, 5, 5000, 7, 7, 0, 0, 0, 0, 8, 3, false);     // size % 16 != 0, % 4 == 0... 5000 % 8 == 0
    case_swap(2, 5, 4100, 7, 7, 0, 0, 4, 8, 4, 9, true);      // bases 4-aligned
    case_swap(2, 5, 4099, 7, 7, 0, 0, 0, 0, 2, 9, false);     // odd size
    case_swap(1, 3, 8192, 4, 4, 0, 0, 1, 3, 8, 2, false);     // odd bases
    case_swap(1, 3, 40000, 4, 4, 3, 5, 2, 6, 16, 2, true);    // odd strides

    for (int unroll : {1, 4, 8, 16}) {
        case_gather_blocks(4, 11, 32768, 20, unroll, 13);
        case_gather_blocks(3, 6, 16384, 9, unroll, 1000);
    }

    // gather_rows: wide rows (block-copy path) and narrow rows (flat path)
    case_gather_rows<int64_t>(64, 32, 32768, 0, 0, 8, 50, false, false);   // config-1 row
    case_gather_rows<int32_t>(64, 32, 32768, 0, 0, 8, 50, true, false);
    case_gather_rows<int64_t>(50, 17, 4096, 0, 0, 8, 4, true, false);      // narrowest wide row
    case_gather_rows<int64_t>(50, 17, 4112, 0, 0, 16, 4, false, false);
    case_gather_rows<int64_t>(50, 17, 4099, 1, 2, 4, 6, true, false);      // wide, byte path
    for (bool f64 : {false, true}) {
        case_gather_rows<int64_t>(500, 333, 1024, 0, 0, 8, 16, false, f64);   // reference's embedding row
        case_gather_rows<int32_t>(500, 333, 1024, 0, 0, 8, 3, true, f64);
        case_gather_rows<int64_t>(100, 77, 16, 0, 0, 8, 2, true, f64);        // one vector per row
        case_gather_rows<int64_t>(100, 1, 48, 0, 0, 8, 2, false, f64);
        case_gather_rows<int64_t>(100, 77, 4080, 0, 0, 8, 9, false, f64);     // widest flat row
        case_gather_rows<int64_t>(100, 55, 1020, 0, 0, 8, 5, true, f64);      // 4-byte units
        case_gather_rows<int32_t>(100, 55, 1024, 4, 8, 8, 5, false, f64);     // 4-byte aligned bases
        case_gather_rows<int64_t>(100, 55, 999, 0, 0, 8, 5, true, f64);       // byte units
        case_gather_rows<int64_t>(100, 55, 1, 0, 0, 8, 5, false, f64);
        case_gather_rows<int32_t>(100, 55, 1024, 1, 0, 8, 700, false, f64);   // odd table base
    }

    // transpose: the reference's test geometry scaled down, README shapes, odd shapes
    case_transpose(64, 32, 1, 128, 1, 0, 0, 7);       // int8, H=1 (tests/test_transfer_kernel.py:15-21 with T cut)
    case_transpose(32, 4, 8, 128, 1, 0, 0, 1000);     // H=8 (README table rows)
    case_transpose(16, 3, 2, 128, 2, 0, 0, 3);        // bf16
    case_transpose(5, 3, 2, 64, 4, 0, 0, 2);          // fp32
    case_transpose(1, 1, 1, 16, 1, 0, 0, 1);
    case_transpose(7, 1, 1, 128, 2, 0, 0, 2);         // L = H = 1: plain copy
    case_transpose(9, 2, 3, 20, 2, 0, 0, 5);          // rows of 40 bytes -> 4-byte units
    case_transpose(9, 2, 3, 7, 1, 0, 0, 5);           // rows of 7 bytes -> byte units
    case_transpose(9, 2, 3, 16, 2, 0, 4, 5);          // layer buffers only 4-byte aligned: per-unit byte stores
    case_transpose(9, 2, 3, 16, 2, 4, 0, 5);          // source 4-byte aligned
    case_transpose(6, 2, 2, 16, 1, 1, 3, 5);          // everything odd
    case_transpose(0, 2, 2, 16, 1, 0, 0, 5);          // empty block

    // duplex swap: equal and unequal sides, one side empty, tails, odd alignment, out-of-range pairs
    for (int unroll : {1, 2, 4, 8, 16}) {
        case_duplex(2, 5, 5, 32768, 16, 16, 0, unroll, 3, false);
        case_duplex(2, 7, 3, 32768, 16, 16, 0, unroll, 1000, true);
        case_duplex(1, 2, 6, 73728, 10, 10, 0, unroll, 5, false);      // MLA block: tail chunks
        case_duplex(2, 4, 0, 16384, 8, 8, 0, unroll, 4, false);        // only swap-out
        case_duplex(2, 0, 4, 16384, 8, 8, 0, unroll, 4, true);         // only swap-in
    }
    case_duplex(2, 3, 4, 4100, 9, 9, 4, 4, 7, false);                  // 4-byte path
    case_duplex(2, 3, 4, 4099, 9, 9, 1, 4, 7, true);                   // byte path
    case_duplex(1, 3, 3, 48, 7, 7, 0, 4, 2, false);                    // blocks smaller than a chunk
    case_duplex(1, 0, 0, 4096, 4, 4, 0, 4, 2, false);                  // nothing at all

    // staged swap, kernel half: gather into and scatter out of the staging buffer
    for (bool to_staging : {true, false})
        for (int unroll : {1, 4, 8, 16}) {
            case_stage(3, 7, 32768, 12, 0, to_staging, unroll, 5, false);
            case_stage(2, 5, 73728, 9, 0, to_staging, unroll, 1000, true);
            case_stage(2, 6, 16384, 8, 64, to_staging, unroll, 3, true);
            case_stage(1, 4, 4100, 6, 0, to_staging, unroll, 2, false);
        }

    // one table split by run length between the staged and the direct mover
    for (bool to_host : {true, false})
        for (uint32_t min_run : {1u, 2u, 3u, 4u, 6u, 9u})
            for (int unroll : {1, 4, 8}) {
                case_auto(3, 20, 32768, 24, 40, to_host, min_run, unroll, 5, false);
                case_auto(2, 30, 16384, 32, 60, to_host, min_run, unroll, 1000, true);
                case_auto(2, 11, 73728, 12, 30, to_host, min_run, unroll, 16, true);
                case_auto(1, 9, 4100, 10, 20, to_host, min_run, unroll, 3, false);
            }

    case_auto_with_disagreeing_columns();
    case_auto_listed_with_disagreeing_columns();

    // block-table transfer, both directions
    for (bool to_packed : {false, true}) {
        case_transpose_table(16, 4, 2, 128, 1, 6, 5, 4, 0, 0, 0, 0, to_packed, false, 7);      // int8 rows of 128 B
        case_transpose_table(8, 3, 2, 64, 2, 5, 7, 5, 0, 0, 0, 0, to_packed, true, 1000);     // bf16 + bad pairs
        case_transpose_table(33, 2, 3, 16, 2, 4, 4, 4, 32, 64, 0, 0, to_packed, false, 3);     // padded strides, odd T
        case_transpose_table(5, 2, 2, 20, 2, 4, 4, 3, 0, 0, 0, 0, to_packed, true, 5);         // 40-byte rows: 4-byte units
        case_transpose_table(5, 2, 2, 7, 1, 4, 4, 3, 0, 0, 0, 0, to_packed, false, 5);         // 7-byte rows: byte units
        case_transpose_table(9, 2, 3, 16, 2, 3, 3, 3, 0, 0, 0, 4, to_packed, false, 5);        // layer caches 4-byte aligned
        case_transpose_table(9, 2, 3, 16, 2, 3, 3, 3, 4, 0, 0, 0, to_packed, true, 5);         // packed stride 4-byte aligned
        case_transpose_table(6, 2, 2, 16, 1, 3, 3, 2, 3, 5, 1, 3, to_packed, false, 5);        // everything odd
        case_transpose_table(64, 2, 1, 128, 1, 3, 3, 3, 0, 0, 0, 0, to_packed, false, 2);      // one-head blocks
    }
    // toward the packed side twice each, so that both launch shapes meet every geometry: the second one
    // goes through LDS tiles where T, L * H and the row size allow (rows of 16 B ... 1 KiB, 4 to 32 rows per tile)
    for (int rep = 0; rep < 2; ++rep) {
        case_transpose_table(16, 4, 8, 128, 1, 6, 5, 4, 0, 0, 0, 0, true, false, 7);       // 128-byte rows, L * H = 32: tiles of 8 tokens x 32 rows
        case_transpose_table(16, 4, 2, 128, 1, 6, 5, 4, 0, 0, 0, 0, true, true, 1000);     // L * H = 8: 8 rows per tile, bad pairs
        case_transpose_table(8, 3, 4, 64, 2, 5, 7, 5, 32, 64, 0, 0, true, false, 3);       // L * H = 12: 4 rows per tile, padded strides
        case_transpose_table(128, 2, 2, 16, 1, 4, 4, 3, 0, 0, 0, 0, true, false, 5);       // 16-byte rows: 64 tokens per tile
        case_transpose_table(3, 8, 2, 512, 2, 4, 4, 4, 0, 0, 0, 0, true, true, 9);         // 1 KiB rows: one token per tile, 16 rows
        case_transpose_table(4, 2, 8, 256, 1, 3, 3, 3, 0, 0, 0, 4, true, false, 4);        // 256-byte rows, layer caches 4-byte aligned
        case_transpose_table(12, 2, 2, 128, 1, 3, 3, 2, 0, 0, 0, 0, true, false, 5);       // T no multiple of 8: not tiled
        case_transpose_table(16, 3, 1, 128, 1, 3, 3, 2, 0, 0, 0, 0, true, false, 5);       // L * H = 3: not tiled
        case_transpose_table(16, 2, 2, 48, 1, 3, 3, 2, 0, 0, 0, 0, true, false, 5);        // 48-byte rows: not tiled
    }
    ++g_cases;
    if (g_tiled_walks < 6) { ++g_failures; std::printf("only %d tiled walks: the tiled cases did not tile\n", g_tiled_walks); }

    // seeded random shapes on top of the hand-picked ones
    auto pick = [&](std::initializer_list<uint64_t> v) { return *(v.begin() + rng() % v.size()); };
    const int kUnrolls[5] = {1, 2, 4, 8, 16};
    for (int it = 0; it < 150; ++it) {
        const int unroll = kUnrolls[rng() % 5];
        const uint32_t grid = (uint32_t)pick({1, 2, 3, 7, 33, 100000});
        const uint64_t bytes = pick({16, 48, 4096, 4112, 8192, 12288 + 16, 16384, 32768, 36864, 65536 + 32, 73728, 1000, 4099, 20});
        const uint32_t planes = 1 + rng() % 3, sb = 2 + rng() % 9, db = 2 + rng() % 9;
        const uint32_t np = 1 + rng() % db;   // destination blocks must be distinct
        const uint64_t pad_s = pick({0, 0, 16, 64}), pad_d = pick({0, 0, 16, 48});
        const size_t mis = (bytes % 16) ? (size_t)pick({0, 1, 4}) : 0;
        case_swap(planes, np, bytes, sb, db, (bytes % 16) ? 0 : pad_s, (bytes % 16) ? 0 : pad_d, mis, mis, unroll, grid,
                  rng() % 2);
        if (it % 3 == 0) case_gather_blocks(planes, np, bytes - bytes % 16 + 16, sb, unroll, grid);
        if (it % 3 == 1) case_duplex(planes, rng() % 5, rng() % 5, bytes, 12, 12, mis, unroll, grid, rng() % 2);
    }
    for (int it = 0; it < 120; ++it) {
        const uint64_t rb = pick({1, 3, 16, 20, 64, 100, 256, 1024, 1040, 2048, 4080, 4095, 4096, 5000, 8192, 8200});
        const uint64_t rows = 1 + rng() % 40, n_ids = rng() % 70;
        const size_t tm = (rb % 16) ? (size_t)pick({0, 1, 4, 8}) : 0, dm = (rb % 16) ? (size_t)pick({0, 2, 4}) : 0;
        if (rng() % 2) case_gather_rows<int64_t>(rows, n_ids, rb, tm, dm, kUnrolls[rng() % 5], 1 + rng() % 50, rng() % 2, rng() % 2);
        else case_gather_rows<int32_t>(rows, n_ids, rb, tm, dm, kUnrolls[rng() % 5], 1 + rng() % 50, rng() % 2, rng() % 2);
    }
    for (int it = 0; it < 120; ++it) {
        const uint32_t T = 1 + rng() % 20, L = 1 + rng() % 4, H = 1 + rng() % 4;
        const uint32_t D = (uint32_t)pick({1, 4, 7, 8, 16, 24, 32, 64, 128}), e = (uint32_t)pick({1, 2, 4});
        const bool aligned = ((uint64_t)D * e) % 16 == 0;
        const size_t m1 = aligned ? 0 : (size_t)pick({0, 1, 4}), m2 = (size_t)pick({0, 0, 4, 3});
        if (it % 2 == 0) case_transpose(T, L, H, D, e, m1, m2, 1 + rng() % 20);
        else case_transpose_table(T, L, H, D, e, 3 + rng() % 4, 3 + rng() % 4, 1 + rng() % 3, aligned ? pick({0, 16, 64}) : 0,
                                  aligned ? pick({0, 32}) : 0, m1, m2, rng() % 2, rng() % 2, 1 + rng() % 20);
    }

    std::printf("%d comparisons, %d failures\n", g_cases, g_failures);
    return g_failures == 0 ? 0 : 1;
}
