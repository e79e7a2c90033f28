// Per-lane bodies of the three data-movement kernels.
//
// Each body is an ordinary function of (workgroup index, workgroup count, lane
// index) and touches memory only through its argument struct, so the same text
// is compiled twice: by hipcc as the body of a __global__ kernel for gfx950, and
// by the host compiler inside the CPU index-math checker used by the unit tests
// (which walks every (workgroup, lane) pair sequentially under a bounds checker).
// No LDS and no barriers are used: these kernels are pure streaming copies whose
// lanes never exchange data, so staging through LDS would only add a hop.
//
// Access shape: a workgroup is 256 lanes (4 wavefronts of 64). In the fast path
// every lane moves 16-byte vectors; lane i of a wavefront touches vector i of a
// 1 KiB contiguous span, so each wavefront instruction is one fully coalesced
// 1 KiB request. A lane issues UNROLL independent loads before its first store
// to keep UNROLL * 16 B in flight per lane (what hides PCIe and HBM latency).
#pragma once

#include <stdint.h>

#if defined(__HIPCC__)
#define HFK_HD __host__ __device__ __forceinline__
#else
#define HFK_HD inline
#endif

// Addresses arrive as integers (plane tables, base + offset arithmetic). A plain
// cast would give a generic pointer and flat_* instructions; every address these
// kernels touch is global memory, so say so and get global_load/global_store.
#if defined(__HIP_DEVICE_COMPILE__)
#define HFK_GLOBAL __attribute__((address_space(1)))
#else
#define HFK_GLOBAL
#endif

// Pacing support: a constant-rate 100 MHz counter (independent of the shader clock) and a
// short sleep. The CPU build walks the same index math without pacing.
#if defined(__HIP_DEVICE_COMPILE__)
#define HFK_CAN_PACE 1
#define HFK_TICKS_100MHZ() wall_clock64()
#define HFK_NAP() __builtin_amdgcn_s_sleep(2)
#else
#define HFK_CAN_PACE 0
#define HFK_TICKS_100MHZ() ((uint64_t)0)
#define HFK_NAP() ((void)0)
#endif

namespace hfk {

constexpr uint32_t kWorkgroupLanes = 256;

typedef uint32_t vec16 __attribute__((ext_vector_type(4)));

// Pacing of a host-facing copy. Offering the PCIe link more than it drains fills the queues
// that every other kernel's memory traffic shares (and, toward the host, even lowers what the
// link accepts); offering it a fixed rate just under its capacity keeps them empty at the same
// throughput. Workgroup `bid` of `nb` starts its k-th work item no earlier than
// (k + bid / nb) * pace_q8 / 256 ticks of the 100 MHz counter after it began, so the launch as a
// whole offers one item per pace_q8 / 256 / nb ticks. pace_q8 == 0: no pacing.
// A pace that is set between launches. What the link takes, and what a tick of the counter is worth,
// differ by a percent from machine to machine and from moment to moment, and the room between a pace that
// keeps the queues empty and one the link cannot hold is smaller than that. A launch cannot find the
// right interval while it runs (its wavefronts hand their stores to the memory pipeline and notice an
// overloaded link only when the queues behind them are full), but all of a launch's workgroups together
// know afterwards how it went: how many of their turns began late (2 % at 0.89 of what the link takes,
// 4 % at 0.895, 7 % at 0.90, 14 % at 0.905, its knee), and whether any of them ended behind its schedule.
// The last workgroup to finish turns that into a factor for the next launch's interval, kept in eight
// words of device memory that belong to the library: [0] the factor in 1/65536 (0 = 1.0), [1] turns and
// [2] late turns of the launch in progress, [3] workgroups finished, [4] workgroups that ended behind
// schedule, [5] launches settled, [6] late turns per 65536 turns of the last launch, [7] unused.
// Launches on one stream see each other's result in order; launches that overlap on two streams may
// read a factor one launch old and may settle on each other's counts, which costs the factor one
// small step in a wrong direction and nothing else (it is bounded, and the data never depend on it).
constexpr uint32_t kPaceFactorOne = 65536;
constexpr uint32_t kPaceFactorMin = 61000;        // the interval may shrink by 7 % ...
constexpr uint32_t kPaceFactorMax = 68157;        // ... and grow by 4 % from the nominal one: what slows a launch down
                                                  // may be a neighbour and not the link, and must not cost it much

HFK_HD uint32_t pace_factor(const uint32_t* state) {
    if (state == nullptr) return kPaceFactorOne;
    const uint32_t f = *reinterpret_cast<const HFK_GLOBAL uint32_t*>(reinterpret_cast<uint64_t>(state));
    return f == 0 ? kPaceFactorOne : f;
}

// The factor for the next launch from this one's account: late turns per 65536 turns, and whether any
// workgroup ended behind its schedule.
HFK_HD uint32_t next_pace_factor(uint32_t factor, uint32_t late_per_65536, bool behind) {
    uint64_t f = factor;
    if (behind) f += f >> 6;                                   // could not hold it: 1.6 % slower
    else if (late_per_65536 > 5243) f += f >> 8;               // more than 8 % late: 0.4 % slower
    else if (late_per_65536 > 3604) f += f >> 9;               // more than 5.5 %: 0.2 % slower
    else if (late_per_65536 < 1638) f -= f >> 8;               // fewer than 2.5 %: 0.4 % faster
    else if (late_per_65536 < 2621) f -= f >> 10;              // fewer than 4 %: 0.1 % faster
    if (f < kPaceFactorMin) f = kPaceFactorMin;
    if (f > kPaceFactorMax) f = kPaceFactorMax;
    return (uint32_t)f;
}

struct Pacer {
    uint64_t t0;
    uint64_t due_q8;
    uint32_t pace_q8;
    // What the schedule did to this workgroup, for callers that ask (pace report): turns taken, turns
    // that began behind schedule (no waiting), and the largest delay behind schedule seen, in 1/256 ticks.
    uint32_t turns;
    uint32_t late_turns;
    uint64_t max_late_q8;

    HFK_HD Pacer(uint32_t pace, uint32_t bid, uint32_t nb)
        : t0(0), due_q8(0), pace_q8(HFK_CAN_PACE ? pace : 0), turns(0), late_turns(0), max_late_q8(0) {
        if (pace_q8 != 0) {
            t0 = HFK_TICKS_100MHZ();
            due_q8 = (uint64_t)pace_q8 * bid / nb;  // workgroups take turns within an interval
        }
    }

    // Call before each work item. The counter always advances; the spin limit ends the wait regardless.
    HFK_HD void wait_turn() {
        if (pace_q8 == 0) return;
        const uint64_t now_q8 = (HFK_TICKS_100MHZ() - t0) << 8;
        if (now_q8 >= due_q8) {
            ++late_turns;
            if (now_q8 - due_q8 > max_late_q8) max_late_q8 = now_q8 - due_q8;
        } else {
            for (uint32_t spin = 0; spin < (1u << 16) && ((HFK_TICKS_100MHZ() - t0) << 8) < due_q8; ++spin) {
                HFK_NAP();
            }
        }
        ++turns;
        due_q8 += pace_q8;
    }

    // Pace report: eight 64-bit words per workgroup at report + 8 * bid, written by lane 0 when the
    // workgroup has finished: ticks it ran, ticks its schedule allotted (the time its next turn
    // would have come), turns, turns that began late, largest delay in ticks, the interval in 1/256
    // ticks; two words unused. A launch that holds its pace ends with ran <= allotted.
    HFK_HD void report(uint64_t* out, uint32_t bid, uint32_t tid) const {
        if (out == nullptr || pace_q8 == 0 || tid != 0) return;
        HFK_GLOBAL uint64_t* row = reinterpret_cast<HFK_GLOBAL uint64_t*>(reinterpret_cast<uint64_t>(out)) + 8 * (uint64_t)bid;
        row[0] = HFK_TICKS_100MHZ() - t0;
        row[1] = due_q8 >> 8;
        row[2] = turns;
        row[3] = late_turns;
        row[4] = max_late_q8 >> 8;
        row[5] = pace_q8;
        row[6] = 0;
        row[7] = 0;
    }

    // End of a workgroup of a launch whose pace is set between launches (see pace_factor): adds its
    // account to the launch's, and the last workgroup settles the factor for the next launch.
    HFK_HD void settle(uint32_t* state, uint32_t factor, uint32_t nb, uint32_t tid) const {
#if defined(__HIP_DEVICE_COMPILE__)
        if (state == nullptr || pace_q8 == 0 || tid != 0) return;
        atomicAdd(&state[1], turns);
        atomicAdd(&state[2], late_turns);
        if (((HFK_TICKS_100MHZ() - t0) << 8) > due_q8 + 2ull * pace_q8) atomicAdd(&state[4], 1u);
        __threadfence();
        if (atomicAdd(&state[3], 1u) + 1u >= nb) {   // >=: counts mixed up by overlapping launches still get cleared
            __threadfence();
            const uint32_t all_turns = atomicAdd(&state[1], 0u), all_late = atomicAdd(&state[2], 0u);
            const uint32_t behind = atomicAdd(&state[4], 0u);
            const uint32_t late_per_65536 = all_turns != 0 ? (uint32_t)(((uint64_t)all_late << 16) / all_turns) : 0u;
            HFK_GLOBAL uint32_t* g = reinterpret_cast<HFK_GLOBAL uint32_t*>(reinterpret_cast<uint64_t>(state));
            g[0] = next_pace_factor(factor, late_per_65536, behind != 0);
            g[1] = 0;
            g[2] = 0;
            g[3] = 0;
            g[4] = 0;
            g[5] = g[5] + 1;
            g[6] = late_per_65536;
        }
#else
        (void)state; (void)factor; (void)nb; (void)tid;
#endif
    }
};

// Block tables and plane-address tables are read, never written, by the kernel that uses them, and
// every lane of a workgroup reads the same entry. Reading them through the constant address space
// tells the compiler both facts, so it uses scalar loads: they are counted apart from the vector
// loads and stores, and a table lookup no longer waits for the workgroup's outstanding stores to
// drain (which, toward host memory, takes microseconds and sits on the critical path of a
// workgroup that keeps little in flight).
#if defined(__HIP_DEVICE_COMPILE__)
#define HFK_CONSTANT __attribute__((address_space(4)))
#else
#define HFK_CONSTANT
#endif

template <typename T>
HFK_HD T table_entry(const T* table, uint64_t index) {
    return reinterpret_cast<const HFK_CONSTANT T*>(reinterpret_cast<uint64_t>(table))[index];
}

// NT bit0: non-temporal loads, bit1: non-temporal stores.
template <typename V>
HFK_HD const HFK_GLOBAL V* global_in(uint64_t addr) {
    return reinterpret_cast<const HFK_GLOBAL V*>(addr);
}

template <typename V>
HFK_HD HFK_GLOBAL V* global_out(uint64_t addr) {
    return reinterpret_cast<HFK_GLOBAL V*>(addr);
}

template <int NT, typename V>
HFK_HD V load_unit(const HFK_GLOBAL V* p) {
    if constexpr ((NT & 1) != 0) {
        return __builtin_nontemporal_load(p);
    } else {
        return *p;
    }
}

template <int NT, typename V>
HFK_HD void store_unit(HFK_GLOBAL V* p, V v) {
    if constexpr ((NT & 2) != 0) {
        __builtin_nontemporal_store(v, p);
    } else {
        *p = v;
    }
}

// Byte k of a unit, without taking the address of a register value.
HFK_HD uint8_t unit_byte(uint8_t v, uint32_t) { return v; }
HFK_HD uint8_t unit_byte(uint32_t v, uint32_t k) { return (uint8_t)(v >> (8u * k)); }
HFK_HD uint8_t unit_byte(vec16 v, uint32_t k) {
    const uint32_t word = (k < 4) ? v.x : (k < 8) ? v.y : (k < 12) ? v.z : v.w;
    return (uint8_t)(word >> (8u * (k & 3u)));
}

// ---------------------------------------------------------------------------
// Block copy: tiles (plane, pair) of block_bytes bytes, each cut into chunks of
// 256 * UNROLL vectors; one workgroup iteration moves one chunk.
// Serves the block-table swap (both directions), the multi-plane block gather
// and the wide-row case of the row gather.
// ---------------------------------------------------------------------------
template <typename IdT>
struct BlockCopyArgs {
    const uint64_t* dst_planes;  // device array of plane base addresses, or null ->
    const uint64_t* src_planes;  //   plane p starts at {dst,src}_base + p * {dst,src}_plane_stride
    uint64_t dst_base;
    uint64_t src_base;
    uint64_t dst_plane_stride;
    uint64_t src_plane_stride;
    const IdT* src_ids;          // entry j at src_ids[j * id_stride]; null -> src block j
    const IdT* dst_ids;          // entry j at dst_ids[j * id_stride]; null -> dst block j
    uint32_t id_stride;
    uint32_t n_planes;
    uint32_t n_pairs;
    uint32_t chunks_per_block;
    uint64_t block_bytes;
    uint64_t src_stride;
    uint64_t dst_stride;
    uint64_t src_limit;          // block indices must be < limit (unsigned compare,
    uint64_t dst_limit;          // so negative ids are rejected as well)
    uint32_t n_work;             // n_planes * n_pairs * chunks_per_block
    uint32_t pace_q8;            // see Pacer; 0 = unpaced
    uint32_t zero_skipped;       // != 0: a pair whose source index is out of range but whose destination is
                                 // valid gets zeros written instead of being left alone (a staging buffer
                                 // must never hand an earlier transfer's bytes on to the host)
    // Run filter (RunFilter below): lets one block table be split between two movers, by the length
    // of the run of consecutive `run_ids` a pair belongs to. run_mode 0 = every pair. With
    // kListedPairs the split has been made beforehand and run_ids is this launch's list of pairs.
    uint32_t run_mode;
    uint32_t run_min;            // a run is "long" from this many consecutive ids on (listed: the table's length)
    const int64_t* run_ids;      // entry j at run_ids[j * id_stride] (listed: entry i at run_ids[i])
    uint64_t* pace_report;       // null, or where each workgroup of a paced launch leaves Pacer::report
    uint32_t* pace_state;        // null, or the library's eight words for a pace set between launches (pace_factor)
};

// Which pairs of a block table a launch moves, when the table is split by run length: pair j belongs to
// the maximal run of entries whose run_ids are consecutive (ids[i + 1] == ids[i] + 1) around it.
// kListedPairs: the launch moves the pairs a list names, in list order: run_ids[i] (stride 1) is the table
// index of the launch's i-th pair, n_pairs the length of the list, run_min the table's length (an entry
// that is not below it is skipped: a list is data, and its tail may be unfilled). A side without an id
// column (a staging buffer) is indexed by the position in the list, not by the table index.
enum RunFilter : uint32_t { kAllPairs = 0, kLongRunsOnly = 1, kShortRunsOnly = 2, kListedPairs = 3 };

// Length of the maximal run of consecutive ids around entry j, counted no further than `cap`: the
// result is min(cap, run length). The host uses the same function to decide which runs it copies,
// so the two sides of a split table agree by construction.
HFK_HD uint32_t run_length_capped(const int64_t* ids, uint32_t stride, uint32_t n, uint32_t j, uint32_t cap) {
    uint32_t len = 1;
    for (uint32_t i = j; i > 0 && len < cap &&
                         table_entry(ids, (uint64_t)(i - 1) * stride) + 1 == table_entry(ids, (uint64_t)i * stride); --i) {
        ++len;
    }
    for (uint32_t i = j; i + 1 < n && len < cap &&
                         table_entry(ids, (uint64_t)(i + 1) * stride) == table_entry(ids, (uint64_t)i * stride) + 1; ++i) {
        ++len;
    }
    return len;
}

// Where work item w of a block copy reads and writes. Everything here is uniform
// over the workgroup, so the compiler keeps it in scalar registers. Returns kSkip
// when the item's block indices are out of range or the run filter leaves the pair
// to another mover, kZeroFill when only the source index is out of range and the
// launch asked for zeros in that case (d_addr is then valid), kCopy otherwise.
enum ChunkAction : uint32_t { kSkip = 0, kCopy = 1, kZeroFill = 2 };

// SPLIT selects, at compile time, the variant that honours the run filter; kernels that move whole
// tables (the hot ones) are built without it and carry none of its code.
// LISTED: the launch's pairs are named by a list (kListedPairs).
template <typename IdT, bool SPLIT = false, bool LISTED = false>
HFK_HD ChunkAction resolve_chunk(const BlockCopyArgs<IdT>& a, uint32_t w, uint64_t& s_addr, uint64_t& d_addr,
                                 uint32_t& chunk) {
    chunk = w % a.chunks_per_block;
    const uint32_t tile = w / a.chunks_per_block;
    uint32_t pair, plane;
    if constexpr (!SPLIT) {             // plane-major: neighbouring workgroups stream neighbouring pairs of one plane
        pair = tile % a.n_pairs;
        plane = tile / a.n_pairs;
    } else {                            // pair-major: all items of a pair are adjacent, so a filtered-out
        pair = tile / a.n_planes;       // pair is stepped over at once (next_pair_item); the filter itself
        plane = tile % a.n_planes;      // is the caller's business (pair_selected), once per pair
    }
    // The four table reads (two block indices, two plane addresses) do not depend on one another and
    // none can fault (pair < n_pairs, plane < n_planes): they are all issued before the first
    // comparison, so a work item pays one scalar-load latency, not a chain of them. A workgroup that
    // keeps little in flight (the duplex swap: one vector per lane and direction) is as fast as its
    // iterations are short.
    uint64_t entry = pair;              // where the pair sits in the block table
    if constexpr (LISTED) {
        entry = (uint64_t)table_entry(a.run_ids, pair);
        if (entry >= a.run_min) return kSkip;
    }
    const uint64_t sb = a.src_ids ? (uint64_t)(int64_t)table_entry(a.src_ids, entry * a.id_stride) : (uint64_t)pair;
    const uint64_t db = a.dst_ids ? (uint64_t)(int64_t)table_entry(a.dst_ids, entry * a.id_stride) : (uint64_t)pair;
    const uint64_t s_plane = a.src_planes ? table_entry(a.src_planes, plane) : a.src_base + (uint64_t)plane * a.src_plane_stride;
    const uint64_t d_plane = a.dst_planes ? table_entry(a.dst_planes, plane) : a.dst_base + (uint64_t)plane * a.dst_plane_stride;
    s_addr = s_plane + sb * a.src_stride;
    d_addr = d_plane + db * a.dst_stride;
    if (db >= a.dst_limit) {
        return kSkip;
    }
    if (sb >= a.src_limit) {
        return a.zero_skipped != 0 ? kZeroFill : kSkip;
    }
    return kCopy;
}

// Whether the launch's run filter leaves pair `pair` to this launch.
template <typename IdT>
HFK_HD bool pair_selected(const BlockCopyArgs<IdT>& a, uint32_t pair) {
    const bool is_long = run_length_capped(a.run_ids, a.id_stride, a.n_pairs, pair, a.run_min) >= a.run_min;
    return is_long == (a.run_mode == kLongRunsOnly);
}

// In pair-major order (run filter on), the first work item after w that belongs to workgroup `bid`
// of `nb` (items bid, bid + nb, ...) and to a later pair than w does.
template <typename IdT>
HFK_HD uint64_t next_pair_item(const BlockCopyArgs<IdT>& a, uint64_t w, uint32_t bid, uint32_t nb) {
    const uint64_t per_pair = (uint64_t)a.n_planes * a.chunks_per_block;
    const uint64_t first = (w / per_pair + 1) * per_pair;             // first item of the next pair
    return first + ((uint64_t)bid + nb - first % nb) % nb;            // >= first, congruent to bid mod nb
}

// U loads, then U stores, 256 vectors apart: the straight-line core of every copy.
template <int U, int NT>
HFK_HD void copy_steps(const HFK_GLOBAL vec16* sv, HFK_GLOBAL vec16* dv) {
    vec16 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        v[u] = load_unit<NT>(sv + u * kWorkgroupLanes);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        store_unit<NT>(dv + u * kWorkgroupLanes, v[u]);
    }
}

// The last, short chunk of a block: `remaining` (< 2 * U * 256, uniform over the workgroup) vectors
// from sv/dv on (which already include the lane's offset). Cut into pieces of U, U/2, ... 1 full
// steps and one guarded step, each piece straight-line code with its loads ahead of its stores, so a
// tail needs no more registers than a full chunk and all branches but the last are uniform.
template <int U, int NT>
HFK_HD void copy_tail(const HFK_GLOBAL vec16* sv, HFK_GLOBAL vec16* dv, uint64_t remaining, uint32_t tid) {
    if (remaining >= (uint64_t)U * kWorkgroupLanes) {
        copy_steps<U, NT>(sv, dv);
        sv += U * kWorkgroupLanes;
        dv += U * kWorkgroupLanes;
        remaining -= (uint64_t)U * kWorkgroupLanes;
    }
    if constexpr (U > 1) {
        copy_tail<U / 2, NT>(sv, dv, remaining, tid);
    } else {
        if (tid < remaining) {
            store_unit<NT>(dv, load_unit<NT>(sv));
        }
    }
}

// Copies chunk `chunk` (256 * UNROLL vectors) of one block of block_bytes bytes.
template <int UNROLL, int NT>
HFK_HD void copy_chunk(uint64_t s_addr, uint64_t d_addr, uint64_t block_bytes, uint32_t chunk, uint32_t tid) {
    constexpr uint32_t kChunkVecs = kWorkgroupLanes * UNROLL;
    constexpr uint64_t kChunkBytes = (uint64_t)kChunkVecs * 16u;
    if (((s_addr | d_addr | block_bytes) & 15u) == 0) {
        const uint64_t block_vecs = block_bytes >> 4;
        const uint64_t first = (uint64_t)chunk * kChunkVecs;
        const HFK_GLOBAL vec16* sv = global_in<vec16>(s_addr) + first + tid;
        HFK_GLOBAL vec16* dv = global_out<vec16>(d_addr) + first + tid;
        if (first + kChunkVecs <= block_vecs) {
            copy_steps<UNROLL, NT>(sv, dv);
        } else if (first < block_vecs) {
            copy_tail<(UNROLL > 1 ? UNROLL / 2 : 1), NT>(sv, dv, block_vecs - first, tid);
        }
    } else {
        // Blocks that are not 16-byte aligned/sized: same chunk, narrower units.
        const uint64_t lo = (uint64_t)chunk * kChunkBytes;
        const uint64_t hi = (lo + kChunkBytes < block_bytes) ? lo + kChunkBytes : block_bytes;
        if (((s_addr | d_addr | block_bytes) & 3u) == 0) {
            const HFK_GLOBAL uint32_t* s4 = global_in<uint32_t>(s_addr);
            HFK_GLOBAL uint32_t* d4 = global_out<uint32_t>(d_addr);
            for (uint64_t o = (lo >> 2) + tid; o < (hi >> 2); o += kWorkgroupLanes) {
                d4[o] = s4[o];
            }
        } else {
            const HFK_GLOBAL uint8_t* s1 = global_in<uint8_t>(s_addr);
            HFK_GLOBAL uint8_t* d1 = global_out<uint8_t>(d_addr);
            for (uint64_t o = lo + tid; o < hi; o += kWorkgroupLanes) {
                d1[o] = s1[o];
            }
        }
    }
}

// Writes zeros over chunk `chunk` of one block (same chunking as copy_chunk).
template <int UNROLL, int NT>
HFK_HD void zero_chunk(uint64_t d_addr, uint64_t block_bytes, uint32_t chunk, uint32_t tid) {
    constexpr uint32_t kChunkVecs = kWorkgroupLanes * UNROLL;
    constexpr uint64_t kChunkBytes = (uint64_t)kChunkVecs * 16u;
    if (((d_addr | block_bytes) & 15u) == 0) {
        const uint64_t block_vecs = block_bytes >> 4;
        const uint64_t lane_first = (uint64_t)chunk * kChunkVecs + tid;
        HFK_GLOBAL vec16* dv = global_out<vec16>(d_addr) + lane_first;
        const vec16 zero = {0u, 0u, 0u, 0u};
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (lane_first + (uint64_t)u * kWorkgroupLanes < block_vecs) {
                store_unit<NT>(dv + u * kWorkgroupLanes, zero);
            }
        }
    } else {
        const uint64_t lo = (uint64_t)chunk * kChunkBytes;
        const uint64_t hi = (lo + kChunkBytes < block_bytes) ? lo + kChunkBytes : block_bytes;
        HFK_GLOBAL uint8_t* d1 = global_out<uint8_t>(d_addr);
        for (uint64_t o = lo + tid; o < hi; o += kWorkgroupLanes) {
            d1[o] = 0;
        }
    }
}

// SPLIT: the launch moves only the pairs its run filter selects (a.run_mode must then be
// kLongRunsOnly or kShortRunsOnly); without it a.run_mode must be kAllPairs.
// PACED: the launch may be paced (a.pace_q8); kernels that never are (everything HBM-bound) are built
// without it and carry none of the pacer's code: one workgroup per 4 KiB chunk pays for every
// instruction of its prologue.
// LISTED: the launch's pairs come from a list (a.run_mode must be kListedPairs); not together with SPLIT.
template <typename IdT, int UNROLL, int NT, bool SPLIT = false, bool PACED = true, bool LISTED = false>
HFK_HD void block_copy_body(const BlockCopyArgs<IdT>& a, uint32_t bid, uint32_t nb, uint32_t tid) {
    static_assert(!(SPLIT && LISTED), "a launch either filters the table's pairs or is handed a list of them");
    const uint32_t factor = PACED ? pace_factor(a.pace_state) : kPaceFactorOne;
    Pacer pacer(PACED ? (uint32_t)(((uint64_t)a.pace_q8 * factor) >> 16) : 0u, bid, nb);
    uint64_t id = bid;                  // 64-bit so that id + nb cannot wrap
    uint32_t judged_pair = 0xffffffffu; // SPLIT: the pair the filter was last evaluated for, and what it said
    bool judged_selected = false;       // (a workgroup's consecutive items mostly belong to one pair)
    while (id < a.n_work) {
        const uint64_t w = id;
        uint64_t s_addr = 0, d_addr = 0;
        uint32_t chunk = 0;
        if constexpr (SPLIT) {
            const uint32_t pair = (uint32_t)(w / ((uint64_t)a.n_planes * a.chunks_per_block));
            if (pair != judged_pair) {
                judged_pair = pair;
                judged_selected = pair_selected(a, pair);
            }
            if (!judged_selected) {
                id = next_pair_item(a, w, bid, nb);
                continue;
            }
        }
        const ChunkAction what = resolve_chunk<IdT, SPLIT, LISTED>(a, (uint32_t)w, s_addr, d_addr, chunk);
        if (what == kSkip) {            // moves nothing, so it takes no turn on the link either
            id = SPLIT ? next_pair_item(a, w, bid, nb) : id + nb;
            continue;
        }
        if constexpr (PACED) pacer.wait_turn();
        if (what == kCopy) {
            copy_chunk<UNROLL, NT>(s_addr, d_addr, a.block_bytes, chunk, tid);
        } else {
            zero_chunk<UNROLL, NT>(d_addr, a.block_bytes, chunk, tid);
        }
        id += nb;
    }
    if constexpr (PACED) {
        pacer.report(a.pace_report, bid, tid);
        pacer.settle(a.pace_state, factor, nb, tid);
    }
}

// ---------------------------------------------------------------------------
// Two block copies in one launch, meant for a swap-out (HBM -> host) and a swap-in
// (host -> HBM) that should share the PCIe link, which is full duplex. Every
// workgroup iteration takes one chunk of each copy and issues the loads of both
// before the stores of either, so reads from the host and writes to the host are
// in flight together and the two directions advance in lock step. Two independent
// launches on two streams reach 67-86 GB/s summed on MI355X depending on how their
// grids happen to interleave; this reaches 97-100 GB/s.
// `second` should be the copy that reads host memory: its loads are issued first.
// ---------------------------------------------------------------------------
struct DuplexCopyArgs {
    BlockCopyArgs<int64_t> first;
    BlockCopyArgs<int64_t> second;
    uint32_t n_work;  // max(first.n_work, second.n_work)
    uint32_t pace_q8; // see Pacer: one turn per iteration (one chunk of each copy); 0 = unpaced
};

template <int UNROLL, int NT>
HFK_HD void duplex_copy_body(const DuplexCopyArgs& a, uint32_t bid, uint32_t nb, uint32_t tid) {
    constexpr uint32_t kChunkVecs = kWorkgroupLanes * UNROLL;
    Pacer pacer(a.pace_q8, bid, nb);
    for (uint64_t w64 = bid; w64 < a.n_work; w64 += nb) {   // 64-bit counter: w + nb cannot wrap
        const uint32_t w = (uint32_t)w64;
        pacer.wait_turn();
        uint64_t s0 = 0, d0 = 0, s1 = 0, d1 = 0;
        uint32_t c0 = 0, c1 = 0;
        const bool v0 = w < a.first.n_work && resolve_chunk(a.first, w, s0, d0, c0) == kCopy;
        const bool v1 = w < a.second.n_work && resolve_chunk(a.second, w, s1, d1, c1) == kCopy;
        const bool fast0 = v0 && ((s0 | d0 | a.first.block_bytes) & 15u) == 0 &&
                           ((uint64_t)c0 + 1) * kChunkVecs <= (a.first.block_bytes >> 4);
        const bool fast1 = v1 && ((s1 | d1 | a.second.block_bytes) & 15u) == 0 &&
                           ((uint64_t)c1 + 1) * kChunkVecs <= (a.second.block_bytes >> 4);
        if (fast0 && fast1) {
            const HFK_GLOBAL vec16* sv0 = global_in<vec16>(s0) + (uint64_t)c0 * kChunkVecs + tid;
            HFK_GLOBAL vec16* dv0 = global_out<vec16>(d0) + (uint64_t)c0 * kChunkVecs + tid;
            const HFK_GLOBAL vec16* sv1 = global_in<vec16>(s1) + (uint64_t)c1 * kChunkVecs + tid;
            HFK_GLOBAL vec16* dv1 = global_out<vec16>(d1) + (uint64_t)c1 * kChunkVecs + tid;
            vec16 x[UNROLL], y[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                y[u] = load_unit<NT>(sv1 + u * kWorkgroupLanes);  // host reads first: longest latency
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                x[u] = load_unit<NT>(sv0 + u * kWorkgroupLanes);
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                store_unit<NT>(dv0 + u * kWorkgroupLanes, x[u]);
            }
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) {
                store_unit<NT>(dv1 + u * kWorkgroupLanes, y[u]);
            }
        } else {
            // Tail chunks, odd alignments, or only one of the copies has work left.
            if (v1) copy_chunk<UNROLL, NT>(s1, d1, a.second.block_bytes, c1, tid);
            if (v0) copy_chunk<UNROLL, NT>(s0, d0, a.first.block_bytes, c0, tid);
        }
    }
}

// ---------------------------------------------------------------------------
// Flat row gather for narrow rows (below one chunk): the destination is one
// contiguous array of n_ids * row_units units of type V; lane g of the flat
// index space copies unit (g % row_units) of row ids[g / row_units].
// Consecutive lanes read consecutive units of a row, so a 1 KiB row is exactly
// one wavefront request and shorter rows share a wavefront.
// ---------------------------------------------------------------------------
template <typename IdT>
struct FlatGatherArgs {
    uint64_t table;       // address; row r at table + r * row_units * sizeof(V)
    uint64_t dst;
    const IdT* ids;
    uint64_t total_units; // n_ids * row_units
    uint32_t row_units;
    uint64_t row_limit;   // ids must be < limit (unsigned compare)
    uint32_t n_work;      // ceil(total_units / (256 * UNROLL))
};

template <typename V, typename IdT, typename IndexT, int UNROLL, int NT>
HFK_HD void flat_gather_body(const FlatGatherArgs<IdT>& a, uint32_t bid, uint32_t nb, uint32_t tid) {
    constexpr uint32_t kChunkUnits = kWorkgroupLanes * UNROLL;
    const HFK_GLOBAL V* table = global_in<V>(a.table);
    HFK_GLOBAL V* dst = global_out<V>(a.dst);
    const IndexT total = (IndexT)a.total_units;
    const IndexT row_units = (IndexT)a.row_units;

    for (uint64_t w64 = bid; w64 < a.n_work; w64 += nb) {
        const uint32_t w = (uint32_t)w64;
        const IndexT g0 = (IndexT)w * kChunkUnits + tid;
        V v[UNROLL];
        bool ok[UNROLL];
        uint64_t id[UNROLL];
        IndexT col[UNROLL];
        // All row ids first, then all rows: the id loads do not wait for one another (one memory
        // round trip per work item, not one per unit).
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            const IndexT g = g0 + (IndexT)u * kWorkgroupLanes;
            id[u] = ~0ull;   // never below row_limit
            col[u] = 0;
            if (g < total) {
                const IndexT row = g / row_units;
                col[u] = g - row * row_units;
                id[u] = (uint64_t)(int64_t)a.ids[row];
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            ok[u] = id[u] < a.row_limit;
            if (ok[u]) {
                v[u] = load_unit<NT>(table + id[u] * a.row_units + col[u]);
            }
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
            if (ok[u]) {
                store_unit<NT>(dst + (uint64_t)(g0 + (IndexT)u * kWorkgroupLanes), v[u]);
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Layout-converting transfer. The "packed" side holds whole blocks [T, L, H, row]
// (pinned host memory in normal use), the "layered" side holds, per layer l, a
// cache of blocks [H, T, row] reached through layer_ptrs[l]:
//   layered[l][db][(h*T + t), row]  <->  packed[pb][((t*L + l)*H + h), row]
// Lanes walk the packed side in memory order, so the side that crosses the PCIe
// link is always fully coalesced; a row (D * elem_bytes bytes) stays contiguous
// on the layered side, so HBM sees row-sized runs. TO_PACKED picks the direction.
// One block with no table is the reference's multi_layer_block_transfer.
// ---------------------------------------------------------------------------
struct TransposeArgs {
    const uint64_t* layer_ptrs;  // device array of L addresses (block 0 of each layer's cache)
    uint64_t packed;             // address of packed block 0
    const int64_t* pairs;        // [n_pairs, 2] = (packed_block, layered_block); null -> (0, 0)
    uint64_t packed_stride;      // bytes between packed blocks
    uint64_t layered_stride;     // bytes between blocks inside one layer's cache
    uint64_t packed_limit;       // block indices must be < limit (unsigned compare)
    uint64_t layered_limit;
    uint32_t n_pairs;
    uint32_t chunks_per_block;   // ceil(total_units / (256 * UNROLL))
    uint32_t T;
    uint32_t L;
    uint32_t H;
    uint32_t row_units;          // D * elem_bytes / sizeof(V)
    uint32_t total_units;        // T * L * H * row_units, per block
    uint32_t n_work;             // n_pairs * chunks_per_block
    uint32_t pace_q8;            // see Pacer; 0 = unpaced
    uint32_t tile_tokens;        // tiled form only (plan_transpose_tiles): tokens and packed rows per tile;
    uint32_t tile_rows;          // chunks_per_block is then the number of tiles per block
    uint64_t mirror;             // 0, or (transfer out of the packed side, bodies built with MIRROR) the address of a
                                 // second copy of the packed blocks, same strides: every unit read is also written there
};

// Where the body finds layer l's address. The layer differs from lane to lane (a 128-byte row is 8
// lanes wide), so this cannot be a scalar load, and as a vector load from the device array it would
// make every work item wait for the stores of the one before it (vector loads and stores share one
// counter) -- microseconds, when those stores go to host memory. The kernels therefore copy the
// table into LDS once and hand the body an accessor over that copy, whose reads are counted with
// the scalar loads; this accessor, over the array itself, serves tables too long for the LDS copy
// and the CPU walk of the bodies.
struct LayerTableInMemory {
    const uint64_t* layer_ptrs;
    HFK_HD uint64_t operator()(uint32_t l) const { return layer_ptrs[l]; }
};

HFK_HD void unit_from_bytes(const HFK_GLOBAL uint8_t* p, uint8_t& v) { v = p[0]; }
HFK_HD void unit_from_bytes(const HFK_GLOBAL uint8_t* p, uint32_t& v) {
    v = (uint32_t)p[0] | ((uint32_t)p[1] << 8) | ((uint32_t)p[2] << 16) | ((uint32_t)p[3] << 24);
}
HFK_HD void unit_from_bytes(const HFK_GLOBAL uint8_t* p, vec16& v) {
    uint32_t w[4];
    for (int i = 0; i < 4; ++i) unit_from_bytes(p + 4 * i, w[i]);
    v.x = w[0];
    v.y = w[1];
    v.z = w[2];
    v.w = w[3];
}

// One work item of the transfer: chunk `chunk` of the pair's packed block.
struct TransposeItem {
    uint64_t packed_addr;   // address of the pair's packed block
    uint64_t layered_off;   // byte offset of the pair's block inside every layer's cache
    uint64_t g0;            // this lane's first unit within the packed block
};

// Where work item w lives; false when the pair's block indices are out of range.
HFK_HD bool transpose_item(const TransposeArgs& a, uint64_t w64, uint32_t tid, uint32_t chunk_units, TransposeItem& it) {
    const uint32_t w = (uint32_t)w64;
    const uint32_t chunk = w % a.chunks_per_block;
    const uint32_t pair = w / a.chunks_per_block;
    const uint64_t pb = a.pairs ? (uint64_t)table_entry(a.pairs, 2 * (uint64_t)pair) : 0;
    const uint64_t db = a.pairs ? (uint64_t)table_entry(a.pairs, 2 * (uint64_t)pair + 1) : 0;
    if (pb >= a.packed_limit || db >= a.layered_limit) {
        return false;
    }
    it.packed_addr = a.packed + pb * a.packed_stride;
    it.layered_off = db * a.layered_stride;
    it.g0 = (uint64_t)chunk * chunk_units + tid;
    return true;
}

// The layered-side address of each of the lane's UNROLL units (0 past the end of the block).
template <typename V, int UNROLL, typename LayerTable>
HFK_HD void transpose_addresses(const TransposeArgs& a, const TransposeItem& it, const LayerTable& layer_address,
                                uint64_t (&layered_addr)[UNROLL]) {
    const uint32_t LH = a.L * a.H;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g64 = it.g0 + (uint64_t)u * kWorkgroupLanes;
        layered_addr[u] = 0;
        if (g64 < a.total_units) {
            const uint32_t g = (uint32_t)g64;
            const uint32_t r = g / a.row_units;      // packed row = (t*L + l)*H + h
            const uint32_t col = g - r * a.row_units;
            const uint32_t t = r / LH;
            const uint32_t lh = r - t * LH;
            const uint32_t l = lh / a.H;
            const uint32_t h = lh - l * a.H;
            const uint64_t unit = ((uint64_t)h * a.T + t) * a.row_units + col;
            layered_addr[u] = layer_address(l) + it.layered_off + unit * sizeof(V);
        }
    }
}

// Loads the lane's units of one work item from the layered side (TO_PACKED) or the packed side.
template <typename V, int UNROLL, int NT, bool TO_PACKED>
HFK_HD void transpose_load(const TransposeArgs& a, const TransposeItem& it, const uint64_t (&layered_addr)[UNROLL], V (&v)[UNROLL]) {
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g64 = it.g0 + (uint64_t)u * kWorkgroupLanes;
        if (g64 < a.total_units) {
            if constexpr (TO_PACKED) {
                if ((layered_addr[u] & (sizeof(V) - 1)) == 0) {
                    v[u] = load_unit<NT>(global_in<V>(layered_addr[u]));
                } else {  // layer cache not aligned to the unit: byte loads keep it correct
                    unit_from_bytes(global_in<uint8_t>(layered_addr[u]), v[u]);
                }
            } else {
                v[u] = load_unit<NT>(global_in<V>(it.packed_addr) + g64);
            }
        }
    }
}

// MIRROR: every unit is also written, as it is, to the second copy of the packed blocks at a.mirror (a variant of
// its own, so that the ordinary transfer carries none of it: a branch per unit cost its 24 x 2 launch 2 %).
template <typename V, int UNROLL, int NT, bool TO_PACKED, bool MIRROR = false>
HFK_HD void transpose_store(const TransposeArgs& a, const TransposeItem& it, const uint64_t (&layered_addr)[UNROLL], const V (&v)[UNROLL]) {
    static_assert(!(MIRROR && TO_PACKED), "only a transfer out of the packed side can mirror what it reads");
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
        const uint64_t g64 = it.g0 + (uint64_t)u * kWorkgroupLanes;
        if (g64 < a.total_units) {
            if constexpr (TO_PACKED) {
                store_unit<NT>(global_out<V>(it.packed_addr) + g64, v[u]);
            } else {
                if ((layered_addr[u] & (sizeof(V) - 1)) == 0) {
                    store_unit<NT>(global_out<V>(layered_addr[u]), v[u]);
                } else {  // byte stores for a misaligned layer cache
                    HFK_GLOBAL uint8_t* d1 = global_out<uint8_t>(layered_addr[u]);
                    for (uint32_t k = 0; k < sizeof(V); ++k) {
                        d1[k] = unit_byte(v[u], k);
                    }
                }
                if constexpr (MIRROR) {   // the packed block as it is, for the caller's staging buffer
                    store_unit<NT>(global_out<V>(a.mirror + (it.packed_addr - a.packed)) + g64, v[u]);
                }
            }
        }
    }
}

template <typename V, int UNROLL, int NT, bool TO_PACKED, bool MIRROR = false, typename LayerTable>
HFK_HD void transpose_body(const TransposeArgs& a, uint32_t bid, uint32_t nb, uint32_t tid, const LayerTable& layer_address) {
    constexpr uint32_t kChunkUnits = kWorkgroupLanes * UNROLL;
    Pacer pacer(a.pace_q8, bid, nb);
    for (uint64_t w64 = bid; w64 < a.n_work; w64 += nb) {
        TransposeItem it;
        if (!transpose_item(a, w64, tid, kChunkUnits, it)) {
            continue;
        }
        pacer.wait_turn();
        V v[UNROLL];
        uint64_t layered_addr[UNROLL];
        transpose_addresses<V, UNROLL>(a, it, layer_address, layered_addr);
        transpose_load<V, UNROLL, NT, TO_PACKED>(a, it, layered_addr, v);
        transpose_store<V, UNROLL, NT, TO_PACKED, MIRROR>(a, it, layered_addr, v);
    }
}

template <typename V, int UNROLL, int NT, bool TO_PACKED, bool MIRROR = false>
HFK_HD void transpose_body(const TransposeArgs& a, uint32_t bid, uint32_t nb, uint32_t tid) {
    transpose_body<V, UNROLL, NT, TO_PACKED, MIRROR>(a, bid, nb, tid, LayerTableInMemory{a.layer_ptrs});
}

// ---------------------------------------------------------------------------
// The transfer toward the packed side, tiled through LDS. The direct body above reads the layered
// side in rows: with 128-byte rows a wavefront's load touches eight different (layer, head) places,
// and toward a packed pool in host memory that form stays 2-3 GB/s under what the link takes from a
// kernel that reads long runs. Here a work item is a tile of 64 / row_units tokens x 4 * U packed rows:
// each wavefront load reads ONE (layer, head) run of 64 units (1 KiB: the tile's tokens are
// consecutive on the layered side), the tile is laid out in LDS in packed order, and each wavefront
// store writes 1 KiB of that order; per token the tile's rows are contiguous on the packed side
// (4 * U rows). Nothing here is indexed per lane by division: layer and head are uniform over a
// wavefront. Needs: 16-byte units, row_units a power of two <= 64, T a multiple of 64 / row_units,
// L * H a multiple of 4 * U (plan_transpose_tiles checks). A workgroup runs load phase, barrier, store
// phase, barrier per tile; the two phases are separate functions so that a CPU walk can do the same.
struct TransposeTile {
    uint64_t packed_addr;   // address of the pair's packed block
    uint64_t layered_off;   // byte offset of the pair's block inside every layer's cache
    uint32_t t0;            // first token of the tile
    uint32_t r0;            // first packed row (l * H + h) of the tile
};

HFK_HD bool transpose_tile_item(const TransposeArgs& a, uint64_t w64, TransposeTile& it) {
    const uint32_t w = (uint32_t)w64;
    const uint32_t pair = w / a.chunks_per_block;
    const uint32_t rem = w - pair * a.chunks_per_block;
    const uint64_t pb = a.pairs ? (uint64_t)table_entry(a.pairs, 2 * (uint64_t)pair) : 0;
    const uint64_t db = a.pairs ? (uint64_t)table_entry(a.pairs, 2 * (uint64_t)pair + 1) : 0;
    if (pb >= a.packed_limit || db >= a.layered_limit) {
        return false;
    }
    const uint32_t row_groups = (a.L * a.H) / a.tile_rows;   // row group fastest: a token group's tiles are neighbours
    const uint32_t tg = rem / row_groups;
    it.packed_addr = a.packed + pb * a.packed_stride;
    it.layered_off = db * a.layered_stride;
    it.t0 = tg * a.tile_tokens;
    it.r0 = (rem - tg * row_groups) * a.tile_rows;
    return true;
}

// Load phase: the lane's U units of the tile, from the layered side into `tile` (64 * 4 * U units, packed order).
template <int U, int NT, typename LayerTable>
HFK_HD void transpose_tile_load(const TransposeArgs& a, const TransposeTile& it, uint32_t tid, const LayerTable& layer_address,
                                vec16* tile) {
    constexpr uint32_t R = 4 * U;
    const uint32_t wave = tid >> 6, lane = tid & 63u;
    const uint32_t tt = lane / a.row_units, col = lane - tt * a.row_units;
    vec16 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t r = it.r0 + wave * U + u;     // uniform over the wavefront
        const uint32_t l = r / a.H;
        const uint32_t h = r - l * a.H;
        const uint64_t addr = layer_address(l) + it.layered_off + (((uint64_t)h * a.T + it.t0) * a.row_units + lane) * sizeof(vec16);
        if ((addr & (sizeof(vec16) - 1)) == 0) {
            v[u] = load_unit<NT>(global_in<vec16>(addr));
        } else {  // layer cache not aligned to the unit: byte loads keep it correct
            unit_from_bytes(global_in<uint8_t>(addr), v[u]);
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        tile[(tt * R + wave * U + u) * a.row_units + col] = v[u];
    }
}

// Store phase: the tile, in packed order, to the packed side: 1 KiB per wavefront store.
template <int U, int NT>
HFK_HD void transpose_tile_store(const TransposeArgs& a, const TransposeTile& it, uint32_t tid, const vec16* tile) {
    const uint32_t wave = tid >> 6, lane = tid & 63u;
    const uint32_t LH = a.L * a.H;
    const uint32_t segment = 4 * U * a.row_units;   // units the tile holds per token, contiguous on the packed side
    HFK_GLOBAL vec16* packed = global_out<vec16>(it.packed_addr);
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t lin = (wave * U + u) * 64u + lane;
        const uint32_t tt = lin / segment;
        const uint32_t within = lin - tt * segment;
        store_unit<NT>(packed + (((uint64_t)(it.t0 + tt) * LH + it.r0) * a.row_units + within), tile[lin]);
    }
}

}  // namespace hfk
