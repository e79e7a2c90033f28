// libhfk_bench.so: comparison paths and yardsticks for the benchmark only (not part of the
// product, not installed with it).
//
//  * hfkb_memcpy_block_loop: the conventional way to move a block table without a custom kernel,
//    one hipMemcpyAsync per (plane, pair), which is also what the reference's caller-side loop
//    amounts to (pcieThrough/tests/test_transfer_kernel.py:58-72).
//  * hfkb_hbm_stream: what HBM gives a kernel of the block gather's shape (256-lane workgroups,
//    one workgroup per chunk of 256 * UNROLL 16-byte vectors, UNROLL loads before the first store)
//    when it only reads, only writes, or copies a contiguous buffer. The read-only and write-only
//    rates bound any copy: moving N bytes takes at least N / read_rate + N / write_rate.
//  * hfkb_host_read: reads pinned host memory and keeps only a checksum, either through the vector
//    memory path (what every copy kernel uses) or through the scalar (constant) path. A compute unit
//    returns the loads of each path in order, so a neighbour's loads queue behind host reads that
//    take microseconds; which neighbour suffers depends on which path it shares with them.
//  * hfkb_idle_resident: workgroups that touch no memory and only sleep for a bounded time. What a
//    kernel on another stream loses beside them is the price of sharing the GPU at all, the floor
//    under every figure measured beside a swap.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "hfk_bodies.h"

namespace {

using hfk::kWorkgroupLanes;
using hfk::vec16;

enum Mode { kRead = 0, kWrite = 1, kCopy = 2 };

typedef uint32_t u32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// One wavefront per 256-byte unit and turn: four 64-byte scalar loads, uniform over the wavefront.
template <int WAVES>
__global__ __launch_bounds__(64 * WAVES) void host_read_scalar_kernel(uint64_t host, uint64_t n_units, uint32_t* out) {
    typedef const __attribute__((address_space(4))) u32x16* constant_units;
    const uint32_t wave = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    const uint64_t first = (uint64_t)blockIdx.x * WAVES + wave, stride = (uint64_t)gridDim.x * WAVES;
    uint32_t acc = 0;
    for (uint64_t u = first; u < n_units; u += stride) {
        constant_units p = (constant_units)(host + u * 256);
        const u32x16 x = p[0] ^ p[1] ^ p[2] ^ p[3];
        acc ^= x[0] ^ x[5] ^ x[10] ^ x[15];
    }
    if ((threadIdx.x & 63u) == 0) out[first] = acc;   // an ordinary vector store
}

__global__ __launch_bounds__(256) void host_read_vector_kernel(const u32x4* host, uint64_t n_vec, uint32_t* out) {
    uint32_t acc = 0;
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < n_vec; i += (uint64_t)gridDim.x * 256) {
        const u32x4 v = __builtin_nontemporal_load(host + i);
        acc ^= v[0] ^ v[3];
    }
    out[blockIdx.x * 256 + threadIdx.x] = acc;
}

__global__ void idle_resident_kernel(uint64_t ticks) {
    const uint64_t t0 = wall_clock64();
    for (uint32_t spin = 0; spin < (1u << 24) && wall_clock64() - t0 < ticks; ++spin) {
        __builtin_amdgcn_s_sleep(20);
    }
}

template <int MODE, int UNROLL, int NT>
__global__ __launch_bounds__(256) void hbm_stream_kernel(uint64_t dst, uint64_t src, uint64_t n_chunks, uint32_t never) {
    constexpr uint64_t kChunkVecs = (uint64_t)kWorkgroupLanes * UNROLL;
    for (uint64_t w = blockIdx.x; w < n_chunks; w += gridDim.x) {
        const HFK_GLOBAL vec16* sv = hfk::global_in<vec16>(src) + w * kChunkVecs + threadIdx.x;
        HFK_GLOBAL vec16* dv = hfk::global_out<vec16>(dst) + w * kChunkVecs + threadIdx.x;
        if constexpr (MODE == kCopy) {
            hfk::copy_steps<UNROLL, NT>(sv, dv);
        } else if constexpr (MODE == kWrite) {
            const vec16 v = {(uint32_t)w, threadIdx.x, 0x5au, never};
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) hfk::store_unit<NT>(dv + u * kWorkgroupLanes, v);
        } else {
            vec16 v[UNROLL];
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) v[u] = hfk::load_unit<NT>(sv + u * kWorkgroupLanes);
            uint32_t acc = 0;
#pragma unroll
            for (int u = 0; u < UNROLL; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
            // The loads must not be optimised away; `never` is a value the data never xors to in
            // the benchmark (a buffer of equal bytes xors to 0), so nothing is ever written.
            if (acc == never) hfk::store_unit<NT>(dv, v[0]);
        }
    }
}

template <int MODE, int UNROLL>
void launch_nt(uint64_t dst, uint64_t src, uint64_t n_chunks, uint32_t grid, int nt, uint32_t lds, hipStream_t s) {
    if (lds > 65536u) {   // more than the default limit must be asked for per kernel
        if (nt) (void)hipFuncSetAttribute((const void*)hbm_stream_kernel<MODE, UNROLL, 3>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        else (void)hipFuncSetAttribute((const void*)hbm_stream_kernel<MODE, UNROLL, 0>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    }
    if (nt) hipLaunchKernelGGL((hbm_stream_kernel<MODE, UNROLL, 3>), dim3(grid), dim3(256), lds, s, dst, src, n_chunks, 0x9e3779b9u);
    else hipLaunchKernelGGL((hbm_stream_kernel<MODE, UNROLL, 0>), dim3(grid), dim3(256), lds, s, dst, src, n_chunks, 0x9e3779b9u);
}

template <int MODE>
int launch_unroll(uint64_t dst, uint64_t src, uint64_t bytes, int unroll, uint32_t workgroups, int nt, uint32_t lds, hipStream_t s) {
    const uint64_t chunk = (uint64_t)kWorkgroupLanes * 16u * (uint64_t)unroll;
    if (bytes == 0 || bytes % chunk != 0) return -2;
    const uint64_t n_chunks = bytes / chunk;
    if (n_chunks > 0x7fffffffull) return -3;
    const uint32_t grid = workgroups != 0 && workgroups < n_chunks ? workgroups : (uint32_t)n_chunks;
    switch (unroll) {
        case 1: launch_nt<MODE, 1>(dst, src, n_chunks, grid, nt, lds, s); break;
        case 2: launch_nt<MODE, 2>(dst, src, n_chunks, grid, nt, lds, s); break;
        case 4: launch_nt<MODE, 4>(dst, src, n_chunks, grid, nt, lds, s); break;
        case 8: launch_nt<MODE, 8>(dst, src, n_chunks, grid, nt, lds, s); break;
        case 16: launch_nt<MODE, 16>(dst, src, n_chunks, grid, nt, lds, s); break;
        default: return -4;
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? 0 : (int)e;
}

}  // namespace

extern "C" {

__attribute__((visibility("default"))) int hfkb_memcpy_block_loop(
    const uint64_t* dst_planes, const uint64_t* src_planes, const int64_t* pairs, uint32_t n_planes,
    uint64_t n_pairs, uint64_t block_bytes, uint64_t src_stride, uint64_t dst_stride, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    for (uint32_t p = 0; p < n_planes; ++p) {
        for (uint64_t j = 0; j < n_pairs; ++j) {
            const void* src = reinterpret_cast<const void*>(src_planes[p] + (uint64_t)pairs[2 * j] * src_stride);
            void* dst = reinterpret_cast<void*>(dst_planes[p] + (uint64_t)pairs[2 * j + 1] * dst_stride);
            hipError_t e = hipMemcpyAsync(dst, src, block_bytes, hipMemcpyDefault, s);
            if (e != hipSuccess) return static_cast<int>(e);
        }
    }
    return 0;
}

// Reads `bytes` (a multiple of 256) of device-mapped pinned host memory and leaves one checksum word
// per wavefront (scalar path: workgroups of 8 wavefronts) or per lane (vector path) in `out`, which
// must hold workgroups * 256 words.
__attribute__((visibility("default"))) int hfkb_host_read(int scalar_path, const void* host_mapped, uint64_t bytes,
                                                          uint32_t workgroups, uint32_t* out, void* stream) {
    if (host_mapped == nullptr || out == nullptr || workgroups == 0 || (bytes & 255u) != 0) return -1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (scalar_path) {
        hipLaunchKernelGGL(host_read_scalar_kernel<8>, dim3(workgroups), dim3(512), 0, s, (uint64_t)(uintptr_t)host_mapped,
                           bytes / 256, out);
    } else {
        hipLaunchKernelGGL(host_read_vector_kernel, dim3(workgroups), dim3(256), 0, s,
                           static_cast<const u32x4*>(host_mapped), bytes / 16, out);
    }
    return (int)hipGetLastError();
}

// `workgroups` x `lanes` that sleep until `ticks` of the 100 MHz counter have passed (at most a few
// seconds: the loop is bounded as well), then exit.
__attribute__((visibility("default"))) int hfkb_idle_resident(uint32_t workgroups, uint32_t lanes, uint64_t ticks,
                                                              void* stream) {
    if (workgroups == 0 || lanes == 0 || lanes > 1024 || ticks > 300000000ull) return -1;
    hipLaunchKernelGGL(idle_resident_kernel, dim3(workgroups), dim3(lanes), 0, static_cast<hipStream_t>(stream), ticks);
    return (int)hipGetLastError();
}

// mode 0: read `bytes` from src; 1: write `bytes` to dst; 2: copy src -> dst. Buffers are device
// memory, 16-byte aligned, `bytes` a multiple of the chunk (4096 * unroll). workgroups 0 = one per
// chunk. lds_bytes = dynamic LDS requested per workgroup, which the kernel does not use: it only
// bounds how many workgroups a compute unit holds at a time (160 KiB of LDS per unit).
__attribute__((visibility("default"))) int hfkb_hbm_stream(int mode, void* dst, const void* src, uint64_t bytes,
                                                           int unroll, uint32_t workgroups, int nontemporal,
                                                           uint32_t lds_bytes, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint64_t d = (uint64_t)(uintptr_t)dst, a = (uint64_t)(uintptr_t)src;
    if (((d | a) & 15u) != 0 || lds_bytes > 163840u) return -1;
    switch (mode) {
        case kRead: return launch_unroll<kRead>(d, a, bytes, unroll, workgroups, nontemporal, lds_bytes, s);
        case kWrite: return launch_unroll<kWrite>(d, a, bytes, unroll, workgroups, nontemporal, lds_bytes, s);
        case kCopy: return launch_unroll<kCopy>(d, a, bytes, unroll, workgroups, nontemporal, lds_bytes, s);
        default: return -4;
    }
}

}  // extern "C"
