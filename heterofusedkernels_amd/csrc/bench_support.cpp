// libhfk_bench.so: comparison paths for the benchmark only (not part of the product).
// The per-block copy loop is the conventional way to move a block table without a
// custom kernel: one hipMemcpyAsync per (plane, pair), which is also what the
// reference's caller-side loop amounts to (pcieThrough/tests/test_transfer_kernel.py:58-72).
#include <hip/hip_runtime_api.h>

#include <cstdint>

extern "C" __attribute__((visibility("default"))) int hfkb_memcpy_block_loop(
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
