// libpcie_through.so: the torch dispatcher ops of the pcie_through namespace.
//
// Schemas of the first three ops are those of the reference
// (pcieThrough/csrc/host/gather_torch.cpp:60,
//  pcieThrough/csrc/host/multi_layer_block_transfer_torch.cpp:113-114);
// multi_layer_block_table_transfer, swap_blocks, swap_blocks_duplex, swap_blocks_staged,
// swap_blocks_staged_static, swap_blocks_auto, gather_blocks and gather_into are additive. Every op unpacks its tensors into
// raw device-visible addresses, takes the current HIP stream of the device that
// owns the device-side tensor, and calls the C-ABI of libhfk_hip.so; nothing is
// allocated and nothing waits.
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <hip/hip_runtime_api.h>
#include <torch/library.h>

#include <optional>

#include "hfk.h"
#define HFK_MANAGED_MEM_NO_TORCH 1   // only the manager is used here; keeps pybind11 out of this library
#include "managed_mem.h"

namespace pciethrough {

namespace {

using managed_memory::HostRegisteredMemoryManager;

// `aiv` is the reference's AI-vector-core count. It is validated exactly as there
// (converted to uint32, zero rejected; gather_torch.cpp:32-36) and otherwise
// unused: the grid is sized from the GPU's CU count, and results never depended on it.
void check_aiv(const std::optional<int64_t>& aiv) {
    if (aiv.has_value()) {
        const uint32_t aivNum = static_cast<uint32_t>(aiv.value());
        TORCH_CHECK(aivNum > 0, "Number of AIV blocks should be positive.");
    }
}

// Address a kernel can use for the tensor's first element. Device tensors are used
// as they are; host tensors must be registered (heterofusedkernels.memory) or at
// least pinned. A pinned tensor that was never registered is resolved through the
// HIP runtime on every call and nothing is recorded for it: torch's pinned
// allocator recycles its blocks, so a recorded range could outlive the tensor.
// The reference passes an unchecked nullptr to the kernel here
// (gather_torch.cpp:51, multi_layer_block_transfer_torch.cpp:78).
// `in_host`, when given, is told where the memory lives (the library would otherwise ask the runtime).
void* device_visible(const at::Tensor& t, const char* what, bool* in_host = nullptr) {
    if (in_host != nullptr) *in_host = !t.is_cuda();
    if (t.is_cuda()) return t.data_ptr();
    TORCH_CHECK(t.device().is_cpu(), what, ": unsupported device ", t.device());
    void* dev = HostRegisteredMemoryManager::GetInstance().getDevicePtr(t.data_ptr());
    if (dev != nullptr) return dev;
    // (an op call always has a device tensor among its arguments, so torch's device hooks are up
    // and is_pinned() answers truthfully)
    TORCH_CHECK(t.is_pinned(), what,
                ": host tensor is neither registered with heterofusedkernels.memory nor pinned");
    const hipError_t e = hipHostGetDevicePointer(&dev, t.data_ptr(), 0);
    if (e != hipSuccess) (void)hipGetLastError();
    TORCH_CHECK(e == hipSuccess && dev != nullptr, what, ": no device-visible address for the pinned host tensor: ",
                hipGetErrorString(e));
    return dev;
}

hfk_stream_t current_stream() {
    return static_cast<hfk_stream_t>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
}

void check_status(int rc, const char* entry) {
    TORCH_CHECK(rc == 0, entry, " failed: ", hfk_status_string(rc), " (", rc, ")");
}

uint32_t flag_bits(int64_t flags, const char* op) {
    TORCH_CHECK(flags >= 0 && flags <= 0xffffffffLL, op, ": flags out of range");
    return static_cast<uint32_t>(flags);
}

uint32_t workgroup_cap(const std::optional<int64_t>& workgroups) {
    if (!workgroups.has_value()) return 0;
    TORCH_CHECK(workgroups.value() >= 0 && workgroups.value() <= 0x7fffffff, "workgroups out of range");
    return static_cast<uint32_t>(workgroups.value());
}

struct BlockGeometry {
    uint32_t T, L, H, D, elem;
};

BlockGeometry block_geometry(const at::Tensor& hostBlockCache) {
    TORCH_CHECK(hostBlockCache.dim() == 4,
                "hostBlockCache must be [blockSize, layers, heads, headDims], got ", hostBlockCache.dim(),
                " dims");
    TORCH_CHECK(hostBlockCache.is_contiguous(), "hostBlockCache must be contiguous");
    for (int i = 0; i < 4; ++i) {
        TORCH_CHECK(hostBlockCache.size(i) <= 0xffffffffLL, "hostBlockCache dimension ", i, " too large");
    }
    return {static_cast<uint32_t>(hostBlockCache.size(0)), static_cast<uint32_t>(hostBlockCache.size(1)),
            static_cast<uint32_t>(hostBlockCache.size(2)), static_cast<uint32_t>(hostBlockCache.size(3)),
            static_cast<uint32_t>(hostBlockCache.element_size())};
}

void check_layer_ptrs(const at::Tensor& deviceBlockCachePtrs, uint32_t layers) {
    TORCH_CHECK(deviceBlockCachePtrs.is_cuda(), "deviceBlockCachePtrs must be a device tensor");
    TORCH_CHECK(deviceBlockCachePtrs.scalar_type() == at::kLong, "deviceBlockCachePtrs must be int64");
    TORCH_CHECK(deviceBlockCachePtrs.is_contiguous(), "deviceBlockCachePtrs must be contiguous");
    TORCH_CHECK(deviceBlockCachePtrs.numel() >= layers, "deviceBlockCachePtrs holds ",
                deviceBlockCachePtrs.numel(), " pointers, hostBlockCache has ", layers, " layers");
}

void check_ptr_table(const at::Tensor& t, const char* what) {
    TORCH_CHECK(t.scalar_type() == at::kLong, what, " must be int64");
    TORCH_CHECK(t.is_contiguous(), what, " must be contiguous");
}

}  // namespace

// dst[i, :] = table[ids[i], :]. Mirrors gather_torch.cpp:30-54. Row size is
// element_size * size(1) for the 2-D tables the reference is used with, and the
// product of all trailing dimensions for higher-rank (e.g. paged KV) tables.
void gather(const at::Tensor& gmEmbed, const at::Tensor& gmEmbedDst, const at::Tensor& gmIds,
            std::optional<int64_t> aiv) {
    check_aiv(aiv);
    TORCH_CHECK(gmEmbed.dim() >= 2, "gmEmbed must have at least 2 dimensions");
    TORCH_CHECK(gmIds.dim() >= 1, "gmIds must be 1-dimensional");
    TORCH_CHECK(gmEmbed.is_contiguous() && gmEmbedDst.is_contiguous() && gmIds.is_contiguous(),
                "gather: tensors must be contiguous");
    TORCH_CHECK(gmEmbedDst.is_cuda(), "gmEmbedDst must be a device tensor");
    TORCH_CHECK(gmIds.scalar_type() == at::kLong || gmIds.scalar_type() == at::kInt, "ScalarType ",
                c10::toString(gmIds.scalar_type()), " not supported.");
    const uint64_t numIds = static_cast<uint64_t>(gmIds.size(0));
    const uint64_t tableRows = static_cast<uint64_t>(gmEmbed.size(0));
    uint64_t rowBytes = static_cast<uint64_t>(gmEmbed.element_size());
    for (int64_t d = 1; d < gmEmbed.dim(); ++d) rowBytes *= static_cast<uint64_t>(gmEmbed.size(d));
    if (numIds == 0) return;
    TORCH_CHECK(rowBytes > 0, "gmEmbed rows are empty");
    TORCH_CHECK(static_cast<uint64_t>(gmEmbedDst.nbytes()) >= numIds * rowBytes, "gmEmbedDst holds ",
                gmEmbedDst.nbytes(), " bytes, ", numIds * rowBytes, " needed");

    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(gmEmbedDst));
    bool table_in_host = false;
    const void* table = device_visible(gmEmbed, "gmEmbed", &table_in_host);
    const void* ids = device_visible(gmIds, "gmIds");
    // workgroups 0: the library sizes the grid for where the table lives (HBM, or host memory
    // behind the PCIe link, the reference's embedding case), which the tensor has just told.
    check_status(hfk_gather_rows(table, gmEmbedDst.data_ptr(), ids, gmIds.scalar_type() == at::kLong, numIds,
                                 rowBytes, tableRows, table_in_host ? HFK_SWAP_SRC_HOST : HFK_SWAP_SRC_DEVICE, 0,
                                 current_stream()),
                 "hfk_gather_rows");
}

// One [T,L,H,D] host block -> L device buffers [H,T,D].
// Mirrors multi_layer_block_transfer_torch.cpp:58-80.
void multi_layer_block_transfer(const at::Tensor& deviceBlockCachePtrs, const at::Tensor& hostBlockCache,
                                std::optional<int64_t> aiv) {
    check_aiv(aiv);
    const BlockGeometry g = block_geometry(hostBlockCache);
    check_layer_ptrs(deviceBlockCachePtrs, g.L);
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(deviceBlockCachePtrs));
    bool src_in_host = false;
    const void* src = device_visible(hostBlockCache, "hostBlockCache", &src_in_host);
    check_status(hfk_multi_layer_block_transfer(deviceBlockCachePtrs.data_ptr(), src, g.T, g.L, g.H, g.D, g.elem,
                                                src_in_host ? HFK_SWAP_SRC_HOST : HFK_SWAP_SRC_DEVICE, 0,
                                                current_stream()),
                 "hfk_multi_layer_block_transfer");
}

// Whole-block async copy into stagingBlockCache, then the same conversion from
// HBM. Mirrors multi_layer_block_transfer_torch.cpp:82-106.
void fused_memcpy_multi_layer_block_transfer(const at::Tensor& deviceBlockCachePtrs,
                                             const at::Tensor& hostBlockCache,
                                             const at::Tensor& stagingBlockCache, std::optional<int64_t> aiv) {
    check_aiv(aiv);
    const BlockGeometry g = block_geometry(hostBlockCache);
    check_layer_ptrs(deviceBlockCachePtrs, g.L);
    TORCH_CHECK(stagingBlockCache.is_cuda(), "stagingBlockCache must be a device tensor");
    TORCH_CHECK(stagingBlockCache.is_contiguous(), "stagingBlockCache must be contiguous");
    TORCH_CHECK(stagingBlockCache.nbytes() >= hostBlockCache.nbytes(), "stagingBlockCache holds ",
                stagingBlockCache.nbytes(), " bytes, ", hostBlockCache.nbytes(), " needed");
    TORCH_CHECK(hostBlockCache.device().is_cpu(), "hostBlockCache must be a host tensor");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(deviceBlockCachePtrs));
    check_status(hfk_fused_memcpy_multi_layer_block_transfer(deviceBlockCachePtrs.data_ptr(),
                                                             hostBlockCache.data_ptr(),
                                                             stagingBlockCache.data_ptr(), g.T, g.L, g.H, g.D,
                                                             g.elem, 0, current_stream()),
                 "hfk_fused_memcpy_multi_layer_block_transfer");
}

// The transfer op over a block table, either direction, one launch; see
// hfk_multi_layer_block_table_transfer. hostBlockPool is [blocks, T, L, H, D];
// deviceLayerCachePtrs[l] points at block 0 of layer l's cache [deviceBlocks][H, T, D].
void multi_layer_block_table_transfer(const at::Tensor& deviceLayerCachePtrs, const at::Tensor& hostBlockPool,
                                      const at::Tensor& blockPairs, int64_t deviceBlockStride, int64_t deviceBlocks,
                                      bool toHost, std::optional<int64_t> workgroups, int64_t flags) {
    TORCH_CHECK(hostBlockPool.dim() == 5,
                "hostBlockPool must be [blocks, blockSize, layers, heads, headDims], got ", hostBlockPool.dim(),
                " dims");
    TORCH_CHECK(hostBlockPool.is_contiguous(), "hostBlockPool must be contiguous");
    for (int i = 1; i < 5; ++i) {
        TORCH_CHECK(hostBlockPool.size(i) <= 0xffffffffLL, "hostBlockPool dimension ", i, " too large");
    }
    const uint32_t T = static_cast<uint32_t>(hostBlockPool.size(1)), L = static_cast<uint32_t>(hostBlockPool.size(2));
    const uint32_t H = static_cast<uint32_t>(hostBlockPool.size(3)), D = static_cast<uint32_t>(hostBlockPool.size(4));
    const uint32_t elem = static_cast<uint32_t>(hostBlockPool.element_size());
    check_layer_ptrs(deviceLayerCachePtrs, L);
    check_ptr_table(blockPairs, "blockPairs");
    TORCH_CHECK(blockPairs.dim() == 2 && blockPairs.size(1) == 2, "blockPairs must be [n, 2]");
    const uint64_t blockBytes = static_cast<uint64_t>(T) * L * H * D * elem;
    TORCH_CHECK(deviceBlockStride >= 0 && static_cast<uint64_t>(deviceBlockStride) >= blockBytes / (L ? L : 1),
                "deviceBlockStride is smaller than one [heads, blockSize, headDims] block");
    TORCH_CHECK(deviceBlocks >= 0, "deviceBlocks must be non-negative");
    if (blockPairs.size(0) == 0 || blockBytes == 0) return;
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(deviceLayerCachePtrs));
    const uint32_t cap = workgroup_cap(workgroups);   // 0: the library sizes the grid for where the pool lives
    bool pool_in_host = false;
    void* pool = device_visible(hostBlockPool, "hostBlockPool", &pool_in_host);
    uint32_t bits = flag_bits(flags, "multi_layer_block_table_transfer");
    constexpr uint32_t kSideBits = HFK_SWAP_SRC_HOST | HFK_SWAP_DST_HOST | HFK_SWAP_SRC_DEVICE | HFK_SWAP_DST_DEVICE;
    if ((bits & kSideBits) == 0) {   // the tensor knows where the pool lives: spare the library the question
        bits |= toHost ? (pool_in_host ? HFK_SWAP_DST_HOST : HFK_SWAP_DST_DEVICE)
                       : (pool_in_host ? HFK_SWAP_SRC_HOST : HFK_SWAP_SRC_DEVICE);
    }
    check_status(hfk_multi_layer_block_table_transfer(
                     deviceLayerCachePtrs.data_ptr(), static_cast<uint64_t>(deviceBlockStride), pool, blockBytes,
                     static_cast<const int64_t*>(device_visible(blockPairs, "blockPairs")),
                     static_cast<uint64_t>(blockPairs.size(0)), static_cast<uint64_t>(hostBlockPool.size(0)),
                     static_cast<uint64_t>(deviceBlocks), T, L, H, D, elem, toHost ? 1 : 0, bits, cap,
                     current_stream()),
                 "hfk_multi_layer_block_table_transfer");
}

// Block-table swap, every plane in one launch; see hfk_swap_blocks. The plane
// tables hold raw addresses (device pointers, or heterofusedkernels.memory
// .get_device_ptr() of pinned host planes), built once by the caller exactly like
// the per-layer pointer tensor of the reference's transfer op
// (pcieThrough/tests/test_transfer_kernel.py:42-47).
void swap_blocks(const at::Tensor& dstPlanePtrs, const at::Tensor& srcPlanePtrs, const at::Tensor& blockPairs,
                 int64_t blockBytes, int64_t srcBlockStride, int64_t dstBlockStride, int64_t srcBlocks,
                 int64_t dstBlocks, std::optional<int64_t> workgroups, int64_t flags) {
    check_ptr_table(dstPlanePtrs, "dstPlanePtrs");
    check_ptr_table(srcPlanePtrs, "srcPlanePtrs");
    check_ptr_table(blockPairs, "blockPairs");
    TORCH_CHECK(flags >= 0 && flags <= 0xffffffffLL, "swap_blocks: flags out of range");
    TORCH_CHECK(dstPlanePtrs.is_cuda(), "dstPlanePtrs must be a device tensor");
    TORCH_CHECK(dstPlanePtrs.numel() == srcPlanePtrs.numel(), "plane tables differ in length");
    TORCH_CHECK(blockPairs.dim() == 2 && blockPairs.size(1) == 2, "blockPairs must be [n, 2]");
    TORCH_CHECK(blockBytes > 0 && srcBlockStride >= blockBytes && dstBlockStride >= blockBytes,
                "swap_blocks: strides must be at least blockBytes, blockBytes positive");
    TORCH_CHECK(srcBlocks >= 0 && dstBlocks >= 0, "swap_blocks: block counts must be non-negative");
    TORCH_CHECK(dstPlanePtrs.numel() <= 0xffffffffLL, "too many planes");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(dstPlanePtrs));
    check_status(
        hfk_swap_blocks(dstPlanePtrs.data_ptr(), device_visible(srcPlanePtrs, "srcPlanePtrs"),
                        static_cast<const int64_t*>(device_visible(blockPairs, "blockPairs")),
                        static_cast<uint32_t>(dstPlanePtrs.numel()), static_cast<uint64_t>(blockPairs.size(0)),
                        static_cast<uint64_t>(blockBytes), static_cast<uint64_t>(srcBlockStride),
                        static_cast<uint64_t>(dstBlockStride), static_cast<uint64_t>(srcBlocks),
                        static_cast<uint64_t>(dstBlocks), static_cast<uint32_t>(flags), workgroup_cap(workgroups),
                        current_stream()),
        "hfk_swap_blocks");
}

// Swap-out (device -> host) and swap-in (host -> device) of the same cache in one
// launch that keeps both directions of the link busy; see hfk_swap_blocks_duplex.
// outBlockPairs rows are (device_block, host_block), inBlockPairs rows are
// (host_block, device_block). The two tables must not name the same block on the
// same side. Either table may be empty.
void swap_blocks_duplex(const at::Tensor& devicePlanePtrs, const at::Tensor& hostPlanePtrs,
                        const at::Tensor& outBlockPairs, const at::Tensor& inBlockPairs, int64_t blockBytes,
                        int64_t deviceBlockStride, int64_t hostBlockStride, int64_t deviceBlocks, int64_t hostBlocks,
                        std::optional<int64_t> workgroups, int64_t flags) {
    check_ptr_table(devicePlanePtrs, "devicePlanePtrs");
    check_ptr_table(hostPlanePtrs, "hostPlanePtrs");
    check_ptr_table(outBlockPairs, "outBlockPairs");
    check_ptr_table(inBlockPairs, "inBlockPairs");
    TORCH_CHECK(devicePlanePtrs.is_cuda(), "devicePlanePtrs must be a device tensor");
    TORCH_CHECK(devicePlanePtrs.numel() == hostPlanePtrs.numel(), "plane tables differ in length");
    TORCH_CHECK(devicePlanePtrs.numel() <= 0xffffffffLL, "too many planes");
    TORCH_CHECK(outBlockPairs.dim() == 2 && outBlockPairs.size(1) == 2, "outBlockPairs must be [n, 2]");
    TORCH_CHECK(inBlockPairs.dim() == 2 && inBlockPairs.size(1) == 2, "inBlockPairs must be [n, 2]");
    TORCH_CHECK(blockBytes > 0 && deviceBlockStride >= blockBytes && hostBlockStride >= blockBytes,
                "swap_blocks_duplex: strides must be at least blockBytes, blockBytes positive");
    TORCH_CHECK(deviceBlocks >= 0 && hostBlocks >= 0, "swap_blocks_duplex: block counts must be non-negative");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(devicePlanePtrs));
    const void* dev_tab = devicePlanePtrs.data_ptr();
    const void* host_tab = device_visible(hostPlanePtrs, "hostPlanePtrs");
    hfk_block_move out_move{};
    out_move.dst_plane_ptrs = host_tab;
    out_move.src_plane_ptrs = dev_tab;
    out_move.n_pairs = static_cast<uint64_t>(outBlockPairs.size(0));
    out_move.block_pairs = out_move.n_pairs ? static_cast<const int64_t*>(device_visible(outBlockPairs, "outBlockPairs"))
                                            : nullptr;
    out_move.src_block_stride = static_cast<uint64_t>(deviceBlockStride);
    out_move.dst_block_stride = static_cast<uint64_t>(hostBlockStride);
    out_move.src_blocks = static_cast<uint64_t>(deviceBlocks);
    out_move.dst_blocks = static_cast<uint64_t>(hostBlocks);
    hfk_block_move in_move{};
    in_move.dst_plane_ptrs = dev_tab;
    in_move.src_plane_ptrs = host_tab;
    in_move.n_pairs = static_cast<uint64_t>(inBlockPairs.size(0));
    in_move.block_pairs = in_move.n_pairs ? static_cast<const int64_t*>(device_visible(inBlockPairs, "inBlockPairs"))
                                          : nullptr;
    in_move.src_block_stride = static_cast<uint64_t>(hostBlockStride);
    in_move.dst_block_stride = static_cast<uint64_t>(deviceBlockStride);
    in_move.src_blocks = static_cast<uint64_t>(hostBlocks);
    in_move.dst_blocks = static_cast<uint64_t>(deviceBlocks);
    check_status(hfk_swap_blocks_duplex(&out_move, &in_move, static_cast<uint32_t>(devicePlanePtrs.numel()),
                                        static_cast<uint64_t>(blockBytes), flag_bits(flags, "swap_blocks_duplex"),
                                        workgroup_cap(workgroups), current_stream()),
                 "hfk_swap_blocks_duplex");
}

// Staged block-table swap: one gather/scatter kernel on HBM plus DMA copies, so no
// compute unit touches host memory; see hfk_swap_blocks_staged. hostPlaneAddrs and
// hostBlockIds are CPU int64 tensors (host addresses of the pinned planes, host slots);
// deviceBlockIds lives on the device. Block-table form of the reference's staged
// variant (multi_layer_block_transfer_torch.cpp:82-106).
void swap_blocks_staged(const at::Tensor& devicePlanePtrs, const at::Tensor& hostPlaneAddrs,
                        const at::Tensor& deviceBlockIds, const at::Tensor& hostBlockIds, const at::Tensor& staging,
                        int64_t blockBytes, int64_t deviceBlockStride, int64_t hostBlockStride, bool toHost,
                        int64_t deviceBlocks, int64_t hostBlocks, std::optional<int64_t> workgroups) {
    check_ptr_table(devicePlanePtrs, "devicePlanePtrs");
    check_ptr_table(hostPlaneAddrs, "hostPlaneAddrs");
    check_ptr_table(deviceBlockIds, "deviceBlockIds");
    check_ptr_table(hostBlockIds, "hostBlockIds");
    TORCH_CHECK(devicePlanePtrs.is_cuda(), "devicePlanePtrs must be a device tensor");
    TORCH_CHECK(hostPlaneAddrs.device().is_cpu() && hostBlockIds.device().is_cpu(),
                "hostPlaneAddrs and hostBlockIds must be CPU tensors");
    TORCH_CHECK(staging.is_cuda() && staging.is_contiguous(), "staging must be a contiguous device tensor");
    TORCH_CHECK(devicePlanePtrs.numel() == hostPlaneAddrs.numel(), "plane tables differ in length");
    TORCH_CHECK(devicePlanePtrs.numel() <= 0xffffffffLL, "too many planes");
    TORCH_CHECK(deviceBlockIds.dim() == 1 && hostBlockIds.dim() == 1 && deviceBlockIds.numel() == hostBlockIds.numel(),
                "deviceBlockIds and hostBlockIds must be 1-dimensional and equally long");
    TORCH_CHECK(blockBytes > 0 && deviceBlockStride >= blockBytes && hostBlockStride >= blockBytes,
                "swap_blocks_staged: strides must be at least blockBytes, blockBytes positive");
    TORCH_CHECK(deviceBlocks >= 0 && hostBlocks >= 0, "swap_blocks_staged: block counts must be non-negative");
    const uint64_t planes = static_cast<uint64_t>(devicePlanePtrs.numel());
    const uint64_t n = static_cast<uint64_t>(deviceBlockIds.numel());
    TORCH_CHECK(static_cast<uint64_t>(staging.nbytes()) >= planes * n * static_cast<uint64_t>(blockBytes),
                "staging holds ", staging.nbytes(), " bytes, ", planes * n * static_cast<uint64_t>(blockBytes),
                " needed");
    if (planes == 0 || n == 0) return;
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(devicePlanePtrs));
    check_status(hfk_swap_blocks_staged(devicePlanePtrs.data_ptr(),
                                        reinterpret_cast<void* const*>(hostPlaneAddrs.data_ptr<int64_t>()),
                                        static_cast<const int64_t*>(device_visible(deviceBlockIds, "deviceBlockIds")),
                                        hostBlockIds.data_ptr<int64_t>(), static_cast<uint32_t>(planes), n,
                                        static_cast<uint64_t>(blockBytes), static_cast<uint64_t>(deviceBlockStride),
                                        static_cast<uint64_t>(hostBlockStride), static_cast<uint64_t>(deviceBlocks),
                                        static_cast<uint64_t>(hostBlocks), staging.data_ptr(), toHost ? 1 : 0,
                                        workgroup_cap(workgroups), current_stream()),
                 "hfk_swap_blocks_staged");
}

// The staged swap through the library's own staging array: no staging tensor, no allocation
// (at most HFK_STATIC_STAGING_BYTES per call); see hfk_swap_blocks_staged_static.
void swap_blocks_staged_static(const at::Tensor& devicePlanePtrs, const at::Tensor& hostPlaneAddrs,
                               const at::Tensor& deviceBlockIds, const at::Tensor& hostBlockIds, int64_t blockBytes,
                               int64_t deviceBlockStride, int64_t hostBlockStride, bool toHost, int64_t deviceBlocks,
                               int64_t hostBlocks, std::optional<int64_t> workgroups) {
    check_ptr_table(devicePlanePtrs, "devicePlanePtrs");
    check_ptr_table(hostPlaneAddrs, "hostPlaneAddrs");
    check_ptr_table(deviceBlockIds, "deviceBlockIds");
    check_ptr_table(hostBlockIds, "hostBlockIds");
    TORCH_CHECK(devicePlanePtrs.is_cuda(), "devicePlanePtrs must be a device tensor");
    TORCH_CHECK(hostPlaneAddrs.device().is_cpu() && hostBlockIds.device().is_cpu(),
                "hostPlaneAddrs and hostBlockIds must be CPU tensors");
    TORCH_CHECK(devicePlanePtrs.numel() == hostPlaneAddrs.numel(), "plane tables differ in length");
    TORCH_CHECK(devicePlanePtrs.numel() <= 0xffffffffLL, "too many planes");
    TORCH_CHECK(deviceBlockIds.dim() == 1 && hostBlockIds.dim() == 1 && deviceBlockIds.numel() == hostBlockIds.numel(),
                "deviceBlockIds and hostBlockIds must be 1-dimensional and equally long");
    TORCH_CHECK(blockBytes > 0 && deviceBlockStride >= blockBytes && hostBlockStride >= blockBytes,
                "swap_blocks_staged_static: strides must be at least blockBytes, blockBytes positive");
    TORCH_CHECK(deviceBlocks >= 0 && hostBlocks >= 0, "swap_blocks_staged_static: block counts must be non-negative");
    const uint64_t planes = static_cast<uint64_t>(devicePlanePtrs.numel());
    const uint64_t n = static_cast<uint64_t>(deviceBlockIds.numel());
    if (planes == 0 || n == 0) return;
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(devicePlanePtrs));
    check_status(hfk_swap_blocks_staged_static(
                     devicePlanePtrs.data_ptr(), reinterpret_cast<void* const*>(hostPlaneAddrs.data_ptr<int64_t>()),
                     static_cast<const int64_t*>(device_visible(deviceBlockIds, "deviceBlockIds")),
                     hostBlockIds.data_ptr<int64_t>(), static_cast<uint32_t>(planes), n,
                     static_cast<uint64_t>(blockBytes), static_cast<uint64_t>(deviceBlockStride),
                     static_cast<uint64_t>(hostBlockStride), static_cast<uint64_t>(deviceBlocks),
                     static_cast<uint64_t>(hostBlocks), toHost ? 1 : 0, workgroup_cap(workgroups), current_stream()),
                 "hfk_swap_blocks_staged_static");
}

// Block-table swap that picks, per run of consecutive host slots, between the staged mover
// (HBM kernel + DMA copies) and the direct one; see hfk_swap_blocks_auto. blockPairs rows are
// (device_block, host_block) when toHost, (host_block, device_block) otherwise. hostPlaneAddrs
// (CPU int64: host addresses of the planes), hostBlockIds (CPU int64: the host column of
// blockPairs) and staging are optional; without them the whole table moves the direct way.
void swap_blocks_auto(const at::Tensor& devicePlanePtrs, const at::Tensor& hostPlanePtrs, const at::Tensor& blockPairs,
                      int64_t blockBytes, int64_t deviceBlockStride, int64_t hostBlockStride, bool toHost,
                      const std::optional<at::Tensor>& hostPlaneAddrs, const std::optional<at::Tensor>& hostBlockIds,
                      const std::optional<at::Tensor>& staging, int64_t deviceBlocks, int64_t hostBlocks,
                      int64_t minRunBlocks, int64_t flags) {
    check_ptr_table(devicePlanePtrs, "devicePlanePtrs");
    check_ptr_table(hostPlanePtrs, "hostPlanePtrs");
    check_ptr_table(blockPairs, "blockPairs");
    TORCH_CHECK(devicePlanePtrs.is_cuda(), "devicePlanePtrs must be a device tensor");
    TORCH_CHECK(devicePlanePtrs.numel() == hostPlanePtrs.numel(), "plane tables differ in length");
    TORCH_CHECK(devicePlanePtrs.numel() <= 0xffffffffLL, "too many planes");
    TORCH_CHECK(blockPairs.dim() == 2 && blockPairs.size(1) == 2, "blockPairs must be [n, 2]");
    TORCH_CHECK(blockBytes > 0 && deviceBlockStride >= blockBytes && hostBlockStride >= blockBytes,
                "swap_blocks_auto: strides must be at least blockBytes, blockBytes positive");
    TORCH_CHECK(deviceBlocks >= 0 && hostBlocks >= 0, "swap_blocks_auto: block counts must be non-negative");
    TORCH_CHECK(minRunBlocks >= 0 && minRunBlocks <= 0xffffffffLL, "swap_blocks_auto: minRunBlocks out of range");
    const uint64_t planes = static_cast<uint64_t>(devicePlanePtrs.numel());
    const uint64_t n = static_cast<uint64_t>(blockPairs.size(0));
    void* const* host_addrs = nullptr;
    const int64_t* host_ids = nullptr;
    void* staging_ptr = nullptr;
    uint64_t staging_bytes = 0;
    if (hostPlaneAddrs.has_value() && hostBlockIds.has_value() && staging.has_value()) {
        check_ptr_table(*hostPlaneAddrs, "hostPlaneAddrs");
        check_ptr_table(*hostBlockIds, "hostBlockIds");
        TORCH_CHECK(hostPlaneAddrs->device().is_cpu() && hostBlockIds->device().is_cpu(),
                    "hostPlaneAddrs and hostBlockIds must be CPU tensors");
        TORCH_CHECK(static_cast<uint64_t>(hostPlaneAddrs->numel()) == planes, "hostPlaneAddrs must hold one address per plane");
        TORCH_CHECK(hostBlockIds->dim() == 1 && static_cast<uint64_t>(hostBlockIds->numel()) == n,
                    "hostBlockIds must hold one slot per row of blockPairs");
        TORCH_CHECK(staging->is_cuda() && staging->is_contiguous(), "staging must be a contiguous device tensor");
        host_addrs = reinterpret_cast<void* const*>(hostPlaneAddrs->data_ptr<int64_t>());
        host_ids = hostBlockIds->data_ptr<int64_t>();
        staging_ptr = staging->data_ptr();
        staging_bytes = static_cast<uint64_t>(staging->nbytes());
    }
    if (planes == 0 || n == 0) return;
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(devicePlanePtrs));
    check_status(hfk_swap_blocks_auto(devicePlanePtrs.data_ptr(), device_visible(hostPlanePtrs, "hostPlanePtrs"),
                                      host_addrs, static_cast<const int64_t*>(device_visible(blockPairs, "blockPairs")),
                                      host_ids, static_cast<uint32_t>(planes), n, static_cast<uint64_t>(blockBytes),
                                      static_cast<uint64_t>(deviceBlockStride), static_cast<uint64_t>(hostBlockStride),
                                      static_cast<uint64_t>(deviceBlocks), static_cast<uint64_t>(hostBlocks),
                                      staging_ptr, staging_bytes, toHost ? 1 : 0, static_cast<uint32_t>(minRunBlocks),
                                      flag_bits(flags, "swap_blocks_auto"), current_stream()),
                 "hfk_swap_blocks_auto");
}

// Shared-id block gather over planes; see hfk_gather_blocks.
void gather_blocks(const at::Tensor& dstPlanePtrs, const at::Tensor& srcPlanePtrs, const at::Tensor& blockIds,
                   int64_t blockBytes, int64_t srcBlockStride, int64_t srcBlocks,
                   std::optional<int64_t> workgroups, int64_t flags) {
    check_ptr_table(dstPlanePtrs, "dstPlanePtrs");
    check_ptr_table(srcPlanePtrs, "srcPlanePtrs");
    check_ptr_table(blockIds, "blockIds");
    TORCH_CHECK(dstPlanePtrs.is_cuda(), "dstPlanePtrs must be a device tensor");
    TORCH_CHECK(dstPlanePtrs.numel() == srcPlanePtrs.numel(), "plane tables differ in length");
    TORCH_CHECK(blockIds.dim() == 1, "blockIds must be 1-dimensional");
    TORCH_CHECK(blockBytes > 0 && srcBlockStride >= blockBytes,
                "gather_blocks: stride must be at least blockBytes, blockBytes positive");
    TORCH_CHECK(srcBlocks >= 0, "gather_blocks: block count must be non-negative");
    TORCH_CHECK(dstPlanePtrs.numel() <= 0xffffffffLL, "too many planes");
    const c10::hip::OptionalHIPGuardMasqueradingAsCUDA device_guard(device_of(dstPlanePtrs));
    check_status(
        hfk_gather_blocks(dstPlanePtrs.data_ptr(), device_visible(srcPlanePtrs, "srcPlanePtrs"),
                          static_cast<const int64_t*>(device_visible(blockIds, "blockIds")),
                          static_cast<uint32_t>(dstPlanePtrs.numel()), static_cast<uint64_t>(blockIds.size(0)),
                          static_cast<uint64_t>(blockBytes), static_cast<uint64_t>(srcBlockStride),
                          static_cast<uint64_t>(srcBlocks), flag_bits(flags, "gather_blocks"),
                          workgroup_cap(workgroups), current_stream()),
        "hfk_gather_blocks");
}

}  // namespace pciethrough

TORCH_LIBRARY(pcie_through, m) {
    m.def("gather(Tensor gmEmbed, Tensor gmEmbedDst, Tensor gmIds, int? aiv=None) -> ()");
    m.def("multi_layer_block_transfer(Tensor deviceBlockCachePtrs, Tensor hostBlockCache, int? aiv=None) -> ()");
    m.def(
        "fused_memcpy_multi_layer_block_transfer(Tensor deviceBlockCachePtrs, Tensor hostBlockCache, Tensor "
        "stagingBlockCache, int? aiv=None) -> ()");
    // Same op with the written tensor annotated as mutated, for tracing / functionalization
    // (the reference notes the missing annotation at multi_layer_block_transfer_torch.cpp:57).
    m.def("gather_into(Tensor gmEmbed, Tensor(a!) gmEmbedDst, Tensor gmIds, int? aiv=None) -> ()");
    m.def(
        "multi_layer_block_table_transfer(Tensor deviceLayerCachePtrs, Tensor hostBlockPool, Tensor blockPairs, int "
        "deviceBlockStride, int deviceBlocks=0, bool toHost=False, int? workgroups=None, int flags=0) -> ()");
    m.def(
        "swap_blocks(Tensor dstPlanePtrs, Tensor srcPlanePtrs, Tensor blockPairs, int blockBytes, int "
        "srcBlockStride, int dstBlockStride, int srcBlocks=0, int dstBlocks=0, int? workgroups=None, int flags=0) -> ()");
    m.def(
        "swap_blocks_duplex(Tensor devicePlanePtrs, Tensor hostPlanePtrs, Tensor outBlockPairs, Tensor inBlockPairs, int "
        "blockBytes, int deviceBlockStride, int hostBlockStride, int deviceBlocks=0, int hostBlocks=0, int? "
        "workgroups=None, int flags=0) -> ()");
    m.def(
        "swap_blocks_staged(Tensor devicePlanePtrs, Tensor hostPlaneAddrs, Tensor deviceBlockIds, Tensor hostBlockIds, "
        "Tensor(a!) staging, int blockBytes, int deviceBlockStride, int hostBlockStride, bool toHost, int "
        "deviceBlocks=0, int hostBlocks=0, int? workgroups=None) -> ()");
    m.def(
        "gather_blocks(Tensor dstPlanePtrs, Tensor srcPlanePtrs, Tensor blockIds, int blockBytes, int "
        "srcBlockStride, int srcBlocks=0, int? workgroups=None, int flags=0) -> ()");
    m.def(
        "swap_blocks_staged_static(Tensor devicePlanePtrs, Tensor hostPlaneAddrs, Tensor deviceBlockIds, Tensor "
        "hostBlockIds, int blockBytes, int deviceBlockStride, int hostBlockStride, bool toHost, int deviceBlocks=0, int "
        "hostBlocks=0, int? workgroups=None) -> ()");
    m.def(
        "swap_blocks_auto(Tensor devicePlanePtrs, Tensor hostPlanePtrs, Tensor blockPairs, int blockBytes, int "
        "deviceBlockStride, int hostBlockStride, bool toHost, Tensor? hostPlaneAddrs=None, Tensor? hostBlockIds=None, "
        "Tensor(a!)? staging=None, int deviceBlocks=0, int hostBlocks=0, int minRunBlocks=0, int flags=0) -> ()");
}

// PyTorch-ROCm files HIP tensors under the CUDA dispatch key. A call whose tensors
// are all on the CPU finds no kernel and raises, which is the intended behaviour:
// there is no CPU implementation of these ops.
TORCH_LIBRARY_IMPL(pcie_through, CUDA, m) {
    m.impl("gather", TORCH_FN(pciethrough::gather));
    m.impl("multi_layer_block_transfer", TORCH_FN(pciethrough::multi_layer_block_transfer));
    m.impl("fused_memcpy_multi_layer_block_transfer", TORCH_FN(pciethrough::fused_memcpy_multi_layer_block_transfer));
    m.impl("gather_into", TORCH_FN(pciethrough::gather));
    m.impl("multi_layer_block_table_transfer", TORCH_FN(pciethrough::multi_layer_block_table_transfer));
    m.impl("swap_blocks", TORCH_FN(pciethrough::swap_blocks));
    m.impl("swap_blocks_duplex", TORCH_FN(pciethrough::swap_blocks_duplex));
    m.impl("swap_blocks_staged", TORCH_FN(pciethrough::swap_blocks_staged));
    m.impl("gather_blocks", TORCH_FN(pciethrough::gather_blocks));
    m.impl("swap_blocks_staged_static", TORCH_FN(pciethrough::swap_blocks_staged_static));
    m.impl("swap_blocks_auto", TORCH_FN(pciethrough::swap_blocks_auto));
}
