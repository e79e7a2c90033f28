"""The reference's own operator test, restated for torch.cuda: same parametrisation,
pointer-table construction, two-stream round robin and permute check as
pcieThrough/tests/test_transfer_kernel.py:15-83 -- but with seeded random blocks
instead of the constant fill (:32), so a wrong permutation cannot pass."""
import numpy as np
import pytest
import torch

import heterofusedkernels_amd  # noqa: F401  (puts the drop-in packages on sys.path)
import pcie_through  # noqa: F401  (registers torch.ops.pcie_through.*)
from oracle import oracle as O

from gpu_helpers import announce

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def memory():
    import heterofusedkernels_amd  # noqa: F401
    import pcie_through  # noqa: F401
    from heterofusedkernels import memory as m

    return m


@pytest.mark.parametrize("block_size", [1024])
@pytest.mark.parametrize("layers", [1, 32, 64])
@pytest.mark.parametrize("heads", [1, 8])               # 8: the README's second geometry (tests/README.md:73,75)
@pytest.mark.parametrize("head_dim", [128])
@pytest.mark.parametrize("num_blocks", [1, 8, 16])       # tests/test_transfer_kernel.py:19
@pytest.mark.parametrize("use_fused_copy", [False, True])
def test_multi_layer_block_kv_transfer(memory, block_size, layers, heads, head_dim, num_blocks, use_fused_copy):
    device = "cuda"
    dtype = torch.int8
    simultaneous_copy = 2
    announce("transfer op T=%d L=%d H=%d D=%d blocks=%d fused=%s" % (block_size, layers, heads, head_dim, num_blocks,
                                                                     use_fused_copy))
    total_host_blocks = num_blocks + 2
    host_shape = (total_host_blocks, block_size, layers, heads, head_dim)
    device_shape = (num_blocks, layers, heads, block_size, head_dim)
    total_host_size = int(np.prod(host_shape))
    pool = memory.alloc_numa_pinned_tensor(total_host_size)
    gen = torch.Generator().manual_seed(layers * 100 + heads * 10 + num_blocks)
    pool.copy_(torch.randint(-128, 128, (total_host_size,), dtype=torch.int8, generator=gen))
    host_blocks_cache = list(pool.view(dtype).view(host_shape).unbind(0))

    device_blocks_cache = torch.full(device_shape, 0x55, dtype=dtype, device=device)
    device_blocks = list(device_blocks_cache.unbind(0))
    device_block_ptrs = []
    for tensor in device_blocks:                              # tests/test_transfer_kernel.py:42-47
        ptrs = torch.empty(layers, dtype=torch.int64, device="cpu")
        for i in range(layers):
            ptrs[i] = tensor[i].data_ptr()
        device_block_ptrs.append(ptrs.to(device))

    streams = [torch.cuda.Stream() for _ in range(simultaneous_copy)]
    staging = [torch.empty([block_size, layers, heads, head_dim], dtype=dtype, device=device)
               for _ in range(simultaneous_copy)] if use_fused_copy else []
    torch.cuda.synchronize()
    for i in range(num_blocks):
        with torch.cuda.stream(streams[i % simultaneous_copy]):
            if use_fused_copy:
                torch.ops.pcie_through.fused_memcpy_multi_layer_block_transfer(
                    device_block_ptrs[i], host_blocks_cache[i], staging[i % simultaneous_copy], 4)
            else:
                torch.ops.pcie_through.multi_layer_block_transfer(device_block_ptrs[i], host_blocks_cache[i], 4)
    for s in streams:
        s.synchronize()

    got = device_blocks_cache.cpu()
    for i in range(num_blocks):
        transposed_block = got[i].permute(2, 0, 1, 3)         # tests/test_transfer_kernel.py:81
        assert torch.equal(host_blocks_cache[i], transposed_block), "block %d" % i
    # one block against the C restatement as well
    want = O.c_multi_layer_block_transfer(host_blocks_cache[0].contiguous().view(torch.uint8).numpy().reshape(-1),
                                          block_size, layers, heads, head_dim, 1, cores=4)
    assert np.array_equal(got[0].view(torch.uint8).numpy().reshape(layers, -1), want)
    if use_fused_copy:                                        # staging ends up equal to the last block it carried
        last = {}
        for i in range(num_blocks):
            last[i % simultaneous_copy] = i
        for slot, i in last.items():
            assert torch.equal(staging[slot].cpu(), host_blocks_cache[i])


@pytest.mark.parametrize("how", ["one_kernel", "copy_engine", "pageable"])
def test_fused_transfer_gives_the_same_bytes_either_way(memory, how):
    """fused_memcpy_multi_layer_block_transfer reads a pinned block once, by the kernel, which fills the staging
    buffer too; with HFK_KNOB_FUSED_COPY_ENGINE, and for a block in pageable memory, it copies into staging first
    and runs the kernel on staging, as the reference does (multi_layer_block_transfer_torch.cpp:82-106). Layers and
    staging hold the same bytes in all three cases, on a geometry with 16-byte units and on one with 4-byte units
    and a staging buffer off the 16-byte grid."""
    from heterofusedkernels_amd import capi
    for (T, L, H, D, e, stage_off) in ((64, 6, 2, 128, 1, 0), (40, 3, 2, 10, 2, 0), (16, 2, 3, 64, 2, 4)):
        announce("fused transfer %s: T=%d L=%d H=%d D=%d elem=%d staging offset %d" % (how, T, L, H, D, e, stage_off))
        nbytes = T * L * H * D * e
        data = torch.randint(-128, 128, (nbytes,), dtype=torch.int8, generator=torch.Generator().manual_seed(T + L + D))
        if how == "pageable":
            host = data.clone().view(T, L, H, D * e)
            assert not host.is_pinned()
        else:
            pool = memory.alloc_numa_pinned_tensor(nbytes)
            pool.copy_(data)
            host = pool.view(torch.int8).view(T, L, H, D * e)
        layers = torch.full((L, H, T, D * e), 0x55, dtype=torch.int8, device="cuda")
        ptrs = torch.tensor([layers[l].data_ptr() for l in range(L)], dtype=torch.int64).cuda()
        backing = torch.full((nbytes + 16,), 0x66, dtype=torch.int8, device="cuda")
        staging = backing[stage_off:stage_off + nbytes].view(T, L, H, D * e)
        with capi.thread_tuning({capi.KNOB_FUSED_COPY_ENGINE: 1 if how == "copy_engine" else 0}):
            torch.ops.pcie_through.fused_memcpy_multi_layer_block_transfer(ptrs, host, staging, 4)
        torch.cuda.synchronize()
        assert torch.equal(staging.cpu(), host), "staging"
        assert bool((backing[:stage_off] == 0x66).all()) and bool((backing[stage_off + nbytes:] == 0x66).all())
        want = O.c_multi_layer_block_transfer(data.view(torch.uint8).numpy(), T, L, H, D, e, cores=3)
        assert np.array_equal(layers.cpu().view(torch.uint8).numpy().reshape(L, -1), want), "layers"


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16, torch.int8, torch.uint8,
                                   torch.float8_e4m3fn])
def test_transfer_dtypes(memory, dtype):
    """Accepted dtypes are a superset of multi_layer_block_transfer_torch.cpp:41-54."""
    T, L, H, D = 48, 5, 3, 64
    announce("transfer dtype %s" % dtype)
    e = torch.empty((), dtype=dtype).element_size()
    nbytes = T * L * H * D * e
    pool = memory.alloc_numa_pinned_tensor(nbytes)
    pool.copy_(torch.randint(-128, 128, (nbytes,), dtype=torch.int8, generator=torch.Generator().manual_seed(e)))
    host = pool.view(dtype).view(T, L, H, D)
    layers = torch.zeros(L, H, T, D * e, dtype=torch.uint8, device="cuda")
    ptrs = torch.tensor([layers[l].data_ptr() for l in range(L)], dtype=torch.int64).cuda()
    torch.ops.pcie_through.multi_layer_block_transfer(ptrs, host)
    torch.cuda.synchronize()
    want = O.c_multi_layer_block_transfer(pool.view(torch.uint8).numpy(), T, L, H, D, e)
    assert np.array_equal(layers.cpu().numpy().reshape(L, -1), want)


def test_op_argument_errors(memory):
    announce("transfer/gather op argument errors")
    ptrs = torch.zeros(4, dtype=torch.int64, device="cuda")
    host = memory.alloc_numa_pinned_tensor(4 * 4 * 2 * 16).view(4, 4, 2, 16)
    with pytest.raises(RuntimeError, match="Number of AIV blocks should be positive"):
        torch.ops.pcie_through.multi_layer_block_transfer(ptrs, host, 0)       # ...torch.cpp:63
    with pytest.raises(RuntimeError, match="Number of AIV blocks should be positive"):
        torch.ops.pcie_through.gather(host.view(4, -1), torch.zeros(1, 128, dtype=torch.int8, device="cuda"),
                                      torch.zeros(1, dtype=torch.int64, device="cuda"), aiv=0)   # gather_torch.cpp:35
    with pytest.raises(RuntimeError, match="neither registered"):
        torch.ops.pcie_through.multi_layer_block_transfer(ptrs, torch.zeros(4, 4, 2, 16, dtype=torch.int8))
    with pytest.raises(RuntimeError, match="holds 4 pointers"):
        torch.ops.pcie_through.multi_layer_block_transfer(ptrs, memory.alloc_numa_pinned_tensor(4 * 5 * 2 * 16)
                                                          .view(4, 5, 2, 16))
    with pytest.raises(RuntimeError, match="not supported"):
        torch.ops.pcie_through.gather(host.view(4, -1), torch.zeros(1, 128, dtype=torch.int8, device="cuda"),
                                      torch.zeros(1, dtype=torch.float32, device="cuda"))


def test_memory_module_on_gpu(memory):
    announce("heterofusedkernels.memory on the GPU box")
    t = memory.alloc_numa_pinned_tensor(1 << 20)
    assert t.dtype == torch.int8 and t.shape == (1 << 20,) and t.is_pinned() and int(t.abs().max()) == 0
    base = memory.get_device_ptr(t.data_ptr())
    assert base != 0 and memory.get_device_ptr(t.data_ptr() + 12345) == base + 12345      # interior pointer
    assert memory.host_register(t) == base                                               # idempotent
    n0 = memory.record_count()
    del t
    assert memory.record_count() == n0 - 1                                               # deleter unregisters
    tp = torch.empty(4096, dtype=torch.float16).pin_memory()                             # pinned by torch itself
    dp = memory.host_register(tp)
    assert dp != 0 and memory.get_device_ptr(tp.data_ptr()) == dp
    memory.host_unregister(tp)
    assert memory.get_device_ptr(tp.data_ptr()) == 0
    with pytest.raises(RuntimeError, match="must be pinned"):
        memory.host_register(torch.zeros(8))
    with pytest.raises(RuntimeError, match="must be pinned"):
        memory.host_register(torch.zeros(8, device="cuda"))


def test_pinned_allocation_bound_to_an_explicit_numa_node():
    """hfk_mm_alloc_pinned with a node number takes the MPOL_BIND + hipHostMallocNumaUser route (the boxes
    report node -1 for the GPU, so alloc_numa_pinned_tensor alone never takes it)."""
    import ctypes

    from heterofusedkernels_amd import _build

    announce("pinned allocation bound to NUMA node 0, then used by a kernel")
    mm = ctypes.CDLL(_build.MANAGED_MEMORY_SO)
    mm.hfk_mm_alloc_pinned.argtypes = [ctypes.c_size_t, ctypes.c_int, ctypes.c_uint, ctypes.POINTER(ctypes.c_void_p)]
    mm.hfk_mm_free_pinned.argtypes = [ctypes.c_void_p]
    mm.hfk_mm_get_device_ptr.argtypes = [ctypes.c_void_p]
    mm.hfk_mm_get_device_ptr.restype = ctypes.c_void_p
    mm.hfk_mm_record_size.argtypes = [ctypes.c_void_p]
    mm.hfk_mm_record_size.restype = ctypes.c_size_t
    torch.cuda.init()
    nbytes = 8 << 20
    ptr = ctypes.c_void_p()
    assert mm.hfk_mm_alloc_pinned(nbytes, 0, 0, ctypes.byref(ptr)) == 0 and ptr.value
    dev_ptr = mm.hfk_mm_get_device_ptr(ptr.value)
    assert dev_ptr and mm.hfk_mm_record_size(ptr.value + 100) == nbytes
    host = (ctypes.c_uint8 * nbytes).from_address(ptr.value)
    assert not any(host[i] for i in range(0, nbytes, 4099))                 # zero-filled
    # a kernel writes it through the mapped address: gather 8 rows of 1 MiB from a device table into it
    from heterofusedkernels_amd import capi
    table = torch.randint(0, 256, (16, 1 << 20), dtype=torch.uint8, device="cuda")
    ids = torch.tensor([3, 1, 4, 1, 5, 9, 2, 6], dtype=torch.int64, device="cuda")
    capi.check(capi.gather_rows(table.data_ptr(), dev_ptr, ids.data_ptr(), True, 8, 1 << 20, 16, 0,
                                torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    got = torch.frombuffer(host, dtype=torch.uint8).view(8, 1 << 20)
    assert torch.equal(got, table.cpu()[ids.cpu()])
    del got
    assert mm.hfk_mm_free_pinned(ptr.value) == 0
    assert mm.hfk_mm_get_device_ptr(ptr.value) is None
