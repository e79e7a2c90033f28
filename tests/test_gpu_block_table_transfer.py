"""Block-table form of the layout-converting transfer (both directions) on the GPU:
golden vectors, the C oracle, equivalence with the reference's per-block loop, and the
host -> device -> host round trip."""
import glob
import os

import numpy as np
import pytest
import torch

import heterofusedkernels_amd  # noqa: F401
import pcie_through  # noqa: F401
from heterofusedkernels import memory
from heterofusedkernels_amd import capi
from oracle import oracle as O

from gpu_helpers import announce, stream_handle

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DEV = "cuda"


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(GOLDEN, "tabletransfer_*.npz"))))
def test_golden_table_transfer(path):
    announce("golden " + os.path.basename(path))
    g = np.load(path)
    T, L, H, D, e, to_packed = (int(x) for x in g["geometry"])
    packed = torch.from_numpy(g["packed"].copy()).to(DEV)
    layers = torch.from_numpy(g["layers"].copy()).to(DEV)
    pairs = torch.from_numpy(g["pairs"]).to(DEV)
    ptrs = torch.tensor([layers[l].data_ptr() for l in range(L)], dtype=torch.int64).to(DEV)
    capi.check(capi.multi_layer_block_table_transfer(ptrs.data_ptr(), layers.shape[2], packed.data_ptr(),
                                                     packed.shape[1], pairs.data_ptr(), pairs.shape[0], packed.shape[0],
                                                     layers.shape[1], T, L, H, D, e, to_packed, 0, stream_handle()))
    torch.cuda.synchronize()
    assert np.array_equal(packed.cpu().numpy(), g["packed_expected"])
    assert np.array_equal(layers.cpu().numpy(), g["layers_expected"])


@pytest.mark.parametrize("T,L,H,D,dtype", [(256, 8, 2, 128, torch.int8), (64, 5, 8, 128, torch.bfloat16),
                                           (1024, 32, 1, 128, torch.int8), (16, 3, 2, 24, torch.float16)])
def test_block_table_transfer_host_to_device_and_back(T, L, H, D, dtype):
    e = torch.empty((), dtype=dtype).element_size()
    host_blocks, dev_blocks, n = 12, 9, 7
    announce("block-table transfer T=%d L=%d H=%d D=%d %s, %d pairs" % (T, L, H, D, dtype, n))
    block_bytes = T * L * H * D * e
    pool = memory.alloc_numa_pinned_tensor(host_blocks * block_bytes)
    gen = torch.Generator().manual_seed(T + L)
    pool.copy_(torch.randint(-128, 128, (host_blocks * block_bytes,), dtype=torch.int8, generator=gen))
    host_pool = pool.view(dtype).view(host_blocks, T, L, H, D)
    caches = torch.zeros(L, dev_blocks, H, T, D, dtype=dtype, device=DEV)            # per-layer [blocks, H, T, D]
    ptrs = torch.tensor([caches[l].data_ptr() for l in range(L)], dtype=torch.int64).to(DEV)
    hb = torch.randperm(host_blocks, generator=gen)[:n]
    db = torch.randperm(dev_blocks, generator=gen)[:n]
    pairs = torch.stack([hb, db], 1).contiguous()
    stride = H * T * D * e
    torch.ops.pcie_through.multi_layer_block_table_transfer(ptrs, host_pool, pairs.to(DEV), stride, dev_blocks)
    torch.cuda.synchronize()
    got = caches.cpu()
    # oracle
    want = np.zeros((L, dev_blocks, stride), dtype=np.uint8)
    O.c_multi_layer_block_table_transfer(want, pool.view(torch.uint8).numpy().reshape(host_blocks, block_bytes),
                                         pairs.numpy(), T, L, H, D, e, False)
    assert np.array_equal(got.view(torch.uint8).numpy().reshape(L, dev_blocks, stride), want)
    # the reference's permute check per block (tests/test_transfer_kernel.py:77-83) ...
    for j in range(n):
        transposed = got[:, db[j]].permute(2, 0, 1, 3).contiguous()      # bytes: random payloads hold NaNs
        assert torch.equal(transposed.view(torch.uint8), host_pool[hb[j]].view(torch.uint8))
    # ... and equality with its per-block op loop (:58-72)
    loop = torch.zeros_like(caches)
    for j in range(n):
        bptrs = torch.tensor([loop[l, db[j]].data_ptr() for l in range(L)], dtype=torch.int64).to(DEV)
        torch.ops.pcie_through.multi_layer_block_transfer(bptrs, host_pool[hb[j]], 4)
    torch.cuda.synchronize()
    assert torch.equal(loop.cpu().view(torch.uint8), got.view(torch.uint8))
    # back to other host slots: device -> host, then byte-compare with the original blocks
    pool2 = memory.alloc_numa_pinned_tensor(host_blocks * block_bytes)
    host_pool2 = pool2.view(dtype).view(host_blocks, T, L, H, D)
    hb2 = torch.randperm(host_blocks, generator=gen)[:n]
    torch.ops.pcie_through.multi_layer_block_table_transfer(ptrs, host_pool2, torch.stack([hb2, db], 1).contiguous().to(DEV),
                                                            stride, dev_blocks, True)
    torch.cuda.synchronize()
    for j in range(n):
        assert torch.equal(host_pool2[hb2[j]].view(torch.uint8), host_pool[hb[j]].view(torch.uint8))
    untouched = torch.ones(host_blocks, dtype=torch.bool)
    untouched[hb2] = False
    assert int(pool2.view(host_blocks, block_bytes)[untouched].abs().max()) == 0


def test_block_table_transfer_skips_out_of_range_pairs():
    announce("block-table transfer: out-of-range pairs are skipped")
    T, L, H, D = 8, 2, 2, 64
    pool = memory.alloc_numa_pinned_tensor(4 * T * L * H * D)
    pool.fill_(3)
    caches = torch.zeros(L, 4, H, T, D, dtype=torch.int8, device=DEV)
    ptrs = torch.tensor([caches[l].data_ptr() for l in range(L)], dtype=torch.int64).to(DEV)
    pairs = torch.tensor([[0, 1], [4, 2], [1, -1], [2, 4], [3, 3]], dtype=torch.int64).to(DEV)
    torch.ops.pcie_through.multi_layer_block_table_transfer(ptrs, pool.view(4, T, L, H, D), pairs, H * T * D, 4)
    torch.cuda.synchronize()
    got = caches.cpu()
    assert (got[:, 1] == 3).all() and (got[:, 3] == 3).all() and (got[:, 0] == 0).all() and (got[:, 2] == 0).all()


def test_block_table_transfer_staged_through_a_device_pool():
    """The reference's staged idea (DMA copy into device staging, then a kernel that reads only HBM,
    multi_layer_block_transfer_torch.cpp:82-106) over a block table, composed from existing pieces: one
    hipMemcpyAsync per run of consecutive host blocks into a device pool, then the block-table transfer
    with the pool as its packed side. Same result as the direct host-memory transfer."""
    T, L, H, D, dtype = 128, 6, 4, 128, torch.bfloat16
    e, host_blocks, dev_blocks = 2, 20, 11
    announce("block-table transfer staged through a device pool, T=%d L=%d H=%d D=%d" % (T, L, H, D))
    gen = torch.Generator().manual_seed(77)
    pool = memory.alloc_numa_pinned_tensor(host_blocks * T * L * H * D * e)
    pool.copy_(torch.randint(-128, 128, (pool.numel(),), dtype=torch.int8, generator=gen))
    host_pool = pool.view(dtype).view(host_blocks, T, L, H, D)
    runs = [(3, 4), (12, 5)]                                            # (first host block, count)
    host_ids = torch.cat([torch.arange(a, a + c) for a, c in runs])
    dev_ids = torch.randperm(dev_blocks, generator=gen)[:host_ids.numel()]
    stride = H * T * D * e

    def fresh():
        caches = torch.zeros(L, dev_blocks, H, T, D, dtype=dtype, device=DEV)
        return caches, torch.tensor([caches[l].data_ptr() for l in range(L)], dtype=torch.int64).to(DEV)

    direct, dptrs = fresh()
    torch.ops.pcie_through.multi_layer_block_table_transfer(dptrs, host_pool, torch.stack([host_ids, dev_ids], 1).to(DEV),
                                                            stride, dev_blocks)
    staged, sptrs = fresh()
    staging = torch.empty(host_ids.numel(), T, L, H, D, dtype=dtype, device=DEV)
    at = 0
    for first, count in runs:
        staging[at:at + count].copy_(host_pool[first:first + count], non_blocking=True)      # one DMA copy per run
        at += count
    torch.ops.pcie_through.multi_layer_block_table_transfer(
        sptrs, staging, torch.stack([torch.arange(host_ids.numel()), dev_ids], 1).to(DEV), stride, dev_blocks)
    torch.cuda.synchronize()
    assert torch.equal(staged.view(torch.uint8), direct.view(torch.uint8))
    want = torch.stack(O.torch_multi_layer_block_transfer(host_pool[host_ids[0]]))     # [L, H, T, D] of the first moved block
    assert torch.equal(staged[:, dev_ids[0]].cpu().contiguous().view(torch.uint8), want.view(torch.uint8))


@pytest.mark.parametrize("T,L,H,D,dtype", [(16, 32, 8, 128, torch.bfloat16), (64, 5, 2, 80, torch.float16)])
def test_block_table_transfer_with_token_major_layer_caches(T, L, H, D, dtype):
    """Layer caches laid out [blocks, T, H, D] (tokens first, the common paged-attention layout) instead of
    the reference's [H, T, D] per block (multi_layer_block_transfer_kernel.h:60-67): a token's H x D values are
    then contiguous on both sides, which is the same transfer with one head of H * D values. Both directions,
    against torch indexing and the C oracle."""
    e = torch.empty((), dtype=dtype).element_size()
    host_blocks, dev_blocks, n = 10, 13, 6
    announce("block-table transfer, token-major layer caches, T=%d L=%d H=%d D=%d %s" % (T, L, H, D, dtype))
    block_bytes = T * L * H * D * e
    gen = torch.Generator().manual_seed(L * 100 + H)
    pool = memory.alloc_numa_pinned_tensor(host_blocks * block_bytes)
    pool.copy_(torch.randint(-128, 128, (pool.numel(),), dtype=torch.int8, generator=gen))
    host_pool = pool.view(dtype).view(host_blocks, T, L, H, D)
    caches = torch.zeros(L, dev_blocks, T, H, D, dtype=dtype, device=DEV)
    ptrs = torch.tensor([caches[l].data_ptr() for l in range(L)], dtype=torch.int64).to(DEV)
    hb = torch.randperm(host_blocks, generator=gen)[:n]
    db = torch.randperm(dev_blocks, generator=gen)[:n]
    pairs = torch.stack([hb, db], 1).contiguous()
    stride = T * H * D * e
    torch.ops.pcie_through.multi_layer_block_table_transfer(ptrs, host_pool.view(host_blocks, T, L, 1, H * D),
                                                            pairs.to(DEV), stride, dev_blocks)
    torch.cuda.synchronize()
    got = caches.cpu()
    want = torch.zeros_like(got)
    want[:, db] = host_pool[hb].permute(2, 0, 1, 3, 4)                    # [n, T, L, H, D] -> [L, n, T, H, D]
    assert torch.equal(got.view(torch.uint8), want.view(torch.uint8))
    oracle_want = np.zeros((L, dev_blocks, stride), dtype=np.uint8)
    O.c_multi_layer_block_table_transfer(oracle_want, pool.view(torch.uint8).numpy().reshape(host_blocks, block_bytes),
                                         pairs.numpy(), T, L, 1, H * D, e, False)
    assert np.array_equal(got.view(torch.uint8).numpy().reshape(L, dev_blocks, stride), oracle_want)
    # and back into other host slots
    pool2 = memory.alloc_numa_pinned_tensor(host_blocks * block_bytes)
    host_pool2 = pool2.view(dtype).view(host_blocks, T, L, H, D)
    hb2 = torch.randperm(host_blocks, generator=gen)[:n]
    torch.ops.pcie_through.multi_layer_block_table_transfer(ptrs, host_pool2.view(host_blocks, T, L, 1, H * D),
                                                            torch.stack([hb2, db], 1).contiguous().to(DEV), stride,
                                                            dev_blocks, True)
    torch.cuda.synchronize()
    for j in range(n):
        assert torch.equal(host_pool2[hb2[j]].view(torch.uint8), host_pool[hb[j]].view(torch.uint8))
    untouched = torch.ones(host_blocks, dtype=torch.bool)
    untouched[hb2] = False
    assert int(pool2.view(host_blocks, block_bytes)[untouched].abs().max()) == 0


def test_more_layers_than_the_lds_copy_of_the_layer_table_holds():
    """L = 513: one layer more than the kernels copy into LDS, so they read the layer addresses from the
    device array instead. Both directions against the oracle, on a tiny geometry."""
    T, L, H, D, e = 1, 513, 1, 48, 1
    host_blocks, dev_blocks, n = 5, 6, 4
    announce("block-table transfer with L=%d layers (layer table read from memory), both directions" % L)
    block_bytes = T * L * H * D * e
    stride = H * T * D * e
    gen = torch.Generator().manual_seed(513)
    pool = memory.alloc_numa_pinned_tensor(host_blocks * block_bytes)
    pool.copy_(torch.randint(-128, 128, (host_blocks * block_bytes,), dtype=torch.int8, generator=gen))
    host_pool = pool.view(host_blocks, T, L, H, D)
    caches = torch.zeros(L, dev_blocks, H, T, D, dtype=torch.int8, device=DEV)
    ptrs = torch.tensor([caches[l].data_ptr() for l in range(L)], dtype=torch.int64).to(DEV)
    pairs = torch.stack([torch.randperm(host_blocks, generator=gen)[:n], torch.randperm(dev_blocks, generator=gen)[:n]], 1).contiguous()
    torch.ops.pcie_through.multi_layer_block_table_transfer(ptrs, host_pool, pairs.to(DEV), stride, dev_blocks)
    torch.cuda.synchronize()
    want = np.zeros((L, dev_blocks, stride), dtype=np.uint8)
    O.c_multi_layer_block_table_transfer(want, pool.view(torch.uint8).numpy().reshape(host_blocks, block_bytes),
                                         pairs.numpy(), T, L, H, D, e, False)
    assert np.array_equal(caches.cpu().view(torch.uint8).numpy().reshape(L, dev_blocks, stride), want)
    # and back out, to other host slots
    pool2 = memory.alloc_numa_pinned_tensor(host_blocks * block_bytes)
    pool2.fill_(0x55)
    pairs2 = torch.stack([torch.randperm(host_blocks, generator=gen)[:n], pairs[:, 1]], 1).contiguous()
    torch.ops.pcie_through.multi_layer_block_table_transfer(ptrs, pool2.view(host_blocks, T, L, H, D), pairs2.to(DEV), stride,
                                                            dev_blocks, True)
    torch.cuda.synchronize()
    want2 = np.full((host_blocks, block_bytes), 0x55, dtype=np.uint8)
    O.c_multi_layer_block_table_transfer(want, want2, pairs2.numpy(), T, L, H, D, e, True)
    assert np.array_equal(pool2.view(torch.uint8).numpy().reshape(host_blocks, block_bytes), want2)
