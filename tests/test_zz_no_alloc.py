"""hfk_swap_blocks_staged_static (the staged swap through the library's own staging array, for
callers that may not allocate) against hfk_swap_blocks_staged with a caller-provided staging
buffer: same block tables, bit-identical host pools and device planes, on two calls in a row,
the second with a smaller input (the array keeps the first call's blocks, which must not show).
Both directions, called through the C-ABI."""
import ctypes

import numpy as np
import pytest
import torch

import heterofusedkernels_amd  # noqa: F401
import pcie_through  # noqa: F401
from heterofusedkernels import memory
from heterofusedkernels_amd import capi

from gpu_helpers import announce, stream_handle

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _host_planes(n_planes, blocks, bb, fill):
    pool = memory.alloc_numa_pinned_tensor(n_planes * blocks * bb).view(torch.uint8)
    pool.fill_(fill)
    return pool, list(pool.view(n_planes, blocks, bb).unbind(0))


def _staged(static, dev_tab, host_planes, dev_ids, host_ids, bb, dev_blocks, host_blocks, to_host, staging=None):
    n_planes, n = len(host_planes), dev_ids.shape[0]
    host_addrs = (ctypes.c_void_p * n_planes)(*[h.data_ptr() for h in host_planes])
    host_np = np.ascontiguousarray(host_ids.numpy(), dtype=np.int64)
    if static:
        rc = capi.swap_blocks_staged_static(dev_tab.data_ptr(), host_addrs, dev_ids.data_ptr(), host_np.ctypes.data,
                                            n_planes, n, bb, bb, bb, dev_blocks, host_blocks, to_host, 0,
                                            stream_handle())
        capi.check(rc, "hfk_swap_blocks_staged_static")
    else:
        rc = capi.swap_blocks_staged(dev_tab.data_ptr(), host_addrs, dev_ids.data_ptr(), host_np.ctypes.data, n_planes, n,
                                     bb, bb, bb, dev_blocks, host_blocks, staging.data_ptr(), to_host, 0, stream_handle())
        capi.check(rc, "hfk_swap_blocks_staged")


@pytest.mark.parametrize("bb", [32768, 16384 + 48])
def test_static_staging_matches_caller_staging_on_two_calls(bb):
    n_planes, dev_blocks, host_blocks = 6, 64, 96
    gen = torch.Generator().manual_seed(1234 + bb)
    dev = torch.randint(0, 256, (n_planes, dev_blocks, bb), dtype=torch.uint8, generator=gen).to(DEV)
    dev_tab = torch.tensor([dev[p].data_ptr() for p in range(n_planes)], dtype=torch.int64).to(DEV)
    # two block tables: a large one, then a smaller one whose staging footprint lies inside the first one's
    tables = []
    for n in (40, 9):
        dev_ids = torch.randperm(dev_blocks, generator=gen)[:n]
        first = int(torch.randint(0, host_blocks - n, (1,), generator=gen))
        run = list(range(first, first + n // 2))                     # a run of consecutive slots, then scattered ones
        others = [h for h in torch.randperm(host_blocks, generator=gen).tolist() if h not in run][:n - len(run)]
        tables.append((dev_ids.contiguous(), torch.tensor(run + others, dtype=torch.int64)))
    assert n_planes * tables[0][0].shape[0] * bb <= capi.STATIC_STAGING_BYTES

    # swap-out, twice in a row: library staging vs. caller staging
    pool_a, host_a = _host_planes(n_planes, host_blocks, bb, 0x5A)
    pool_b, host_b = _host_planes(n_planes, host_blocks, bb, 0x5A)
    for call, (dev_ids, host_ids) in enumerate(tables):
        announce("static staging, swap-out call %d: %d planes x %d blocks of %d B" % (call, n_planes, dev_ids.shape[0], bb))
        ids_d = dev_ids.to(DEV)
        _staged(True, dev_tab, host_a, ids_d, host_ids, bb, dev_blocks, host_blocks, True)
        staging = torch.full((n_planes * dev_ids.shape[0] * bb,), 0xEE, dtype=torch.uint8, device=DEV)
        _staged(False, dev_tab, host_b, ids_d, host_ids, bb, dev_blocks, host_blocks, True, staging)
        torch.cuda.synchronize()
        assert torch.equal(pool_a, pool_b), "swap-out call %d: host pools differ" % call
        for p in range(n_planes):     # and both are right
            assert torch.equal(host_a[p].index_select(0, host_ids), dev[p].index_select(0, ids_d).cpu())

    # swap-in, twice in a row, into two copies of a device cache
    dev_a = torch.full_like(dev, 0x11)
    dev_b = torch.full_like(dev, 0x11)
    tab_a = torch.tensor([dev_a[p].data_ptr() for p in range(n_planes)], dtype=torch.int64).to(DEV)
    tab_b = torch.tensor([dev_b[p].data_ptr() for p in range(n_planes)], dtype=torch.int64).to(DEV)
    pool_a.copy_(torch.randint(0, 256, pool_a.shape, dtype=torch.uint8, generator=gen))
    for call, (dev_ids, host_ids) in enumerate(tables):
        announce("static staging, swap-in call %d: %d planes x %d blocks of %d B" % (call, n_planes, dev_ids.shape[0], bb))
        ids_d = dev_ids.to(DEV)
        _staged(True, tab_a, host_a, ids_d, host_ids, bb, dev_blocks, host_blocks, False)
        staging = torch.full((n_planes * dev_ids.shape[0] * bb,), 0xEE, dtype=torch.uint8, device=DEV)
        _staged(False, tab_b, host_a, ids_d, host_ids, bb, dev_blocks, host_blocks, False, staging)
        torch.cuda.synchronize()
        assert torch.equal(dev_a, dev_b), "swap-in call %d: device caches differ" % call
        for p in range(n_planes):
            assert torch.equal(dev_a[p].index_select(0, ids_d).cpu(), host_a[p].index_select(0, host_ids))


def test_static_staging_rejects_what_does_not_fit():
    n_planes, bb = 4, 1 << 20
    n = capi.STATIC_STAGING_BYTES // (n_planes * bb) + 1
    dev = torch.zeros(8, dtype=torch.uint8, device=DEV)           # never touched: the call is rejected on the host
    host_addrs = (ctypes.c_void_p * n_planes)(*([4096] * n_planes))
    ids = np.zeros(n, dtype=np.int64)
    rc = capi.swap_blocks_staged_static(dev.data_ptr(), host_addrs, dev.data_ptr(), ids.ctypes.data, n_planes, n, bb, bb,
                                        bb, 0, 0, True, 0, stream_handle())
    assert rc == capi.ERR_STAGING_TOO_SMALL
    assert "static staging" in capi.status_string(rc)
