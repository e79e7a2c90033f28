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


def _device_memory_state():
    """Free device memory as the driver reports it and the counters of torch's allocator."""
    torch.cuda.synchronize()
    stats = torch.cuda.memory_stats()
    return (torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated(), torch.cuda.memory_reserved(),
            stats.get("allocation.all.allocated", 0), stats.get("segment.all.allocated", 0))


def test_static_call_allocates_nothing_eager_and_under_capture():
    """Around the static entry point nothing is allocated: free device memory and every counter of torch's
    allocator read the same before and after, for eager calls and for a capture with its replays. (The
    arguments are built beforehand; the first call on the device, which asks the runtime for the array's
    address and creates the library's one event, is made before the measurement.)"""
    n_planes, dev_blocks, host_blocks, bb, n = 4, 32, 48, 32768, 12
    gen = torch.Generator().manual_seed(77)
    dev = torch.randint(0, 256, (n_planes, dev_blocks, bb), dtype=torch.uint8, generator=gen).to(DEV)
    dev_tab = torch.tensor([dev[p].data_ptr() for p in range(n_planes)], dtype=torch.int64).to(DEV)
    pool, host = _host_planes(n_planes, host_blocks, bb, 0x33)
    host_addrs = (ctypes.c_void_p * n_planes)(*[h.data_ptr() for h in host])
    dev_ids = torch.randperm(dev_blocks, generator=gen)[:n].to(DEV)
    host_ids = torch.randperm(host_blocks, generator=gen)[:n]
    host_np = np.ascontiguousarray(host_ids.numpy(), dtype=np.int64)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()

    def call(to_host, stream):
        capi.check(capi.swap_blocks_staged_static(dev_tab.data_ptr(), host_addrs, dev_ids.data_ptr(), host_np.ctypes.data,
                                                  n_planes, n, bb, bb, bb, dev_blocks, host_blocks, to_host, 0, stream),
                   "hfk_swap_blocks_staged_static")

    announce("static staging: nothing allocated across eager calls")
    call(True, stream_handle())                       # set-up call
    before = _device_memory_state()
    for _ in range(3):
        call(True, stream_handle())
        call(False, stream_handle())
    assert _device_memory_state() == before, "eager static calls changed the device memory state"
    for p in range(n_planes):
        assert torch.equal(host[p].index_select(0, host_ids), dev[p].index_select(0, dev_ids).cpu())

    announce("static staging: nothing allocated by the call under capture, nor by replays")
    pool.fill_(0x33)
    side.wait_stream(torch.cuda.current_stream())
    torch.cuda.synchronize()
    def torch_counters():
        stats = torch.cuda.memory_stats()
        return (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), stats.get("allocation.all.allocated", 0),
                stats.get("segment.all.allocated", 0))

    with torch.cuda.graph(graph, stream=side):
        # (torch's own capture set-up allocates a little before this point; the call must add nothing to it)
        inside = torch_counters()
        call(True, side.cuda_stream)
        assert torch_counters() == inside, "torch's allocator moved during the captured call"
    captured = _device_memory_state()
    for _ in range(3):
        graph.replay()
    assert _device_memory_state() == captured, "replays changed the device memory state"
    for p in range(n_planes):
        assert torch.equal(host[p].index_select(0, host_ids), dev[p].index_select(0, dev_ids).cpu())


def test_static_call_on_another_stream_is_refused_while_the_last_one_is_pending():
    """Two static calls that would overlap on one GPU: the second, on another stream, gets
    HFK_ERR_STAGING_BUSY and moves nothing; on the same stream, or once the first has finished, it runs."""
    n_planes, dev_blocks, host_blocks, bb, n = 2, 16, 16, 4096, 5
    gen = torch.Generator().manual_seed(78)
    dev = torch.randint(0, 256, (n_planes, dev_blocks, bb), dtype=torch.uint8, generator=gen).to(DEV)
    dev_tab = torch.tensor([dev[p].data_ptr() for p in range(n_planes)], dtype=torch.int64).to(DEV)
    pool, host = _host_planes(n_planes, host_blocks, bb, 0x44)
    host_addrs = (ctypes.c_void_p * n_planes)(*[h.data_ptr() for h in host])
    dev_ids = torch.randperm(dev_blocks, generator=gen)[:n].to(DEV)
    host_ids = torch.randperm(host_blocks, generator=gen)[:n]
    host_np = np.ascontiguousarray(host_ids.numpy(), dtype=np.int64)
    a, b = torch.cuda.Stream(), torch.cuda.Stream()

    def call(stream):
        return capi.swap_blocks_staged_static(dev_tab.data_ptr(), host_addrs, dev_ids.data_ptr(), host_np.ctypes.data, n_planes,
                                              n, bb, bb, bb, dev_blocks, host_blocks, True, 0, stream.cuda_stream)

    announce("static staging: a call on a second stream while the first is pending")
    torch.cuda.synchronize()
    with torch.cuda.stream(a):
        torch.cuda._sleep(400000000)            # some tenths of a second of GPU time ahead of the first call
    assert call(a) == 0
    assert call(a) == 0                         # same stream: ordered, accepted
    rc = call(b)
    assert rc == capi.ERR_STAGING_BUSY, rc
    assert "static staging" in capi.status_string(rc)
    torch.cuda.synchronize()
    assert call(b) == 0                         # the first has finished: accepted
    torch.cuda.synchronize()
    for p in range(n_planes):
        assert torch.equal(host[p].index_select(0, host_ids), dev[p].index_select(0, dev_ids).cpu())
