"""The benchmark configurations at their full sizes, launched exactly as the benchmark
launches them (the caller names the host side, so a swap-out of 64 MiB or more runs on
the link-sized grid with plain stores and a swap-in on 40 workgroups of one vector per
lane), and checked two ways:

* four planes of every case against the C oracle, whole destination planes compared
  (moved blocks and every untouched block alike);
* all planes through size-independent properties: every destination block equals its
  source block as read back through an independent path (torch indexing on the device +
  a plain device-to-host copy), every byte outside the destination blocks keeps its
  sentinel, swap-out followed by swap-in is the identity, the gather equals index_select.

The multi-GiB caches are generated on the device so that nothing has to be mirrored on
the host; the oracle gets the four planes it checks copied back.
"""
import ctypes
import time

import numpy as np
import pytest
import torch

import heterofusedkernels_amd  # noqa: F401
import pcie_through  # noqa: F401
from heterofusedkernels import memory
from heterofusedkernels_amd import capi
from heterofusedkernels_amd import workloads as W

from gpu_helpers import (announce, gather_blocks, host_ptr_table, oracle_swap_planes, ptr_table, stream_handle,
                         swap)

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(600)]
DEV = "cuda"


def _mem_available_gib():
    with open("/proc/meminfo") as f:
        for line in f:
            if line.startswith("MemAvailable"):
                return int(line.split()[1]) / 2**20
    return 0.0


def _need(host_gib, dev_gib):
    if _mem_available_gib() < host_gib * 1.5 + 8:
        pytest.skip("needs %.0f GiB of pinned host memory" % host_gib)
    free, _ = torch.cuda.mem_get_info()
    if free / 2**30 < dev_gib + 4:
        pytest.skip("needs %.0f GiB of device memory" % dev_gib)


def _device_cache(cfg, blocks):
    t0 = time.time()
    planes = [W.make_plane(cfg, l, kv, blocks, device=DEV) for l in range(cfg.layers) for kv in range(cfg.kv)]
    torch.cuda.synchronize()
    announce("  device cache %d planes x %d blocks: %.1f GiB in %.1fs" %
             (len(planes), blocks, len(planes) * blocks * cfg.block_bytes / 2**30, time.time() - t0))
    return planes, [W.as_bytes(p) for p in planes]


def _host_cache(cfg, blocks, max_alloc_gib=8, skip_on_failure=True):
    """Pinned host planes, allocated in groups of at most max_alloc_gib (one hipHostMalloc of
    80 GiB is refused on the test machines; the registry handles any number of ranges).
    Returns (None, None) instead of skipping when skip_on_failure is False."""
    t0 = time.time()
    plane_bytes = blocks * cfg.block_bytes
    per_alloc = max(1, int(max_alloc_gib * 2**30) // plane_bytes)
    pools, planes = [], []
    for first in range(0, cfg.planes, per_alloc):
        count = min(per_alloc, cfg.planes - first)
        try:
            pool = memory.alloc_numa_pinned_tensor(count * plane_bytes)
        except RuntimeError as exc:
            del pools, planes
            if not skip_on_failure:
                announce("  could not pin %.0f GiB of host memory: %s" % (cfg.planes * plane_bytes / 2**30, exc))
                return None, None
            pytest.skip("could not pin %.0f GiB of host memory: %s" % (cfg.planes * plane_bytes / 2**30, exc))
        pools.append(pool)
        planes.extend(pool.view(torch.uint8).view(count, blocks, cfg.block_bytes).unbind(0))
    announce("  pinned host cache %d planes x %d blocks: %.1f GiB in %d allocations, %.1fs" %
             (cfg.planes, blocks, cfg.planes * plane_bytes / 2**30, len(pools), time.time() - t0))
    return pools, planes


def _oracle_planes(n_planes):
    """Four planes spread over the cache: first, last and two in between."""
    return sorted({0, n_planes // 3, (2 * n_planes) // 3, n_planes - 1})


def _check_against_oracle(got_planes, dst_before, src_planes, pairs, plane_ids, what):
    """got_planes[p] (CPU uint8 [blocks, bb]) for p in plane_ids must equal the oracle's result
    on dst_before / src_planes (lists parallel to plane_ids), every block of the plane compared."""
    want = oracle_swap_planes(dst_before, src_planes, pairs, plane_ids)
    for k, p in enumerate(plane_ids):
        assert np.array_equal(got_planes[k].numpy(), want[k]), "%s: plane %d differs from the oracle" % (what, p)


def test_config3_llama70b_swap_in_full():
    cfg = W.C3_LLAMA70B_SWAP_IN
    _need(40, 41)
    announce("config 3 full: 80 layers x {K,V}, pinned [16384,16,8,128] bf16 -> device [8192,...], 1024 blocks")
    pool, host = (None, None)
    if _mem_available_gib() > 130:
        pool, host = _host_cache(cfg, cfg.host_blocks, skip_on_failure=False)
    if host is None:
        # The test machines pin at most 64 GiB per process. Everything else stays as specified
        # (160 planes, 1024 blocks per launch, device cache of 8192 blocks); only the host pool
        # the 1024 source blocks are drawn from shrinks from 16384 to 8192 blocks per plane.
        cfg = cfg.scaled(host_blocks=8192)
        announce("  host pool scaled down to %d blocks per plane (%.0f GiB)" %
                 (cfg.host_blocks, cfg.planes * cfg.host_blocks * cfg.block_bytes / 2**30))
        pool, host = _host_cache(cfg, cfg.host_blocks)
    t0 = time.time()
    for p in range(cfg.planes):                                          # U(-1,1) generated on the device, copied by hipMemcpy
        layer, kv = divmod(p, cfg.kv)
        host[p].copy_(W.as_bytes(W.make_plane(cfg, layer, kv, cfg.host_blocks, device=DEV)))
    announce("  host cache filled in %.1fs" % (time.time() - t0))
    dev = [torch.full((cfg.dev_blocks, cfg.block_bytes), 0x7E, dtype=torch.uint8, device=DEV) for _ in range(cfg.planes)]
    gen = torch.Generator().manual_seed(cfg.base_seed)
    perm = torch.randperm(cfg.host_blocks, generator=gen)
    src_ids = perm[:cfg.n_blocks].contiguous()                           # block table = slice of a random permutation
    dst_ids = torch.randperm(cfg.dev_blocks, generator=gen)[:cfg.n_blocks].contiguous()
    pairs = W.pairs_tensor(src_ids, dst_ids)
    # flags = HFK_SWAP_SRC_HOST: the launch the benchmark times for a swap-in (half as much in flight per lane)
    swap(ptr_table(dev), host_ptr_table(host), pairs.to(DEV), cfg.planes, cfg.block_bytes,
         src_blocks=cfg.host_blocks, dst_blocks=cfg.dev_blocks, flags=capi.SWAP_SRC_HOST)
    torch.cuda.synchronize()
    announce("  swap-in done, verifying")
    untouched = torch.ones(cfg.dev_blocks, dtype=torch.bool, device=DEV)
    untouched[dst_ids.to(DEV)] = False
    dst_dev = dst_ids.to(DEV)
    for p in range(cfg.planes):
        got = dev[p].index_select(0, dst_dev).cpu()
        assert torch.equal(got, host[p].index_select(0, src_ids)), "plane %d" % p
        assert bool((dev[p][untouched] == 0x7E).all()), "plane %d: untouched device blocks changed" % p
    ids = _oracle_planes(cfg.planes)
    before = torch.full((cfg.dev_blocks, cfg.block_bytes), 0x7E, dtype=torch.uint8)
    _check_against_oracle([dev[p].cpu() for p in ids], [before] * len(ids), [host[p] for p in ids], pairs, ids,
                          "config 3 swap-in")


@pytest.mark.parametrize("named", [True, False], ids=["host_side_named", "no_flags"])
def test_config4_mla_round_trip_full(named):
    cfg = W.C4_MLA_ROUNDTRIP
    _need(9, 10)
    announce("config 4 full: 61 layers [2048,64,576] bf16, swap-out 128 blocks then swap-in to other slots, host side "
             "named: %s" % named)
    planes, dev_bytes = _device_cache(cfg, cfg.dev_blocks)
    pool, host = _host_cache(cfg, cfg.host_blocks)
    gen = torch.Generator().manual_seed(cfg.base_seed)
    perm = torch.randperm(cfg.dev_blocks, generator=gen)
    out_src, in_dst = perm[:128].contiguous(), perm[128:256].contiguous()        # disjoint device slots
    host_slots = torch.randperm(cfg.host_blocks, generator=gen)[:128].contiguous()
    original = [dev_bytes[p].index_select(0, out_src.to(DEV)).clone() for p in range(cfg.planes)]
    ids = _oracle_planes(cfg.planes)
    dev_before = [dev_bytes[p].cpu() for p in ids]
    dtab, htab = ptr_table(planes), host_ptr_table(host)
    out_pairs, in_pairs = W.pairs_tensor(out_src, host_slots), W.pairs_tensor(host_slots, in_dst)
    # 549 MiB each way: with the host side named the swap-out runs on 32 workgroups of four vectors per lane
    # (72 KiB blocks in 4.5 chunks of 16 KiB: the tail-chunk path), the swap-in on 40 of one
    swap(htab, dtab, out_pairs.to(DEV), cfg.planes, cfg.block_bytes, src_blocks=cfg.dev_blocks,
         dst_blocks=cfg.host_blocks, flags=capi.SWAP_DST_HOST if named else 0)
    swap(dtab, htab, in_pairs.to(DEV), cfg.planes, cfg.block_bytes, src_blocks=cfg.host_blocks,
         dst_blocks=cfg.dev_blocks, flags=capi.SWAP_SRC_HOST if named else 0)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        assert torch.equal(dev_bytes[p].index_select(0, in_dst.to(DEV)), original[p]), "plane %d round trip" % p
        assert torch.equal(dev_bytes[p].index_select(0, out_src.to(DEV)), original[p]), "plane %d source changed" % p
        assert torch.equal(host[p].index_select(0, host_slots), original[p].cpu()), "plane %d host copy" % p
    zeros = torch.zeros(cfg.host_blocks, cfg.block_bytes, dtype=torch.uint8)
    _check_against_oracle([host[p] for p in ids], [zeros] * len(ids), dev_before, out_pairs, ids, "config 4 swap-out")
    _check_against_oracle([dev_bytes[p].cpu() for p in ids], dev_before, [host[p] for p in ids], in_pairs, ids,
                          "config 4 swap-in")


def test_config5_fp8_fragmented_full():
    cfg = W.C5_FP8_FRAGMENTED
    host_blocks = 8192
    _need(8, 17)
    announce("config 5 full: 32 layers x {K,V} [8192,16,8,128] fp8, 4096 fragmented ids: gather + swap-out, then the "
             "run-splitting swap over fragmented host slots, out and back")
    planes, dev_bytes = _device_cache(cfg, cfg.dev_blocks)
    ids = W.fragmented_ids(cfg.dev_blocks, cfg.n_blocks)
    ids_dev = ids.to(DEV)
    prefill = torch.zeros(cfg.planes, cfg.n_blocks, cfg.block_bytes, dtype=torch.uint8, device=DEV)
    gather_blocks(ptr_table(list(prefill.unbind(0))), ptr_table(planes), ids_dev, cfg.planes, cfg.block_bytes,
                  src_blocks=cfg.dev_blocks)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        assert torch.equal(prefill[p], dev_bytes[p].index_select(0, ids_dev)), "plane %d gather" % p
    pool, host = _host_cache(cfg, host_blocks)
    pairs = W.pairs_tensor(ids, torch.arange(cfg.n_blocks))
    # 4 GiB toward the host, the host side named: the launch the benchmark times for this configuration
    # (16 KiB blocks: 32 workgroups of four vectors per lane, plain stores)
    swap(host_ptr_table(host), ptr_table(planes), pairs.to(DEV), cfg.planes, cfg.block_bytes, src_blocks=cfg.dev_blocks,
         dst_blocks=host_blocks, flags=capi.SWAP_DST_HOST)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        assert torch.equal(host[p][:cfg.n_blocks], prefill[p].cpu()), "plane %d swap-out" % p
        assert int(host[p][cfg.n_blocks:].max()) == 0, "plane %d: swap-out wrote outside its slots" % p
    sel = _oracle_planes(cfg.planes)
    zeros = torch.zeros(host_blocks, cfg.block_bytes, dtype=torch.uint8)
    _check_against_oracle([host[p] for p in sel], [zeros] * len(sel), [dev_bytes[p].cpu() for p in sel], pairs, sel,
                          "config 5 swap-out")
    from oracle import oracle as O
    for p in sel:                                                        # the gather against the oracle as well
        assert np.array_equal(prefill[p].cpu().numpy(), O.c_gather_rows(dev_bytes[p].cpu().numpy(), ids.numpy())), \
            "plane %d gather differs from the oracle" % p

    # The same fragmented device blocks onto fragmented HOST slots through the mover that chooses per run of host
    # slots (long runs: staging + copy engines; the rest: the direct kernel over the short runs), 4 GiB out and back.
    host_ids = W.fragmented_ids(host_blocks, cfg.n_blocks, seed=11)
    for h in host:
        h.zero_()
    n, bb = cfg.n_blocks, cfg.block_bytes
    staging = torch.empty(cfg.planes * n * bb, dtype=torch.uint8, device=DEV)
    host_addrs = (ctypes.c_void_p * cfg.planes)(*[h.data_ptr() for h in host])
    host_np = host_ids.numpy().astype(np.int64)
    dtab, htab = ptr_table(planes), host_ptr_table(host)
    src_before = {p: dev_bytes[p].cpu() for p in sel}
    out_pairs = W.pairs_tensor(ids, host_ids)                            # rows = (device block, host slot)
    capi.check(capi.swap_blocks_auto(dtab.data_ptr(), htab.data_ptr(), host_addrs, out_pairs.to(DEV).data_ptr(),
                                     host_np.ctypes.data, cfg.planes, n, bb, bb, bb, cfg.dev_blocks, host_blocks,
                                     staging.data_ptr(), staging.numel(), True, 0, capi.SWAP_BESIDE_COMPUTE,
                                     stream_handle()), "hfk_swap_blocks_auto (out)")
    torch.cuda.synchronize()
    untouched = torch.ones(host_blocks, dtype=torch.bool)
    untouched[host_ids] = False
    for p in range(cfg.planes):
        assert torch.equal(host[p].index_select(0, host_ids), prefill[p].cpu()), "plane %d run-splitting swap-out" % p
        assert int(host[p][untouched].max()) == 0, "plane %d: run-splitting swap-out wrote outside its slots" % p
    _check_against_oracle([host[p] for p in sel], [torch.zeros(host_blocks, bb, dtype=torch.uint8)] * len(sel),
                          [src_before[p] for p in sel], out_pairs, sel, "config 5 run-splitting swap-out")
    # ... and back into other device blocks of the same set
    back = torch.roll(ids, 7)
    in_pairs = W.pairs_tensor(host_ids, back)                            # rows = (host slot, device block)
    capi.check(capi.swap_blocks_auto(dtab.data_ptr(), htab.data_ptr(), host_addrs, in_pairs.to(DEV).data_ptr(),
                                     host_np.ctypes.data, cfg.planes, n, bb, bb, bb, cfg.dev_blocks, host_blocks,
                                     staging.data_ptr(), staging.numel(), False, 0, 0, stream_handle()),
               "hfk_swap_blocks_auto (in)")
    torch.cuda.synchronize()
    back_dev = back.to(DEV)
    for p in range(cfg.planes):
        assert torch.equal(dev_bytes[p].index_select(0, back_dev), prefill[p]), "plane %d run-splitting swap-in" % p
    _check_against_oracle([dev_bytes[p].cpu() for p in sel], [src_before[p] for p in sel], [host[p] for p in sel],
                          W.pairs_tensor(host_ids, back), sel, "config 5 run-splitting swap-in")


# ---- configuration 2: one pair of caches shared by every way of launching the same swap. Kept last in
# the file: the caches stay pinned until the module ends, and configuration 3 above needs the room. ----
@pytest.fixture(scope="module")
def c2():
    """Configuration 2 at full size, shared by the tests that only differ in how they launch."""
    cfg = W.C2_LLAMA8B_SWAP_OUT
    _need(16, 11)
    announce("config 2 caches: 32 layers x {K,V} [4096,16,8,128] bf16 on the device, pinned [8192,...] per plane")
    planes, dev_bytes = _device_cache(cfg, cfg.dev_blocks)
    pool, host = _host_cache(cfg, cfg.host_blocks)                       # zero-filled by the allocator
    src_ids, dst_ids = W.block_table(cfg, src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
    assert src_ids.unique().numel() == 256 and dst_ids.unique().numel() == 256
    state = dict(cfg=cfg, planes=planes, dev_bytes=dev_bytes, pool=pool, host=host, src_ids=src_ids, dst_ids=dst_ids,
                 dtab=ptr_table(planes), htab=host_ptr_table(host))
    yield state
    state.clear()
    torch.cuda.empty_cache()


def _clear_host(host):
    for h in host:
        h.zero_()


def _verify_swap_out(c2, src_ids, dst_ids, what):
    """All planes by read-back + sentinel, four planes against the oracle."""
    cfg, host, dev_bytes = c2["cfg"], c2["host"], c2["dev_bytes"]
    untouched = torch.ones(cfg.host_blocks, dtype=torch.bool)
    untouched[dst_ids] = False
    ids_dev = src_ids.to(DEV)
    for p in range(cfg.planes):
        want = dev_bytes[p].index_select(0, ids_dev).cpu()               # independent read-back path
        assert torch.equal(host[p].index_select(0, dst_ids), want), "%s: plane %d" % (what, p)
        assert not host[p][untouched].any(), "%s: plane %d: bytes outside the destination slots changed" % (what, p)
    assert host[0].index_select(0, dst_ids).any(dim=1).all()            # N(0,1) bf16 blocks are never all zero
    ids = _oracle_planes(cfg.planes)
    zeros = torch.zeros(cfg.host_blocks, cfg.block_bytes, dtype=torch.uint8)
    _check_against_oracle([host[p] for p in ids], [zeros] * len(ids), [dev_bytes[p].cpu() for p in ids],
                          W.pairs_tensor(src_ids, dst_ids), ids, what)


@pytest.mark.parametrize("flags", [capi.SWAP_DST_HOST, 0, capi.SWAP_DST_HOST | capi.SWAP_BESIDE_COMPUTE],
                         ids=["dst_host", "no_flags", "beside_compute"])
def test_config2_llama8b_swap_out_full(c2, flags):
    """flags = HFK_SWAP_DST_HOST is the launch the benchmark times: 512 MiB >= 64 MiB, so 12 workgroups of eight
    vectors per lane, unpaced, non-temporal loads and plain stores."""
    cfg = c2["cfg"]
    announce("config 2 full, swap-out of 256 pairs x 64 planes in one launch, flags %d" % flags)
    _clear_host(c2["host"])
    swap(c2["htab"], c2["dtab"], W.pairs_tensor(c2["src_ids"], c2["dst_ids"]).to(DEV), cfg.planes, cfg.block_bytes,
         src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks, flags=flags)
    torch.cuda.synchronize()
    _verify_swap_out(c2, c2["src_ids"], c2["dst_ids"], "swap-out flags %d" % flags)


def test_config2_duplex_full(c2):
    """Swap-out of the configuration's table and a swap-in of 256 other blocks in one duplex launch."""
    cfg, host, dev_bytes = c2["cfg"], c2["host"], c2["dev_bytes"]
    announce("config 2 full, duplex: 256 pairs out + 256 pairs in, one launch")
    _clear_host(host)
    gen = torch.Generator().manual_seed(77)
    free_dev = torch.ones(cfg.dev_blocks, dtype=torch.bool)
    free_dev[c2["src_ids"]] = False
    free_host = torch.ones(cfg.host_blocks, dtype=torch.bool)
    free_host[c2["dst_ids"]] = False
    dev_free, host_free = free_dev.nonzero().flatten(), free_host.nonzero().flatten()
    in_dev = dev_free[torch.randperm(dev_free.numel(), generator=gen)[:256]].contiguous()
    in_host = host_free[torch.randperm(host_free.numel(), generator=gen)[:256]].contiguous()
    fill = torch.Generator().manual_seed(78)
    for p in range(cfg.planes):                                          # known bytes in the host slots that come in
        host[p][in_host] = torch.randint(0, 256, (256, cfg.block_bytes), dtype=torch.uint8, generator=fill)
    ids = _oracle_planes(cfg.planes)
    dev_before = [dev_bytes[p].cpu() for p in ids]
    host_before = [host[p].clone() for p in ids]
    saved = [dev_bytes[p].index_select(0, in_dev.to(DEV)).clone() for p in range(cfg.planes)]   # restored afterwards
    out_pairs = W.pairs_tensor(c2["src_ids"], c2["dst_ids"]).to(DEV)
    in_pairs = W.pairs_tensor(in_host, in_dev).to(DEV)
    bb = cfg.block_bytes
    om = capi.BlockMove(c2["htab"].data_ptr(), c2["dtab"].data_ptr(), out_pairs.data_ptr(), 256, bb, bb, cfg.dev_blocks,
                        cfg.host_blocks)
    im = capi.BlockMove(c2["dtab"].data_ptr(), c2["htab"].data_ptr(), in_pairs.data_ptr(), 256, bb, bb, cfg.host_blocks,
                        cfg.dev_blocks)
    capi.check(capi.swap_blocks_duplex(om, im, cfg.planes, bb, 0, stream_handle()), "hfk_swap_blocks_duplex")
    torch.cuda.synchronize()
    try:
        for p in range(cfg.planes):
            assert torch.equal(host[p].index_select(0, c2["dst_ids"]),
                               dev_bytes[p].index_select(0, c2["src_ids"].to(DEV)).cpu()), "plane %d out" % p
            assert torch.equal(dev_bytes[p].index_select(0, in_dev.to(DEV)).cpu(), host[p].index_select(0, in_host)), \
                "plane %d in" % p
        _check_against_oracle([host[p] for p in ids], host_before, dev_before, out_pairs, ids, "duplex, host side")
        _check_against_oracle([dev_bytes[p].cpu() for p in ids], dev_before, host_before, in_pairs, ids,
                              "duplex, device side")
    finally:
        for p in range(cfg.planes):                                      # the cache is shared: undo the swap-in
            dev_bytes[p].index_copy_(0, in_dev.to(DEV), saved[p])
        torch.cuda.synchronize()


@pytest.mark.parametrize("mover", ["staged", "auto_fragmented", "auto_no_staging"])
def test_config2_staged_and_auto_full(c2, mover):
    """The same swap-out through the staged mover (one run of host slots), and through the
    run-splitting mover on a table whose host slots are fragmented (runs + single slots)."""
    cfg, host = c2["cfg"], c2["host"]
    n, bb, planes = 256, cfg.block_bytes, cfg.planes
    announce("config 2 full, swap-out through %s" % mover)
    _clear_host(host)
    src_ids = c2["src_ids"]
    if mover == "staged":
        host_ids = torch.arange(1000, 1000 + n)
    else:
        host_ids = W.fragmented_ids(cfg.host_blocks, n, seed=9)          # geometric runs + 20 % single slots
    host_addrs = (ctypes.c_void_p * planes)(*[h.data_ptr() for h in host])
    host_np = host_ids.numpy().astype(np.int64)
    staging = torch.empty(planes * n * bb, dtype=torch.uint8, device=DEV)
    ids_dev = src_ids.to(DEV)
    if mover == "staged":
        capi.check(capi.swap_blocks_staged(c2["dtab"].data_ptr(), host_addrs, ids_dev.data_ptr(), host_np.ctypes.data,
                                           planes, n, bb, bb, bb, cfg.dev_blocks, cfg.host_blocks, staging.data_ptr(),
                                           True, 0, stream_handle()), "hfk_swap_blocks_staged")
    else:
        pairs = W.pairs_tensor(src_ids, host_ids).to(DEV)
        with_staging = mover == "auto_fragmented"
        capi.check(capi.swap_blocks_auto(c2["dtab"].data_ptr(), c2["htab"].data_ptr(), host_addrs, pairs.data_ptr(),
                                         host_np.ctypes.data, planes, n, bb, bb, bb, cfg.dev_blocks, cfg.host_blocks,
                                         staging.data_ptr() if with_staging else None,
                                         staging.numel() if with_staging else 0, True, 0, 0, stream_handle()),
                   "hfk_swap_blocks_auto")
    torch.cuda.synchronize()
    _verify_swap_out(c2, src_ids, host_ids, mover)


@pytest.mark.parametrize("bb", [4096, 8192, 12288, 20480, 69632, 131072 + 16])
def test_long_swap_out_shapes_by_block_size(bb):
    """A swap-out of 64 MiB or more toward a named host side picks its grid and its vectors per lane from the
    block size (96 x 1, 64 x 2, 32 x 4, 12 x 8; one workgroup more where the grid would split evenly over chunks
    of unequal size) and stores plainly. One launch of 64-66 MiB per block size, among them sizes with a short
    last chunk and one that is not a multiple of 256 bytes; two planes against the C oracle, all planes against
    torch indexing."""
    n_planes = 8
    n = (64 << 20) // (n_planes * bb) + 1
    dev_blocks, host_blocks = n + 7, n + 11
    announce("long swap-out, blocks of %d B: %d planes x %d blocks = %.1f MiB" % (bb, n_planes, n, n_planes * n * bb / 2**20))
    gen = torch.Generator().manual_seed(bb)
    dev = [torch.randint(0, 256, (dev_blocks, bb), dtype=torch.uint8, device=DEV,
                         generator=torch.Generator(device=DEV).manual_seed(bb + p)) for p in range(n_planes)]
    pool = memory.alloc_numa_pinned_tensor(n_planes * host_blocks * bb).view(torch.uint8)
    pool.fill_(0x6B)
    host = list(pool.view(n_planes, host_blocks, bb).unbind(0))
    src, dst = torch.randperm(dev_blocks, generator=gen)[:n], torch.randperm(host_blocks, generator=gen)[:n]
    pairs = W.pairs_tensor(src, dst)
    assert n_planes * n * bb >= 64 << 20
    swap(host_ptr_table(host), ptr_table(dev), pairs.to(DEV), n_planes, bb, src_blocks=dev_blocks, dst_blocks=host_blocks,
         flags=capi.SWAP_DST_HOST)
    torch.cuda.synchronize()
    ids = [0, n_planes - 1]
    before = [torch.full((host_blocks, bb), 0x6B, dtype=torch.uint8) for _ in ids]
    _check_against_oracle([host[p] for p in ids], before, [dev[p].cpu() for p in ids], pairs, ids, "blocks of %d B" % bb)
    src_dev = src.to(DEV)
    untouched = torch.ones(host_blocks, dtype=torch.bool)
    untouched[dst] = False
    for p in range(n_planes):
        assert torch.equal(host[p].index_select(0, dst), dev[p].index_select(0, src_dev).cpu()), "plane %d" % p
        assert bool((host[p][untouched] == 0x6B).all()), "plane %d: wrote outside its slots" % p
