#!/usr/bin/env python3
"""Benchmark of the pcieThrough hot path on one MI355X.

A *step* is one block-table swap-out launch of the Llama-3-8B-shaped configuration:
32 layers x {K,V} planes of [4096 blocks, 16, 8, 128] bf16 in HBM, 256 random distinct
source blocks -> 256 distinct slots of a pinned host cache of 8192 blocks per plane,
all 64 planes in one launch (512 MiB over the PCIe link per step). `value` is the
swap-out rate of the timed steps. The same run also measures, on the same cache,
swap-in, the multi-plane block gather (HBM -> HBM), the duplex, staged and run-splitting
swaps and what each costs a kernel on another stream, the PCIe peak seen by one large
pinned hipMemcpyAsync in each direction, a per-block hipMemcpyAsync loop, what HBM gives
a read-only / write-only / copy kernel of the gather's shape, and the torch CPU
index_select / index_copy_ path on the host cores (the reported CPU baseline). The other
three multi-layer configurations (Llama-3-70B swap-in, MLA round trip, fragmented fp8)
are then built one after the other and their swap-out, swap-in and gather measured the
same way (`configs` in the output). Every number is printed only after the moved bytes
were verified.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PCIE5_X16_GBPS = 32.0 * 16 * (128.0 / 130.0) / 8.0   # 63.0 GB/s per direction, before packet overheads
HBM_PEAK_GBPS = 8000.0                               # MI355X HBM3E
ALL_SECTIONS = ("swap_out", "swap_in", "gather", "gather_orders", "duplex", "staged", "hbm_ceiling", "tables", "repeat",
                "reference_ops")


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


def rate(nbytes, ms):
    return None if ms is None else nbytes / (ms * 1e6)


def frac(x, peak):
    return None if x is None else x / peak


class Bench:
    """Everything one run shares: modules, device, streams, timing helpers."""

    def __init__(self, args):
        import numpy as np
        import torch

        import heterofusedkernels_amd  # noqa: F401
        import pcie_through
        from heterofusedkernels import memory
        from heterofusedkernels_amd import _build, capi
        from heterofusedkernels_amd import workloads as W

        self.args, self.np, self.torch, self.pcie_through = args, np, torch, pcie_through
        self.memory, self.build, self.capi, self.W = memory, _build, capi, W
        assert torch.cuda.is_available(), "bench.py needs a GPU"
        torch.cuda.set_device(0)
        self.dev = torch.device("cuda:0")
        self.stream = torch.cuda.current_stream().cuda_stream
        # Two extra streams for the sections that run things side by side. Created once, first: HIP maps
        # streams onto a few hardware queues round-robin, and two streams that share a queue do not overlap.
        self.stream_a, self.stream_b = torch.cuda.Stream(), torch.cuda.Stream()

    def timed(self, fn, iters, warm):
        """Runs `warm` untimed calls, then `iters` calls back to back between two synchronizes.
        Returns (wall seconds for the iters calls, average milliseconds per call from one HIP event
        pair recorded on the launch stream around the whole batch, so that launch gaps of short
        kernels are hidden by the queue exactly as in steady-state use)."""
        torch = self.torch
        for _ in range(warm):
            fn()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        start.record()
        for _ in range(iters):
            fn()
        end.record()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        return wall, start.elapsed_time(end) / iters

    def launch_spread(self, fn, iters):
        """The same launch timed one at a time (an event pair per launch, a synchronize between launches):
        the first call (module load and first-touch included, by the host clock), then
        median / min / max of `iters` isolated launches by HIP events."""
        torch = self.torch
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        first_ms = (time.perf_counter() - t0) * 1e3
        times = []
        for _ in range(iters):
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            fn()
            end.record()
            torch.cuda.synchronize()
            times.append(start.elapsed_time(end))
        times.sort()
        return {"first_call_ms": first_ms, "median_ms": times[len(times) // 2], "min_ms": times[0], "max_ms": times[-1],
                "isolated_launches": iters}


class Workload:
    """One configuration's caches and block tables, resident until `release()`."""

    def __init__(self, b, cfg, key):
        torch, W, memory, pcie_through = b.torch, b.W, b.memory, b.pcie_through
        self.b, self.key, self.specified_host_blocks = b, key, cfg.host_blocks
        planes, bb, n = cfg.planes, cfg.block_bytes, cfg.n_blocks
        t0 = time.time()
        self.dev_planes = [W.make_plane(cfg, l, kv, cfg.dev_blocks, device=b.dev) for l in range(cfg.layers)
                           for kv in range(cfg.kv)]
        torch.cuda.synchronize()
        log("%s device cache: %d planes x %d blocks x %d B = %.2f GiB (%.1fs)" %
            (key, planes, cfg.dev_blocks, bb, planes * cfg.dev_blocks * bb / 2**30, time.time() - t0))
        t0 = time.time()
        # Pinned host cache, in allocations of at most 8 GiB (one huge hipHostMalloc is refused on some
        # machines). If the machine will not pin the whole pool, the pool is halved and the run says so.
        host_blocks = cfg.host_blocks
        while True:
            plane_bytes = host_blocks * bb
            per_alloc = max(1, (8 << 30) // plane_bytes)
            pools, host_planes = [], []
            try:
                for first in range(0, planes, per_alloc):
                    count = min(per_alloc, planes - first)
                    pool = memory.alloc_numa_pinned_tensor(count * plane_bytes)
                    pools.append(pool)
                    host_planes.extend(pool.view(torch.uint8).view(count, host_blocks, bb).unbind(0))
                break
            except RuntimeError as exc:
                del pools, host_planes
                if host_blocks // 2 < 2 * n:
                    raise
                log("could not pin %.1f GiB (%s); halving the host pool" % (planes * plane_bytes / 2**30, str(exc)[:80]))
                host_blocks //= 2
        if host_blocks != cfg.host_blocks:
            from dataclasses import replace
            cfg = replace(cfg, host_blocks=host_blocks)
        self.cfg, self.host_pools, self.host_planes = cfg, pools, host_planes
        log("%s pinned host cache: %d blocks per plane = %.2f GiB in %d allocations (%.1fs, NUMA node %d)" %
            (key, cfg.host_blocks, planes * cfg.host_blocks * bb / 2**30, len(pools), time.time() - t0,
             memory.device_numa_node(0)))
        self.dev_bytes = [W.as_bytes(t) for t in self.dev_planes]           # uint8 views, same storage
        self.dev_tab = pcie_through.plane_pointer_table(self.dev_planes, b.dev)
        self.host_tab = pcie_through.plane_pointer_table(host_planes, b.dev)
        if key == "c5":
            self.src_ids = W.fragmented_ids(cfg.dev_blocks, n)
            self.dst_ids = torch.arange(n)
        else:
            self.src_ids, self.dst_ids = W.block_table(cfg, src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
        self.pairs_out = W.pairs_tensor(self.src_ids, self.dst_ids).to(b.dev)      # device block -> host slot
        self.back_ids = torch.roll(self.src_ids, 1)                                # swap-in lands in other device slots
        self.pairs_in = W.pairs_tensor(self.dst_ids, self.back_ids).to(b.dev)
        self.prefill = torch.empty(planes, n, bb, dtype=torch.uint8, device=b.dev)
        self.prefill_tab = pcie_through.plane_pointer_table(list(self.prefill.unbind(0)), b.dev)
        self.ids_dev = self.src_ids.to(b.dev)
        self.payload = cfg.payload_bytes
        self.gather_alg_bytes = 2 * self.payload + 8 * n                           # read + write + the id list

    def release(self):
        for name in list(self.__dict__):
            if name not in ("b", "key"):
                delattr(self, name)
        self.b.torch.cuda.empty_cache()

    # ---- the three launches every configuration is measured on ----
    def swap_out(self, flags, stream=None):
        c, cfg = self.b.capi, self.cfg
        bb = cfg.block_bytes
        c.check(c.swap_blocks(self.host_tab.data_ptr(), self.dev_tab.data_ptr(), self.pairs_out.data_ptr(), cfg.planes,
                              cfg.n_blocks, bb, bb, bb, cfg.dev_blocks, cfg.host_blocks, 0,
                              self.b.stream if stream is None else stream, flags), "hfk_swap_blocks(out)")

    def swap_in(self, flags, stream=None):
        c, cfg = self.b.capi, self.cfg
        bb = cfg.block_bytes
        c.check(c.swap_blocks(self.dev_tab.data_ptr(), self.host_tab.data_ptr(), self.pairs_in.data_ptr(), cfg.planes,
                              cfg.n_blocks, bb, bb, bb, cfg.host_blocks, cfg.dev_blocks, 0,
                              self.b.stream if stream is None else stream, flags), "hfk_swap_blocks(in)")

    def gather(self):
        c, cfg = self.b.capi, self.cfg
        bb = cfg.block_bytes
        c.check(c.gather_blocks(self.prefill_tab.data_ptr(), self.dev_tab.data_ptr(), self.ids_dev.data_ptr(), cfg.planes,
                                cfg.n_blocks, bb, bb, cfg.dev_blocks, 0, self.b.stream), "hfk_gather_blocks")

    # ---- timed + verified sections ----
    def measure_swap_out(self, steps, warmup, flags):
        torch, cfg = self.b.torch, self.cfg
        spread = self.b.launch_spread(lambda: self.swap_out(flags), min(steps, 10))
        wall, ms = self.b.timed(lambda: self.swap_out(flags), steps, warmup)
        # verify: host slots == device source blocks read back by an independent path (torch index + D2H copy)
        t0 = time.time()
        for p in range(cfg.planes):
            want = self.dev_bytes[p].index_select(0, self.ids_dev).cpu()
            assert torch.equal(self.host_planes[p].index_select(0, self.dst_ids), want), "swap-out mismatch in plane %d" % p
        untouched = torch.ones(cfg.host_blocks, dtype=torch.bool)
        untouched[self.dst_ids] = False
        if bool(untouched.any()):
            for p in (0, cfg.planes // 2, cfg.planes - 1):
                assert int(self.host_planes[p][untouched].max()) == 0, "swap-out wrote outside its slots (plane %d)" % p
        log("%s swap-out: %.2f GB/s whole-job (%.3f ms/step wall, %.3f ms/launch by events), verified bit-exact on all %d "
            "planes (%.1fs)" % (self.key, steps * self.payload / wall / 1e9, wall * 1e3 / steps, ms, cfg.planes,
                                time.time() - t0))
        return wall, ms, spread

    def fill_host_slots(self):
        """Later sections need the swap-out's host slots filled; without that section plain torch copies do it."""
        for p in range(self.cfg.planes):
            self.host_planes[p][self.dst_ids] = self.dev_bytes[p].index_select(0, self.ids_dev).cpu()

    def measure_swap_in(self, steps, warmup, flags):
        torch, cfg = self.b.torch, self.cfg
        expect = {p: self.host_planes[p].index_select(0, self.dst_ids).clone() for p in range(cfg.planes)}
        spread = self.b.launch_spread(lambda: self.swap_in(flags), min(steps, 10))
        wall, ms = self.b.timed(lambda: self.swap_in(flags), steps, warmup)
        back_dev = self.back_ids.to(self.b.dev)
        for p in range(cfg.planes):
            got = self.dev_bytes[p].index_select(0, back_dev).cpu()
            assert torch.equal(got, expect[p]), "swap-in mismatch in plane %d" % p
        log("%s swap-in: %.2f GB/s (%.3f ms/launch), verified" % (self.key, steps * self.payload / wall / 1e9, ms))
        return wall, ms, spread

    def measure_gather(self, steps, warmup):
        """The gather is over in 0.2-2 ms: it is timed over at least 50 ms of back-to-back launches, so that
        the figure is that of a GPU at its steady clocks, like the 10-100 ms swap launches beside it."""
        torch, cfg = self.b.torch, self.cfg
        spread = self.b.launch_spread(self.gather, min(steps, 10))
        _, probe_ms = self.b.timed(self.gather, 5, warmup)
        iters = max(steps, min(400, int(50.0 / max(probe_ms, 1e-3)) + 1))
        _, ms = self.b.timed(self.gather, iters, 0)
        self.gather_iters = iters
        for p in range(cfg.planes):
            assert torch.equal(self.prefill[p], self.dev_bytes[p].index_select(0, self.ids_dev)), "gather mismatch %d" % p
        log("%s gather: %.1f GB/s of HBM traffic (%.1f payload GB/s, %.4f ms/launch over %d launches), verified" %
            (self.key, self.gather_alg_bytes / (ms * 1e6), self.payload / (ms * 1e6), ms, iters))
        return ms, spread


def pcie_peaks(b, host_pool):
    """The link as one large pinned copy sees it, both directions."""
    torch = b.torch
    big = min(1 << 30, host_pool.numel())
    big_d = torch.empty(big, dtype=torch.int8, device=b.dev)
    big_h = host_pool[:big]
    _, ms = b.timed(lambda: big_h.copy_(big_d, non_blocking=True), 5, 2)
    d2h = big / (ms * 1e6)
    _, ms = b.timed(lambda: big_d.copy_(big_h, non_blocking=True), 5, 2)
    h2d = big / (ms * 1e6)
    host_pool[:big].zero_()
    log("hipMemcpyAsync %d MiB pinned: D2H %.2f GB/s, H2D %.2f GB/s (link %.1f GB/s theoretical)" %
        (big >> 20, d2h, h2d, PCIE5_X16_GBPS))
    return d2h, h2d, big


def section_duplex(b, w, steps, warmup):
    """Both directions at once: two launches on two streams, one duplex launch, two opposite memcpys."""
    torch, capi, W, cfg = b.torch, b.capi, b.W, w.cfg
    planes, bb, n = cfg.planes, cfg.block_bytes, cfg.n_blocks
    gen = torch.Generator().manual_seed(cfg.base_seed + 77)
    free_dev = torch.ones(cfg.dev_blocks, dtype=torch.bool)
    free_dev[w.src_ids] = False
    free_dev[w.back_ids] = False
    free_host = torch.ones(cfg.host_blocks, dtype=torch.bool)
    free_host[w.dst_ids] = False
    dev_free, host_free = free_dev.nonzero().flatten(), free_host.nonzero().flatten()
    n2 = min(n, dev_free.numel(), host_free.numel())
    in_dev = dev_free[torch.randperm(dev_free.numel(), generator=gen)[:n2]]      # disjoint from the swap-out's blocks
    in_host = host_free[torch.randperm(host_free.numel(), generator=gen)[:n2]]
    for p in range(planes):                                                      # give the host slots known content
        w.host_planes[p][in_host] = w.dev_bytes[p].index_select(0, w.ids_dev[:n2]).cpu()
    pairs_in2 = W.pairs_tensor(in_host, in_dev).to(b.dev)
    s_out, s_in = b.stream_a, b.stream_b

    def both():
        capi.check(capi.swap_blocks(w.host_tab.data_ptr(), w.dev_tab.data_ptr(), w.pairs_out.data_ptr(), planes, n, bb,
                                    bb, bb, cfg.dev_blocks, cfg.host_blocks, 0, s_out.cuda_stream))
        capi.check(capi.swap_blocks(w.dev_tab.data_ptr(), w.host_tab.data_ptr(), pairs_in2.data_ptr(), planes, n2, bb,
                                    bb, bb, cfg.host_blocks, cfg.dev_blocks, 0, s_in.cuda_stream))

    def check_both():
        for p in range(planes):
            assert torch.equal(w.host_planes[p].index_select(0, w.dst_ids), w.dev_bytes[p].index_select(0, w.ids_dev).cpu())
            assert torch.equal(w.dev_bytes[p].index_select(0, in_dev.to(b.dev)).cpu(), w.host_planes[p].index_select(0, in_host))

    both()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        both()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    check_both()
    total = steps * (n + n2) * planes * bb
    # ... and the same two block tables in ONE duplex launch
    om = capi.BlockMove(w.host_tab.data_ptr(), w.dev_tab.data_ptr(), w.pairs_out.data_ptr(), n, bb, bb, cfg.dev_blocks,
                        cfg.host_blocks)
    im = capi.BlockMove(w.dev_tab.data_ptr(), w.host_tab.data_ptr(), pairs_in2.data_ptr(), n2, bb, bb, cfg.host_blocks,
                        cfg.dev_blocks)

    def clear_targets():                                                 # make a launch prove itself
        for p in range(planes):
            w.host_planes[p][w.dst_ids] = 0
            w.dev_bytes[p].index_fill_(0, in_dev.to(b.dev), 0)

    clear_targets()
    _, ms_d = b.timed(lambda: capi.check(capi.swap_blocks_duplex(om, im, planes, bb, 0, b.stream), "hfk_swap_blocks_duplex"),
                      steps, warmup)
    check_both()
    clear_targets()
    _, ms_b = b.timed(lambda: capi.check(capi.swap_blocks_duplex(om, im, planes, bb, 0, b.stream, capi.SWAP_BESIDE_COMPUTE),
                                         "hfk_swap_blocks_duplex(beside)"), steps, warmup)
    check_both()
    duplex_gbps = (n + n2) * planes * bb / (ms_d * 1e6)
    # the copy engines doing the same thing: two opposite 512 MiB pinned copies on the two streams
    host_pool = w.host_pools[0]
    half = min(1 << 29, host_pool.numel() // 2)
    d_a = torch.empty(half, dtype=torch.int8, device=b.dev)
    d_b = torch.empty(half, dtype=torch.int8, device=b.dev)
    h_a, h_b = host_pool[-half:], host_pool[-2 * half:-half]
    keep_a, keep_b = h_a.clone(), h_b.clone()   # these bytes belong to the host cache: put them back afterwards

    def both_memcpy():
        with torch.cuda.stream(s_out):
            h_a.copy_(d_a, non_blocking=True)
        with torch.cuda.stream(s_in):
            d_b.copy_(h_b, non_blocking=True)

    both_memcpy()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        both_memcpy()
    torch.cuda.synchronize()
    dt_m = time.perf_counter() - t0
    h_a.copy_(keep_a)
    h_b.copy_(keep_b)
    out = {"one_launch_GBps_both_directions": duplex_gbps,
           "one_launch_pct_of_2x_pcie5_x16": 100 * duplex_gbps / (2 * PCIE5_X16_GBPS),
           "one_launch_beside_compute_GBps_both_directions": (n + n2) * planes * bb / (ms_b * 1e6),
           "two_launches_two_streams_GBps_both_directions": total / dt / 1e9, "out_blocks": n, "in_blocks": n2,
           "memcpy_both_directions_GBps": 5 * 2 * half / dt_m / 1e9}
    log("duplex, verified: swap_blocks_duplex (one launch) %.2f GB/s summed (%.2f with HFK_SWAP_BESIDE_COMPUTE); swap-out + "
        "swap-in on two streams %.2f GB/s summed; two opposite hipMemcpyAsync %.2f GB/s summed" %
        (duplex_gbps, out["one_launch_beside_compute_GBps_both_directions"], total / dt / 1e9,
         out["memcpy_both_directions_GBps"]))
    return out, {"om": om, "im": im, "keepalive": pairs_in2}


def section_staged(b, w, steps, warmup, out_flags):
    """The staged swap (HBM kernel + DMA copies), the run-splitting swap on fragmented host slots, the
    HFK_SWAP_BESIDE_COMPUTE launch shapes, and what each way of swapping costs a kernel on another stream."""
    torch, capi, W, np, cfg = b.torch, b.capi, b.W, b.np, w.cfg
    planes, bb, n, payload = cfg.planes, cfg.block_bytes, cfg.n_blocks, w.payload
    stream = b.stream
    host_run = torch.arange(0, n)     # the earlier sections' results are verified by now: their host slots may be reused
    host_addrs = torch.tensor([t.data_ptr() for t in w.host_planes], dtype=torch.int64)
    staging_buf = torch.empty(planes, n, bb, dtype=torch.uint8, device=b.dev)
    back_dev = w.back_ids.to(b.dev)

    def staged(to_host, dev_ids, host_ids, st=None, staging=staging_buf):
        capi.check(capi.swap_blocks_staged(w.dev_tab.data_ptr(), host_addrs.data_ptr(), dev_ids.data_ptr(),
                                           host_ids.data_ptr(), planes, n, bb, bb, bb, cfg.dev_blocks, cfg.host_blocks,
                                           staging.data_ptr(), to_host, 0, stream if st is None else st),
                   "hfk_swap_blocks_staged")

    def staged_out(st=None):
        staged(True, w.ids_dev, host_run, st)

    def staged_in(st=None):
        staged(False, back_dev, host_run, st)

    _, ms_so = b.timed(staged_out, steps, warmup)
    for p in range(planes):
        assert torch.equal(w.host_planes[p][:n], w.dev_bytes[p].index_select(0, w.ids_dev).cpu())
    _, ms_si = b.timed(staged_in, steps, warmup)
    for p in range(planes):
        assert torch.equal(w.dev_bytes[p].index_select(0, back_dev).cpu(), w.host_planes[p][:n])
    # both directions at once on two streams (two DMA engines); disjoint device blocks and host runs
    staging_b = torch.empty(planes, n, bb, dtype=torch.uint8, device=b.dev)
    run_b = torch.arange(n, 2 * n)

    def staged_both():
        staged(True, w.ids_dev, host_run, b.stream_a.cuda_stream)
        staged(False, back_dev, run_b, b.stream_b.cuda_stream, staging_b)

    staged_both()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        staged_both()
    torch.cuda.synchronize()
    staged_duplex_gbps = steps * 2 * payload / (time.perf_counter() - t0) / 1e9
    del staging_b

    # ---- fragmented host slots: runs of consecutive slots (geometric lengths) + 20 % single slots ----
    frag_host = W.fragmented_ids(cfg.host_blocks, n, seed=cfg.base_seed + 40)
    frag_np = np.ascontiguousarray(frag_host.numpy(), dtype=np.int64)
    runs = int((np.diff(frag_np) != 1).sum()) + 1
    pairs_frag_out = W.pairs_tensor(w.src_ids, frag_host).to(b.dev)
    pairs_frag_in = W.pairs_tensor(frag_host, w.back_ids).to(b.dev)

    def auto(to_host, flags, min_run=0, st=None):
        pairs = pairs_frag_out if to_host else pairs_frag_in
        capi.check(capi.swap_blocks_auto(w.dev_tab.data_ptr(), w.host_tab.data_ptr(), host_addrs.data_ptr(), pairs.data_ptr(),
                                         frag_np.ctypes.data, planes, n, bb, bb, bb, cfg.dev_blocks, cfg.host_blocks,
                                         staging_buf.data_ptr(), staging_buf.numel(), to_host, min_run, flags,
                                         stream if st is None else st), "hfk_swap_blocks_auto")

    def check_frag_out():
        for p in range(planes):
            assert torch.equal(w.host_planes[p].index_select(0, frag_host), w.dev_bytes[p].index_select(0, w.ids_dev).cpu()), \
                "fragmented swap-out mismatch in plane %d" % p

    def check_frag_in():
        for p in range(planes):
            assert torch.equal(w.dev_bytes[p].index_select(0, back_dev).cpu(), w.host_planes[p].index_select(0, frag_host)), \
                "fragmented swap-in mismatch in plane %d" % p

    def clear_frag():
        for p in range(planes):
            w.host_planes[p][frag_host] = 0

    frag = {"host_slots": "%d slots in %d runs of consecutive slots (geometric run lengths, 20 %% single slots)" % (n, runs)}
    beside = capi.SWAP_BESIDE_COMPUTE

    def timed_frag(fn, check, clear):
        if clear:
            clear_frag()
        _, ms = b.timed(fn, max(3, steps // 2), 2)
        check()
        return payload / (ms * 1e6)

    for name, fn, check in (
            ("auto_out_GBps", lambda: auto(True, 0), check_frag_out),
            ("auto_beside_compute_out_GBps", lambda: auto(True, beside), check_frag_out),
            ("staged_out_GBps", lambda: staged(True, w.ids_dev, frag_host), check_frag_out),
            ("direct_out_GBps", lambda: auto(True, 0, 5000), check_frag_out),
            ("auto_in_GBps", lambda: auto(False, 0), check_frag_in),
            ("auto_beside_compute_in_GBps", lambda: auto(False, beside), check_frag_in),
            ("staged_in_GBps", lambda: staged(False, back_dev, frag_host), check_frag_in),
            ("direct_in_GBps", lambda: auto(False, 0, 5000), check_frag_in)):
        frag[name] = timed_frag(fn, check, name.endswith("out_GBps"))
    # the whole trade-off: runs of at least k slots to the copy engines, the rest to the paced small grid
    frag["by_min_run_blocks"] = {}
    for k in (1, 2, 3, 4, 6, 8, 16):
        in_long = int(sum(len(r) for r in np.split(frag_np, np.flatnonzero(np.diff(frag_np) != 1) + 1) if len(r) >= k))
        frag["by_min_run_blocks"][str(k)] = {
            "blocks_to_copy_engines": in_long,
            "out_GBps": timed_frag(lambda: auto(True, beside, k), check_frag_out, True),
            "in_GBps": timed_frag(lambda: auto(False, beside, k), check_frag_in, False)}
    log("fragmented host slots (%d runs), verified: out auto %.2f / auto beside compute %.2f / staged %.2f / direct %.2f GB/s; "
        "in %.2f / %.2f / %.2f / %.2f GB/s" %
        (runs, frag["auto_out_GBps"], frag["auto_beside_compute_out_GBps"], frag["staged_out_GBps"], frag["direct_out_GBps"],
         frag["auto_in_GBps"], frag["auto_beside_compute_in_GBps"], frag["staged_in_GBps"], frag["direct_in_GBps"]))
    log("  by smallest run sent to the copy engines (HFK_SWAP_BESIDE_COMPUTE), out/in GB/s: " +
        ", ".join("%s: %.1f/%.1f (%d blocks)" % (k, v["out_GBps"], v["in_GBps"], v["blocks_to_copy_engines"])
                  for k, v in frag["by_min_run_blocks"].items()))

    # ---- kernels on another stream: alone, and beside each way of swapping. Three neighbours: a compute-bound
    # GEMM, an HBM-bound 1 GiB device copy and an attention kernel (mixed). ----
    side, comp = b.stream_a, b.stream_b
    ga = torch.randn(8192, 8192, device=b.dev, dtype=torch.bfloat16)
    gb = torch.randn(8192, 8192, device=b.dev, dtype=torch.bfloat16)
    ca = torch.empty(1 << 30, dtype=torch.uint8, device=b.dev)
    cb = torch.empty(1 << 30, dtype=torch.uint8, device=b.dev)
    qkv = torch.randn(8, 32, 2048, 128, device=b.dev, dtype=torch.bfloat16)
    neighbours = {
        "gemm_8192_bf16": (lambda: torch.mm(ga, gb), 30),
        "device_copy_1GiB": (lambda: ca.copy_(cb), 40),
        "sdpa_8x32x2048x128_bf16": (lambda: torch.nn.functional.scaled_dot_product_attention(qkv, qkv, qkv, is_causal=True), 30),
    }
    for fn, _ in neighbours.values():
        for _ in range(3):
            fn()

    def neighbour_ms(fn, reps, side_fn=None, side_reps=0):
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(side_reps):
            side_fn(side.cuda_stream)
        with torch.cuda.stream(comp):
            e0.record()
            for _ in range(reps):
                fn()
            e1.record()
        e1.synchronize()
        covered = side_fn is None or not side.query()      # the swaps must outlast the neighbour
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / reps, covered

    out_host, in_host = capi.SWAP_DST_HOST, capi.SWAP_SRC_HOST
    ways = {"throughput_out": lambda st: w.swap_out(out_flags, st), "throughput_in": lambda st: w.swap_in(in_host, st),
            "beside_compute_out": lambda st: w.swap_out(out_host | beside, st),
            "beside_compute_in": lambda st: w.swap_in(in_host | beside, st),
            "staged_out": staged_out, "staged_in": staged_in,
            "auto_fragmented_out": lambda st: auto(True, 0, 0, st),
            "auto_fragmented_in": lambda st: auto(False, 0, 0, st),
            "auto_fragmented_beside_compute_out": lambda st: auto(True, beside, 0, st),
            "auto_fragmented_beside_compute_in": lambda st: auto(False, beside, 0, st),
            "staged_fragmented_out": lambda st: staged(True, w.ids_dev, frag_host, st),
            "staged_fragmented_in": lambda st: staged(False, back_dev, frag_host, st)}
    for k in (2, 8):      # the other ends of the trade-off: more of the table on the copy engines, or less
        ways["auto_fragmented_beside_compute_out_min_run_%d" % k] = lambda st, k=k: auto(True, beside, k, st)
        ways["auto_fragmented_beside_compute_in_min_run_%d" % k] = lambda st, k=k: auto(False, beside, k, st)
    # The floor: kernels that touch no memory at all and only stay resident (one sleeping wavefront; 16 workgroups)
    bench_lib = ctypes.CDLL(b.build.HFK_BENCH_SO)
    bench_lib.hfkb_idle_resident.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p]
    idle_ticks = int(payload / 55e9 * 1e8)                                  # as long as one swap
    ways["one_idle_wavefront"] = lambda st: bench_lib.hfkb_idle_resident(1, 64, idle_ticks, st)
    ways["sixteen_idle_workgroups"] = lambda st: bench_lib.hfkb_idle_resident(16, 256, idle_ticks, st)
    # Reading host memory and nothing else, through the vector memory path (24 workgroups, like the
    # beside-compute swap-in) and through the scalar path (40 workgroups of 8 wavefronts): the same bytes
    # of the host pool, a checksum kept.
    bench_lib.hfkb_host_read.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_void_p,
                                         ctypes.c_void_p]
    read_bytes = min(payload, w.host_pools[0].numel()) & ~255
    read_from = b.memory.get_device_ptr(w.host_pools[0].data_ptr())
    checksums = torch.zeros(40 * 256, dtype=torch.int32, device=b.dev)
    ways["host_read_vector_path"] = lambda st: bench_lib.hfkb_host_read(0, read_from, read_bytes, 24, checksums.data_ptr(), st)
    ways["host_read_scalar_path"] = lambda st: bench_lib.hfkb_host_read(1, read_from, read_bytes, 40, checksums.data_ptr(), st)
    host_read_gbps = {}
    for name in ("host_read_vector_path", "host_read_scalar_path"):
        _, ms_r = b.timed(lambda: ways[name](stream), max(3, steps // 4), 1)
        host_read_gbps[name] = round(read_bytes / (ms_r * 1e6), 2)
    # own rate of the beside-compute launch shape, GPU otherwise idle; result checked like the plain swap-out's
    for p_ in range(planes):
        w.host_planes[p_][w.dst_ids] = 0
    _, ms_bo = b.timed(lambda: ways["beside_compute_out"](stream), steps, warmup)
    for p_ in range(planes):
        assert torch.equal(w.host_planes[p_].index_select(0, w.dst_ids), w.dev_bytes[p_].index_select(0, w.ids_dev).cpu()), \
            "beside-compute swap-out mismatch in plane %d" % p_
    _, ms_bi = b.timed(lambda: ways["beside_compute_in"](stream), steps, warmup)
    for p_ in range(planes):
        assert torch.equal(w.dev_bytes[p_].index_select(0, back_dev).cpu(), w.host_planes[p_].index_select(0, w.dst_ids)), \
            "beside-compute swap-in mismatch in plane %d" % p_
    alone = {k: neighbour_ms(fn, reps)[0] for k, (fn, reps) in neighbours.items()}
    side_reps = max(2, int(round(0.09 / (payload / 55e9))))          # about 90 ms of swapping
    slowdown = {}
    for way, side_fn in ways.items():
        slowdown[way] = {}
        for k, (fn, reps) in neighbours.items():
            ms, covered = neighbour_ms(fn, reps, side_fn, side_reps)
            slowdown[way][k] = round(ms / alone[k], 3) if covered else None
    del ga, gb, ca, cb, qkv, staging_buf
    staged_out_json = {"swap_out_GBps": payload / (ms_so * 1e6), "swap_in_GBps": payload / (ms_si * 1e6),
                       "out_and_in_on_two_streams_GBps": staged_duplex_gbps,
                       "host_slots": "one run of %d consecutive slots per plane (%.1f MiB per plane, 2-D DMA copies over "
                                     "evenly spaced planes)" % (n, n * bb / 2**20)}
    beside_json = {"swap_out_GBps": payload / (ms_bo * 1e6), "swap_in_GBps": payload / (ms_bi * 1e6),
                   "link_MBps_from_sysfs": capi.get_tuning(capi.KNOB_LINK_MBPS),
                   "neighbour_ms_alone": alone,
                   "host_read_GBps": host_read_gbps,
                   "neighbour_slowdown": slowdown,
                   "how": "each neighbour runs %s times on one stream while %d swaps of %d MiB are queued on another; "
                          "x = its time per call / its time alone; null = the swaps ended first. one_idle_wavefront / "
                          "sixteen_idle_workgroups: kernels that only sleep, the price of sharing the GPU at all" %
                          ("/".join(str(r) for _, r in neighbours.values()), side_reps, payload >> 20)}
    log("staged swap, verified: out %.2f GB/s, in %.2f GB/s, both on two streams %.2f GB/s summed" %
        (staged_out_json["swap_out_GBps"], staged_out_json["swap_in_GBps"], staged_duplex_gbps))
    log("swap with HFK_SWAP_BESIDE_COMPUTE, verified: out %.2f GB/s, in %.2f GB/s" %
        (beside_json["swap_out_GBps"], beside_json["swap_in_GBps"]))
    for way in ways:
        log("  neighbours beside %-35s %s" % (way + ":", ", ".join("%s x%s" % (k.split("_")[0], v)
                                                                    for k, v in slowdown[way].items())))
    return staged_out_json, beside_json, frag


def section_tables(b, w, steps):
    """The swap-out over different kinds of block table (same size as the workload's own): a paced launch must hold
    its rate whatever the table looks like. Destroys the host cache's content, so it runs after everything else;
    every launch shape is verified on every table (two planes, moved blocks byte for byte)."""
    torch, capi, W, cfg = b.torch, b.capi, b.W, w.cfg
    planes, bb, n = cfg.planes, cfg.block_bytes, cfg.n_blocks
    gen = torch.Generator().manual_seed(cfg.base_seed + 99)
    ar = torch.arange(n)

    def runs_of(k, blocks):
        starts = torch.randperm(blocks // k, generator=gen)[:n // k]
        return (starts[:, None] * k + torch.arange(k)).flatten()[:n]

    tables = {
        "consecutive_both": (ar + 7, ar + 5),
        "device_descending": ((n - 1 - ar) + 7, ar + 5),
        "device_every_2nd": (2 * ar, ar + 5),
        "host_every_2nd": (ar + 7, 2 * ar),
        "both_every_2nd": (2 * ar, 2 * ar + 1),
        "runs_of_8_shuffled": (runs_of(8, cfg.dev_blocks), runs_of(8, cfg.host_blocks)),
        "random": (torch.randperm(cfg.dev_blocks, generator=gen)[:n], torch.randperm(cfg.host_blocks, generator=gen)[:n]),
        "the_workloads_own": (w.src_ids, w.dst_ids),
    }
    tables = {k: v for k, v in tables.items()                       # a pool too small for a strided table goes without it
              if int(v[0].max()) < cfg.dev_blocks and int(v[1].max()) < cfg.host_blocks}
    shapes = {"host_side_named": capi.SWAP_DST_HOST, "beside_compute": capi.SWAP_DST_HOST | capi.SWAP_BESIDE_COMPUTE,
              "no_flags": 0}
    payload = planes * n * bb
    out = {k: {} for k in shapes}
    for name, (src, dst) in tables.items():
        pairs = W.pairs_tensor(src, dst).to(b.dev)
        src_dev = src.to(b.dev)
        for shape, flags in shapes.items():
            for p in (0, planes - 1):
                w.host_planes[p][dst] = 0
            _, ms = b.timed(lambda: capi.check(capi.swap_blocks(
                w.host_tab.data_ptr(), w.dev_tab.data_ptr(), pairs.data_ptr(), planes, n, bb, bb, bb, cfg.dev_blocks,
                cfg.host_blocks, 0, b.stream, flags), "hfk_swap_blocks"), max(4, steps // 2), 1)
            for p in (0, planes - 1):
                assert torch.equal(w.host_planes[p].index_select(0, dst), w.dev_bytes[p].index_select(0, src_dev).cpu()), \
                    "swap-out mismatch on table %s, shape %s, plane %d" % (name, shape, p)
            out[shape][name] = round(payload / (ms * 1e6), 2)
    for shape, rates in out.items():
        log("swap-out by block table, %-16s min %.2f max %.2f GB/s | %s" %
            (shape + ":", min(rates.values()), max(rates.values()), ", ".join("%s %.1f" % kv for kv in rates.items())))
    return {"GBps": out, "blocks": n, "how": "%d launches per table and shape, one HIP event pair around them; "
            "two planes verified per table and shape" % max(4, steps // 2)}


def section_gather_orders(b, w, steps):
    """The block gather on the workload's own cache under different orders of the same kind of work: which
    blocks are read (in sequence, random, random but sorted, random within 2 MiB neighbourhoods) and in
    which order the destination is written (in sequence, or at random with the source in sequence). Every
    launch reads and writes the same number of bytes with the same kernel shape; what differs is locality in
    DRAM rows and in address translation. Verified on every plane before a figure is kept."""
    torch, capi, cfg = b.torch, b.capi, w.cfg
    planes, bb, n = cfg.planes, cfg.block_bytes, cfg.n_blocks
    gen = torch.Generator().manual_seed(cfg.base_seed + 7)
    own = w.src_ids
    per_2mib = max(1, (2 << 20) // bb)
    groups = torch.randperm(cfg.dev_blocks // per_2mib, generator=gen)[:max(1, n // per_2mib)]
    grouped = torch.cat([g * per_2mib + torch.randperm(per_2mib, generator=gen) for g in groups.tolist()])[:n]
    orders = {
        "the_workloads_own_random": own,
        "sequential": torch.arange(n) + 7,
        "random_sorted": torch.sort(own).values,
        "random_within_2MiB_groups": grouped,
    }
    out = {}
    iters = max(steps, 200)
    for name, ids in orders.items():
        if ids.numel() != n or int(ids.max()) >= cfg.dev_blocks:
            continue
        ids_dev = ids.to(b.dev)

        def launch():
            capi.check(capi.gather_blocks(w.prefill_tab.data_ptr(), w.dev_tab.data_ptr(), ids_dev.data_ptr(), planes, n, bb, bb,
                                          cfg.dev_blocks, 0, b.stream), "hfk_gather_blocks")
        w.prefill.zero_()
        _, ms = b.timed(launch, iters, 3)
        for p in range(planes):
            assert torch.equal(w.prefill[p], w.dev_bytes[p].index_select(0, ids_dev)), "gather mismatch (%s, plane %d)" % (name, p)
        out[name] = round(w.gather_alg_bytes / (ms * 1e6), 1)
    # the same bytes with the source in sequence and the destination at random: a device-to-device swap through the
    # same block-copy body, one vector per lane and one workgroup per chunk like the gather
    perm = torch.randperm(n, generator=gen)
    pairs = b.W.pairs_tensor(torch.arange(n) + 7, perm).to(b.dev)
    with capi.thread_tuning({capi.KNOB_SWAP_UNROLL: capi.get_tuning(capi.KNOB_UNROLL)}):
        def scatter():
            capi.check(capi.swap_blocks(w.prefill_tab.data_ptr(), w.dev_tab.data_ptr(), pairs.data_ptr(), planes, n, bb, bb, bb,
                                        cfg.dev_blocks, n, 1 << 20, b.stream, 0), "hfk_swap_blocks(device to device)")
        w.prefill.zero_()
        _, ms = b.timed(scatter, iters, 3)
    seq_dev, perm_dev = (torch.arange(n) + 7).to(b.dev), perm.to(b.dev)
    for p in range(planes):
        assert torch.equal(w.prefill[p].index_select(0, perm_dev), w.dev_bytes[p].index_select(0, seq_dev)), "scatter mismatch %d" % p
    out["sequential_source_random_destination"] = round(w.gather_alg_bytes / (ms * 1e6), 1)
    log("gather by order of work, GB/s of HBM traffic: " + ", ".join("%s %.0f" % kv for kv in out.items()))
    return {"traffic_GBps": out, "launches_timed": iters, "frac_of_hbm_peak": {k: round(v / HBM_PEAK_GBPS, 4) for k, v in out.items()}}


def section_repeat(b, w, steps, warmup, flags, first_value):
    """The timed step once more, as the last thing done on the headline workload: the same launch on the same
    table and pool after everything else has run. Also what a paced launch of the same swap does with its
    schedule (hfk's pace report): a launch that holds its pace ends with ran <= allotted."""
    torch, capi, cfg = b.torch, b.capi, w.cfg
    for p in range(cfg.planes):
        w.host_planes[p][w.dst_ids] = 0
    spread = b.launch_spread(lambda: w.swap_out(flags), min(steps, 10))
    batches = []
    for _ in range(3):      # three batches like the timed one: what one batch alone says about this machine's noise
        wall, ms = b.timed(lambda: w.swap_out(flags), steps, warmup)
        batches.append((steps * w.payload / wall / 1e9, w.payload / (ms * 1e6)))
    for p in range(cfg.planes):
        want = w.dev_bytes[p].index_select(0, w.ids_dev).cpu()
        assert torch.equal(w.host_planes[p].index_select(0, w.dst_ids), want), "repeated swap-out mismatch in plane %d" % p
    gbps, kernel_gbps = sorted(batches)[1]
    iso = {k: round(w.payload / (spread[k] * 1e6), 2) for k in ("median_ms", "min_ms", "max_ms")}
    out = {"GBps": gbps, "kernel_GBps": kernel_gbps, "how": "median of three batches of %d back-to-back launches" % steps,
           "batches_GBps": [round(x[0], 2) for x in batches],
           "isolated_launches_GBps": {"median": iso["median_ms"], "slowest": iso["max_ms"], "fastest": iso["min_ms"]},
           "first_measurement_GBps": first_value,
           "last_over_first": None if not first_value else gbps / first_value}
    log("swap-out repeated at the end: %s GB/s in three batches (first measurement %s), isolated launches %.2f / %.2f / %.2f "
        "(slowest / median / fastest)" % (" / ".join("%.2f" % x[0] for x in batches),
                                           "%.2f" % first_value if first_value else "-", iso["max_ms"], iso["median_ms"], iso["min_ms"]))
    # a paced launch of the same swap and how it kept its schedule: at a fixed pace, and with the pace that the
    # launches before it set (the library's default for a paced throughput-mode swap)
    report = torch.zeros(64 * 8, dtype=torch.int64, device=b.dev)
    paced = {}
    for permille in (890, 900):
        with capi.thread_tuning({capi.KNOB_THROUGHPUT_PACE_PERMILLE: permille, capi.KNOB_ADAPTIVE_PACE: 0,
                                 capi.KNOB_PACE_REPORT: report.data_ptr()}):
            _, pms = b.timed(lambda: w.swap_out(capi.SWAP_DST_HOST), max(4, steps // 2), 1)
            grid = capi.get_tuning(capi.KNOB_PACED_WORKGROUPS)
        rows = report.cpu().view(64, 8)[:grid]
        ran, allotted, turns, late, worst = (rows[:, i].double() for i in range(5))
        paced["fixed_at_0.%d_of_link" % (permille // 10)] = {
            "GBps": round(w.payload / (pms * 1e6), 2), "workgroups": grid, "launch_ms": round(pms, 4),
            "slowest_workgroup_ran_ms": round(float(ran.max()) / 1e5, 4),
            "allotted_ms": round(float(allotted.max()) / 1e5, 4),
            "ran_over_allotted": round(float((ran / allotted.clamp(min=1)).max()), 4),
            "late_turns_pct": round(100 * float(late.sum() / turns.sum().clamp(min=1)), 2),
            "largest_delay_us": round(float(worst.max()) / 100.0, 1)}
    for permille in (870, 910):          # wherever it starts, the pace set between launches ends up in the same place
        with capi.thread_tuning({capi.KNOB_THROUGHPUT_PACE_PERMILLE: permille}):
            b.timed(lambda: w.swap_out(capi.SWAP_DST_HOST), 40, 0)
            _, pms = b.timed(lambda: w.swap_out(capi.SWAP_DST_HOST), max(4, steps // 2), 0)
        st = capi.pace_state()
        paced["set_between_launches_from_0.%d" % (permille // 10)] = {
            "GBps": round(w.payload / (pms * 1e6), 2), "factor": round(st[0] / 65536.0, 4),
            "offered_share_of_link": round(permille / 1000.0 / (st[0] / 65536.0), 4),
            "late_turns_pct_of_last_launch": round(100 * st[6] / 65536.0, 2), "launches_settled": st[5]}
    for p in (0, cfg.planes - 1):
        want = w.dev_bytes[p].index_select(0, w.ids_dev).cpu()
        assert torch.equal(w.host_planes[p].index_select(0, w.dst_ids), want), "paced swap-out mismatch in plane %d" % p
    out["paced_launch_of_the_same_swap"] = paced
    log("paced launches of the same swap: %s" % json.dumps(paced))
    return out


def section_reference_ops(b):
    """The reference's own three ops on the shapes its README quotes (pcieThrough/tests/README.md:34-42,70-75):
    gather out of a registered host table of [4 000 000, 512] fp16 rows, one call per batch and ten batches per
    call, and the layout-converting transfer of one block, direct and staged, on four shapes; next to them
    the block-table transfer of eight blocks in one launch, both directions, and the row gather out of a
    table in device memory. Every figure is printed only after its bytes were compared."""
    from heterofusedkernels_amd import reference_shapes_bench as R
    t0 = time.time()
    out = {"gather": [], "transfer": [], "rows": 4000000, "runs": 60}
    R.config1_latency(out, runs=200)
    R.gather_table(out["rows"], out["runs"], out, fill="bytes")
    R.gather_hbm_table(out)
    R.transfer_table(out)
    out["seconds"] = round(time.time() - t0, 1)
    out["how"] = ("gather: host wall time per call over %d calls, as pcieThrough/tests/test_gather.py:50-61; transfer: mean of "
                  "per-op HIP event times, as tests/test_transfer_kernel.py:51-52,86-88; table_in / table_out: 8 blocks "
                  "in one launch, one event pair around 5 launches" % out["runs"])
    return out


def section_hbm_ceiling(b, steps, warmup):
    """What HBM gives a kernel of the gather's shape (256-lane workgroups, one workgroup per chunk, 16-byte
    non-temporal accesses) that only reads, only writes, or copies 512 MiB of contiguous device memory.
    Moving N bytes takes at least N / read_rate + N / write_rate, so
    2 / (1 / read + 1 / write) bounds the traffic rate of any copy, the gather included."""
    torch = b.torch
    lib = ctypes.CDLL(b.build.HFK_BENCH_SO)
    lib.hfkb_hbm_stream.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int,
                                    ctypes.c_uint32, ctypes.c_int, ctypes.c_uint32, ctypes.c_void_p]
    nbytes = 1 << 29
    src = torch.full((nbytes,), 7, dtype=torch.uint8, device=b.dev)
    dst = torch.zeros(nbytes, dtype=torch.uint8, device=b.dev)
    out = {"bytes": nbytes, "how": "hbm_stream_kernel<mode, unroll, nt=3>, one workgroup per chunk of 4096 x unroll bytes; "
                                   "GB/s of HBM traffic (copy counts read + write)"}
    for unroll in (1, 8):
        row = {}
        for mode, name, mult in ((0, "read_only", 1), (1, "write_only", 1), (2, "copy", 2)):
            def launch():
                rc = lib.hfkb_hbm_stream(mode, dst.data_ptr(), src.data_ptr(), nbytes, unroll, 0, 1, 0, b.stream)
                assert rc == 0, rc
            _, ms = b.timed(launch, max(steps, 20), warmup)
            row[name + "_GBps"] = mult * nbytes / (ms * 1e6)
        row["copy_bound_from_read_and_write_GBps"] = 2.0 / (1.0 / row["read_only_GBps"] + 1.0 / row["write_only_GBps"])
        out["unroll_%d" % unroll] = row
        log("HBM yardsticks, %d vector(s) per lane: read-only %.0f, write-only %.0f, copy %.0f GB/s of traffic "
            "(a copy cannot pass %.0f)" % (unroll, row["read_only_GBps"], row["write_only_GBps"], row["copy_GBps"],
                                           row["copy_bound_from_read_and_write_GBps"]))
    assert bool((dst == 7).all()), "copy yardstick moved wrong bytes"
    del src, dst
    torch.cuda.empty_cache()
    return out


def section_memcpy_loop(b, w):
    np, torch, W, cfg = b.np, b.torch, b.W, w.cfg
    lib = ctypes.CDLL(b.build.HFK_BENCH_SO)
    lib.hfkb_memcpy_block_loop.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_uint32] + [ctypes.c_uint64] * 4 + [ctypes.c_void_p]
    dst_addrs = np.array([t.data_ptr() for t in w.host_planes], dtype=np.uint64)
    src_addrs = np.array([t.data_ptr() for t in w.dev_planes], dtype=np.uint64)
    pairs_np = np.ascontiguousarray(W.pairs_tensor(w.src_ids, w.dst_ids).numpy())
    bb = cfg.block_bytes

    def loop():
        rc = lib.hfkb_memcpy_block_loop(dst_addrs.ctypes.data, src_addrs.ctypes.data, pairs_np.ctypes.data, cfg.planes,
                                        cfg.n_blocks, bb, bb, bb, b.stream)
        assert rc == 0, rc

    loop()
    torch.cuda.synchronize()
    reps = 2
    t0 = time.perf_counter()
    for _ in range(reps):
        loop()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / reps
    log("per-block hipMemcpyAsync loop (%d calls): %.2f GB/s" % (cfg.planes * cfg.n_blocks, w.payload / dt / 1e9))
    return {"GBps": w.payload / dt / 1e9, "ms": dt * 1e3, "calls": cfg.planes * cfg.n_blocks}


def section_cpu_baseline(b, w):
    """The torch CPU path on this box's host cores (the oracle's torch statement, timed)."""
    torch, W, cfg = b.torch, b.W, w.cfg
    planes, n, bb = cfg.planes, cfg.n_blocks, cfg.block_bytes
    sample_planes = min(planes, 64)   # the whole block table where it fits: a few planes alone sit in the CPU's L3
    cpu_src = [w.dev_planes[p].cpu() for p in range(sample_planes)]
    if cfg.dtype == torch.float8_e4m3fn:      # CPU index ops on fp8 are not guaranteed: move its bytes
        cpu_src = [s.view(torch.uint8) for s in cpu_src]
    cpu_dst = [torch.zeros((cfg.host_blocks,) + tuple(cfg.block_shape), dtype=cpu_src[0].dtype) for _ in range(sample_planes)]

    from oracle import oracle as O      # the checker, timed here as the CPU baseline; never on the GPU path

    def cpu_pass():
        for s, d in zip(cpu_src, cpu_dst):
            O.torch_swap_blocks(d, s, w.src_ids, w.dst_ids)   # dst.index_copy_(0, dst_ids, src.index_select(0, src_ids))

    cpu_pass()
    for p in range(sample_planes):      # the baseline computes the same bytes the GPU produced
        assert torch.equal(W.as_bytes(cpu_dst[p]).index_select(0, w.dst_ids), W.as_bytes(cpu_src[p]).index_select(0, w.src_ids))
    passes, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < 10.0:
        cpu_pass()
        passes += 1
    dt = time.perf_counter() - t0
    cpu_gbps = passes * sample_planes * n * bb / dt / 1e9
    t1 = time.perf_counter()
    gpasses = 0
    while time.perf_counter() - t1 < 3.0:
        for s in cpu_src:
            O.torch_gather_rows(s, w.src_ids)
        gpasses += 1
    cpu_gather_gbps = gpasses * sample_planes * n * bb / (time.perf_counter() - t1) / 1e9
    # the C restatement of the same swap (one thread, memcpy per block), on the same planes, about 2 s of it
    src_np = [W.as_bytes(s).numpy().reshape(-1, bb) for s in cpu_src]
    dst_np = [W.as_bytes(d).numpy().reshape(-1, bb) for d in cpu_dst]
    pairs_np = W.pairs_tensor(w.src_ids, w.dst_ids).numpy()
    O.c_swap_blocks(dst_np, src_np, pairs_np)
    cpasses, t2 = 0, time.perf_counter()
    while time.perf_counter() - t2 < 2.0:
        O.c_swap_blocks(dst_np, src_np, pairs_np)
        cpasses += 1
    c_oracle_gbps = cpasses * sample_planes * n * bb / (time.perf_counter() - t2) / 1e9
    cpu_model = ""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    cpu_model = line.split(":", 1)[1].strip()
                    break
    except OSError:
        pass
    log("CPU baseline (torch, %d threads): swap %.2f GB/s, gather %.2f GB/s payload; the C restatement on one thread: "
        "swap %.2f GB/s" % (torch.get_num_threads(), cpu_gbps, cpu_gather_gbps, c_oracle_gbps))
    return {
        "value": cpu_gbps, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
        "sample": "torch CPU dst.index_copy_(0, dst_ids, src.index_select(0, src_ids)) per plane on %d of %d "
                  "planes of the same block table (%d blocks x %d B each), %d passes in %.1fs" %
                  (sample_planes, planes, n, bb, passes, dt),
        "gather_index_select_GBps": cpu_gather_gbps, "c_restatement_one_thread_GBps": c_oracle_gbps,
        "os_cpu_count": os.cpu_count(),
        "affinity": len(os.sched_getaffinity(0)), "cpu_model": cpu_model,
    }


def config_summary(w, extra=None):
    cfg = w.cfg
    out = {"workload": cfg.name, "planes": cfg.planes, "layers": cfg.layers, "block_bytes": cfg.block_bytes,
           "blocks_per_launch": cfg.n_blocks, "device_blocks": cfg.dev_blocks, "host_blocks": cfg.host_blocks,
           "host_blocks_specified": w.specified_host_blocks, "payload_bytes_per_step": w.payload,
           "cache_dtype": str(cfg.dtype).replace("torch.", "")}
    out.update(extra or {})
    return out


def measure_other_config(b, key, cfg, steps, warmup, d2h_peak, h2d_peak):
    """Swap-out, swap-in and gather of one further configuration, each verified on every plane."""
    capi = b.capi
    w = Workload(b, cfg, key)
    try:
        steps = max(3, min(steps, int(2.0e9 * steps / max(w.payload, 1)) or 3))   # about as many bytes as the headline config moves
        _, ms_out, _ = w.measure_swap_out(steps, min(warmup, 2), capi.SWAP_DST_HOST)
        _, ms_in, _ = w.measure_swap_in(steps, min(warmup, 2), capi.SWAP_SRC_HOST)
        ms_g, _ = w.measure_gather(steps, min(warmup, 2))
        out_gbps, in_gbps, g_gbps = rate(w.payload, ms_out), rate(w.payload, ms_in), rate(w.gather_alg_bytes, ms_g)
        return {
            "config": config_summary(w), "steps": steps,
            "swap_out": {"kernel_GBps": out_gbps, "avg_launch_ms": ms_out, "frac_of_pcie5_x16": frac(out_gbps, PCIE5_X16_GBPS),
                         "frac_of_measured_d2h": frac(out_gbps, d2h_peak)},
            "swap_in": {"kernel_GBps": in_gbps, "avg_launch_ms": ms_in, "frac_of_pcie5_x16": frac(in_gbps, PCIE5_X16_GBPS),
                        "frac_of_measured_h2d": frac(in_gbps, h2d_peak)},
            "gather": {"traffic_GBps": g_gbps, "avg_launch_ms": ms_g, "frac_of_hbm_peak": frac(g_gbps, HBM_PEAK_GBPS),
                       "algorithmic_bytes_per_launch": w.gather_alg_bytes, "launches_timed": w.gather_iters},
            "verified": "bit-exact on every plane: swap_out, swap_in, gather",
        }
    finally:
        w.release()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c2", choices=["c2", "c3", "c4", "c5"],
                    help="c2 (default) = Llama-3-8B swap-out, the configuration the metric is quoted on")
    ap.add_argument("--configs", default="c3,c4,c5",
                    help="further configurations measured after the headline one (swap-out, swap-in, gather each), "
                         "comma list of c2..c5, empty for none")
    ap.add_argument("--sections", default=",".join(ALL_SECTIONS),
                    help="comma list of the GPU sections to run on the headline workload; swap_out is the timed step and "
                         "always runs unless a profile of one other kernel alone is wanted")
    ap.add_argument("--tune", default="", help="comma list of library knobs for experiments, e.g. unroll=4,nt=0 "
                    "(unroll, nt, wg_per_cu, swap_wgs, swap_unroll, duplex_unroll, duplex_wgs, pace_mbps, link_mbps, "
                    "throughput_pace, hbm_lds, paced_unroll, paced_wgs, transfer_pace, transfer_tiled, duplex_pace); defaults are "
                    "the shipped ones")
    ap.add_argument("--out-flags", type=int, default=1, help="flags of the timed swap-out (default HFK_SWAP_DST_HOST = 1: "
                    "the caller knows its destination is host memory; 0 = say nothing)")
    ap.add_argument("--skip-cpu-baseline", action="store_true")
    ap.add_argument("--skip-memcpy-loop", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU; --gpus %d is not supported (every (plane, block) tile "
              "is independent, so N GPUs run N copies of this launch on their own caches)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    b = Bench(args)
    capi, W = b.capi, b.W
    knobs = {"unroll": capi.KNOB_UNROLL, "nt": capi.KNOB_NONTEMPORAL, "wg_per_cu": capi.KNOB_WORKGROUPS_PER_CU,
             "swap_wgs": capi.KNOB_SWAP_WORKGROUPS, "duplex_unroll": capi.KNOB_DUPLEX_UNROLL,
             "swap_unroll": capi.KNOB_SWAP_UNROLL, "pace_mbps": capi.KNOB_SWAP_PACE_MBPS, "link_mbps": capi.KNOB_LINK_MBPS,
             "duplex_wgs": capi.KNOB_DUPLEX_WORKGROUPS, "throughput_pace": capi.KNOB_THROUGHPUT_PACE_PERMILLE,
             "hbm_lds": capi.KNOB_HBM_LDS_BYTES, "paced_unroll": capi.KNOB_PACED_UNROLL,
             "paced_wgs": capi.KNOB_PACED_WORKGROUPS,
             "transfer_pace": capi.KNOB_TRANSFER_PACE_PERMILLE, "transfer_tiled": capi.KNOB_TRANSFER_TILED,
             "duplex_pace": capi.KNOB_DUPLEX_PACE_PERMILLE}
    tuned = {}
    for item in filter(None, args.tune.split(",")):
        key, val = item.split("=")
        capi.check(capi.set_tuning(knobs[key], int(val)), "hfk_set_tuning(%s)" % item)
        tuned[key] = int(val)
    by_key = {"c2": W.C2_LLAMA8B_SWAP_OUT, "c3": W.C3_LLAMA70B_SWAP_IN, "c4": W.C4_MLA_ROUNDTRIP, "c5": W.C5_FP8_FRAGMENTED}
    sections = set(x for x in args.sections.split(",") if x)
    assert sections <= set(ALL_SECTIONS), sections
    others = [k for k in args.configs.split(",") if k and k != args.workload]
    assert set(others) <= set(by_key), others

    w = Workload(b, by_key[args.workload], args.workload)
    cfg = w.cfg
    d2h_peak, h2d_peak, big = pcie_peaks(b, w.host_pools[0])

    # ---- the timed steps: swap-out -------------------------------------------
    value = ms_per_step = kernel_ms_out = spread_out = None
    if "swap_out" in sections:
        wall, kernel_ms_out, spread_out = w.measure_swap_out(args.steps, args.warmup, args.out_flags)
        value = args.steps * w.payload / wall / 1e9
        ms_per_step = wall * 1e3 / args.steps
    else:
        w.fill_host_slots()

    swap_in_gbps = kernel_ms_in = spread_in = None
    if "swap_in" in sections:
        wall_in, kernel_ms_in, spread_in = w.measure_swap_in(args.steps, args.warmup, capi.SWAP_SRC_HOST)
        swap_in_gbps = args.steps * w.payload / wall_in / 1e9

    kernel_ms_g = spread_gather = gather_traffic_gbps = gather_payload_gbps = torch_gather_gbps = gather_iters = None
    if "gather" in sections:
        kernel_ms_g, spread_gather = w.measure_gather(args.steps, args.warmup)
        gather_iters = w.gather_iters
        gather_traffic_gbps = w.gather_alg_bytes / (kernel_ms_g * 1e6)
        gather_payload_gbps = w.payload / (kernel_ms_g * 1e6)
        _, ms_t = b.timed(lambda: b.torch.index_select(w.dev_bytes[0], 0, w.ids_dev), args.steps, args.warmup)
        torch_gather_gbps = 2 * cfg.n_blocks * cfg.block_bytes / (ms_t * 1e6)
        log("torch.index_select on one plane: %.1f GB/s" % torch_gather_gbps)

    gather_orders = section_gather_orders(b, w, args.steps) if "gather_orders" in sections else None

    duplex = None
    if "duplex" in sections:
        duplex, _keep = section_duplex(b, w, args.steps, args.warmup)
        del _keep

    staged = beside = fragmented = None
    if "staged" in sections:
        staged, beside, fragmented = section_staged(b, w, args.steps, args.warmup, args.out_flags)

    # ---- plain device copy of known size: yardstick for reachable HBM bandwidth, and the
    # calibration row for the rocprofv3 FETCH_SIZE / WRITE_SIZE counters -----------------
    torch = b.torch
    cal_bytes = 1 << 29
    cal_a = torch.empty(cal_bytes, dtype=torch.uint8, device=b.dev)
    cal_b = torch.full((cal_bytes,), 7, dtype=torch.uint8, device=b.dev)
    _, ms_c = b.timed(lambda: cal_a.copy_(cal_b), args.steps, args.warmup)
    d2d_copy_gbps = 2 * cal_bytes / (ms_c * 1e6)
    del cal_a, cal_b
    log("torch device copy of %d MiB: %.1f GB/s of HBM traffic" % (cal_bytes >> 20, d2d_copy_gbps))

    hbm_ceiling = section_hbm_ceiling(b, args.steps, args.warmup) if "hbm_ceiling" in sections else None
    memcpy_loop = None if args.skip_memcpy_loop else section_memcpy_loop(b, w)
    cpu_baseline = None if args.skip_cpu_baseline else section_cpu_baseline(b, w)
    tables = section_tables(b, w, args.steps) if "tables" in sections else None
    repeat = section_repeat(b, w, args.steps, args.warmup, args.out_flags, value) if "repeat" in sections else None
    headline_config = config_summary(w, {"tuning_overrides": tuned})
    link_known = capi.get_tuning(capi.KNOB_LINK_MBPS) > 0
    gather_unroll = capi.get_tuning(capi.KNOB_UNROLL)
    paced_unroll, paced_wgs = capi.get_tuning(capi.KNOB_PACED_UNROLL), capi.get_tuning(capi.KNOB_PACED_WORKGROUPS)
    pace_permille = capi.get_tuning(capi.KNOB_THROUGHPUT_PACE_PERMILLE)
    w.release()

    # ---- the other configurations, one after the other --------------------------
    configs = {}
    for key in others:
        configs[key] = measure_other_config(b, key, by_key[key], args.steps, args.warmup, d2h_peak, h2d_peak)

    reference_ops = section_reference_ops(b) if "reference_ops" in sections else None

    # ---- HBM traffic measured offline with rocprofv3 --pmc, if recorded -------------
    traffic = {}
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            traffic = json.load(f).get(args.workload, {})
    except (OSError, ValueError):
        pass

    w_payload = headline_config["payload_bytes_per_step"]
    out_kernel_gbps = rate(w_payload, kernel_ms_out)
    in_kernel_gbps = rate(w_payload, kernel_ms_in)
    gather_alg_bytes = 2 * w_payload + 8 * headline_config["blocks_per_launch"]
    long_out = (args.out_flags & capi.SWAP_DST_HOST) and w_payload >= (64 << 20)
    paced = long_out and link_known and pace_permille > 0
    if paced:
        out_kernel = "swap_blocks_kernel<%d, 3>, %d workgroups, paced at 0.%d of the link" % (paced_unroll, paced_wgs, pace_permille // 10)
    elif long_out:
        out_kernel = "swap_blocks_kernel<8, 1>, 12 workgroups (non-temporal loads, plain stores), unpaced"
    else:
        out_kernel = "swap_blocks_kernel<8, 3>, 16 workgroups"
    result = {
        "metric": "KV swap GB/s (% of PCIe5 x16 peak); block gather GB/s (% of HBM peak)",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": headline_config,
        # Dominant kernel of the step. A swap never touches HBM twice; the resource it saturates is the
        # PCIe Gen5 x16 link, so that is the roofline it is priced against (theoretical link rate as
        # `peak`, the rate one large pinned hipMemcpyAsync reaches in this run as `peak_measured`).
        "roofline": {
            "kernel": out_kernel + " via hfk_swap_blocks (swap-out, HBM -> pinned host)", "bound": "pcie",
            "achieved": out_kernel_gbps, "peak": PCIE5_X16_GBPS, "unit": "GB/s",
            "frac": frac(out_kernel_gbps, PCIE5_X16_GBPS),
            "traffic": traffic.get("swap_out_hbm_bytes_per_launch"),
            "traffic_source": "profiles/hbm_traffic.json (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this launch, collected "
                              "in a run of its own; this run does not measure it)",
            "peak_measured": d2h_peak, "frac_of_measured": frac(out_kernel_gbps, d2h_peak),
            "algorithmic_bytes_per_launch": w_payload, "avg_launch_ms": kernel_ms_out,
        },
        # The HBM-bound kernel of the path: the multi-plane block gather on the same cache.
        "roofline_gather": {
            "kernel": "gather_blocks_kernel<%d, 3> via hfk_gather_blocks (HBM -> HBM)" % gather_unroll, "bound": "hbm",
            "achieved": gather_traffic_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": frac(gather_traffic_gbps, HBM_PEAK_GBPS), "traffic": traffic.get("gather_hbm_bytes_per_launch"),
            "algorithmic_bytes_per_launch": gather_alg_bytes, "avg_launch_ms": kernel_ms_g,
            "launches_timed": gather_iters, "payload_GBps": gather_payload_gbps, "torch_index_select_GBps": torch_gather_gbps,
            "torch_device_copy_GBps": d2d_copy_gbps, "launch_spread": spread_gather,
        },
        "swap_out": {"GBps": value, "kernel_GBps": out_kernel_gbps, "launch_spread": spread_out,
                     "pct_of_measured_d2h": None if out_kernel_gbps is None else 100 * out_kernel_gbps / d2h_peak,
                     "pct_of_pcie5_x16": None if out_kernel_gbps is None else 100 * out_kernel_gbps / PCIE5_X16_GBPS},
        "swap_in": {"GBps": swap_in_gbps, "kernel_GBps": in_kernel_gbps, "launch_spread": spread_in,
                    "pct_of_measured_h2d": None if in_kernel_gbps is None else 100 * in_kernel_gbps / h2d_peak,
                    "pct_of_pcie5_x16": None if in_kernel_gbps is None else 100 * in_kernel_gbps / PCIE5_X16_GBPS},
        "pcie_peak_measured": {"d2h_GBps": d2h_peak, "h2d_GBps": h2d_peak, "theoretical_GBps": PCIE5_X16_GBPS,
                               "how": "mean of 5 back-to-back hipMemcpyAsync of %d MiB pinned" % (big >> 20)},
        "configs": configs,
        "hbm_ceiling": hbm_ceiling,
        "duplex": duplex,
        "staged": staged,
        "fragmented_host_slots": fragmented,
        "swap_out_by_block_table": tables,
        "swap_out_repeat": repeat,
        "gather_by_order_of_work": gather_orders,
        "reference_ops": reference_ops,
        "beside_compute": beside,
        "memcpy_block_loop": memcpy_loop,
        "cpu_baseline": cpu_baseline,
        "verified": "bit-exact on every plane: " + ", ".join(sorted(sections - {"hbm_ceiling", "tables", "reference_ops"})),
    }
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
