#!/usr/bin/env python3
"""Benchmark of the pcieThrough hot path on one MI355X.

A *step* is one block-table swap-out launch of the Llama-3-8B-shaped configuration:
32 layers x {K,V} planes of [4096 blocks, 16, 8, 128] bf16 in HBM, 256 random distinct
source blocks -> 256 distinct slots of a pinned host cache of 8192 blocks per plane,
all 64 planes in one launch (512 MiB over the PCIe link per step). `value` is the
swap-out rate of the timed steps. The same run also measures, on the same cache,
swap-in, the multi-plane block gather (HBM -> HBM), the PCIe peak seen by one large
pinned hipMemcpyAsync in each direction, a per-block hipMemcpyAsync loop, and the
torch CPU index_select / index_copy_ path on the host cores (the reported CPU
baseline). Every number is printed only after the moved bytes were verified.

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


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="c2", choices=["c2", "c3", "c4", "c5"],
                    help="c2 (default) = Llama-3-8B swap-out, the configuration the metric is quoted on")
    ap.add_argument("--sections", default="swap_out,swap_in,gather,duplex,staged",
                    help="comma list of the GPU sections to run; swap_out is the timed step and always runs unless "
                         "a profile of one other kernel alone is wanted")
    ap.add_argument("--tune", default="", help="comma list of library knobs for experiments, e.g. unroll=4,nt=0 "
                    "(unroll, nt, wg_per_cu, swap_wgs, swap_unroll, duplex_unroll, pace_mbps, link_mbps); defaults are the shipped ones")
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

    import numpy as np
    import torch

    import heterofusedkernels_amd  # noqa: F401
    import pcie_through  # noqa: F401
    from heterofusedkernels import memory
    from heterofusedkernels_amd import _build, capi
    from heterofusedkernels_amd import workloads as W

    knobs = {"unroll": capi.KNOB_UNROLL, "nt": capi.KNOB_NONTEMPORAL, "wg_per_cu": capi.KNOB_WORKGROUPS_PER_CU,
             "swap_wgs": capi.KNOB_SWAP_WORKGROUPS, "duplex_unroll": capi.KNOB_DUPLEX_UNROLL,
             "swap_unroll": capi.KNOB_SWAP_UNROLL, "pace_mbps": capi.KNOB_SWAP_PACE_MBPS, "link_mbps": capi.KNOB_LINK_MBPS}
    tuned = {}
    for item in filter(None, args.tune.split(",")):
        key, val = item.split("=")
        capi.check(capi.set_tuning(knobs[key], int(val)), "hfk_set_tuning(%s)" % item)
        tuned[key] = int(val)
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")
    cfg = {"c2": W.C2_LLAMA8B_SWAP_OUT, "c3": W.C3_LLAMA70B_SWAP_IN, "c4": W.C4_MLA_ROUNDTRIP,
           "c5": W.C5_FP8_FRAGMENTED}[args.workload]
    sections = set(x for x in args.sections.split(",") if x)
    assert sections <= {"swap_out", "swap_in", "gather", "duplex", "staged"}, sections
    CONFIG_HOST_BLOCKS = cfg.host_blocks
    planes, bb, n = cfg.planes, cfg.block_bytes, cfg.n_blocks
    payload = cfg.payload_bytes
    stream = torch.cuda.current_stream().cuda_stream
    # Two extra streams for the sections that run things side by side. Created once, first: HIP maps
    # streams onto a few hardware queues round-robin, and two streams that share a queue do not overlap.
    stream_a, stream_b = torch.cuda.Stream(), torch.cuda.Stream()

    # ---- caches -------------------------------------------------------------
    t0 = time.time()
    dev_planes = [W.make_plane(cfg, l, kv, cfg.dev_blocks, device=dev) for l in range(cfg.layers)
                  for kv in range(cfg.kv)]
    torch.cuda.synchronize()
    log("device cache: %d planes x %d blocks x %d B = %.2f GiB (%.1fs)" %
        (planes, cfg.dev_blocks, bb, planes * cfg.dev_blocks * bb / 2**30, time.time() - t0))
    t0 = time.time()
    # Pinned host cache, in allocations of at most 8 GiB (one huge hipHostMalloc is refused on some
    # machines). If the machine will not pin the whole pool, the pool is halved and the run says so.
    host_blocks = cfg.host_blocks
    while True:
        plane_bytes = host_blocks * bb
        per_alloc = max(1, (8 << 30) // plane_bytes)
        host_pools, host_planes = [], []
        try:
            for first in range(0, planes, per_alloc):
                count = min(per_alloc, planes - first)
                pool = memory.alloc_numa_pinned_tensor(count * plane_bytes)
                host_pools.append(pool)
                host_planes.extend(pool.view(torch.uint8).view(count, host_blocks, bb).unbind(0))
            break
        except RuntimeError as exc:
            del host_pools, host_planes
            if host_blocks // 2 < 2 * n:
                raise
            log("could not pin %.1f GiB (%s); halving the host pool" % (planes * plane_bytes / 2**30, str(exc)[:80]))
            host_blocks //= 2
    if host_blocks != cfg.host_blocks:
        from dataclasses import replace
        cfg = replace(cfg, host_blocks=host_blocks)
    host_pool = host_pools[0]
    log("pinned host cache: %d blocks per plane = %.2f GiB in %d allocations (%.1fs, NUMA node %d)" %
        (cfg.host_blocks, planes * cfg.host_blocks * bb / 2**30, len(host_pools), time.time() - t0,
         memory.device_numa_node(0)))
    dev_bytes = [W.as_bytes(t) for t in dev_planes]           # uint8 views, same storage
    dev_tab = pcie_through.plane_pointer_table(dev_planes, dev)
    host_tab = pcie_through.plane_pointer_table(host_planes, dev)
    if args.workload == "c5":
        src_ids = W.fragmented_ids(cfg.dev_blocks, n)
        dst_ids = torch.arange(n)
    else:
        src_ids, dst_ids = W.block_table(cfg, src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
    pairs_out = W.pairs_tensor(src_ids, dst_ids).to(dev)      # device block -> host slot
    back_ids = torch.roll(src_ids, 1)                         # swap-in lands in other device slots
    prefill = torch.empty(planes, n, bb, dtype=torch.uint8, device=dev)
    prefill_tab = pcie_through.plane_pointer_table(list(prefill.unbind(0)), dev)
    ids_dev = src_ids.to(dev)

    def swap_out():
        capi.check(capi.swap_blocks(host_tab.data_ptr(), dev_tab.data_ptr(), pairs_out.data_ptr(), planes, n, bb, bb,
                                    bb, cfg.dev_blocks, cfg.host_blocks, 0, stream, args.out_flags), "hfk_swap_blocks(out)")

    def gather():
        capi.check(capi.gather_blocks(prefill_tab.data_ptr(), dev_tab.data_ptr(), ids_dev.data_ptr(), planes, n, bb, bb,
                                      cfg.dev_blocks, 0, stream), "hfk_gather_blocks")

    def timed(fn, iters, warm):
        """Runs `warm` untimed calls, then `iters` calls back to back between two synchronizes.
        Returns (wall seconds for the iters calls, average milliseconds per call from one HIP event
        pair recorded on the launch stream around the whole batch, so that launch gaps of short
        kernels are hidden by the queue exactly as in steady-state use)."""
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

    def launch_spread(fn, iters):
        """The same launch timed one at a time (an event pair per launch, a synchronize between launches):
        the first call of the process (module load and first-touch included, by the host clock), then
        median / min / max of `iters` isolated launches by HIP events."""
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

    # ---- PCIe peak as one large pinned copy sees it --------------------------
    big = min(1 << 30, host_pool.numel())
    big_d = torch.empty(big, dtype=torch.int8, device=dev)
    big_h = host_pool[:big]
    _, ms = timed(lambda: big_h.copy_(big_d, non_blocking=True), 5, 2)
    d2h_peak = big / (ms * 1e6)
    _, ms = timed(lambda: big_d.copy_(big_h, non_blocking=True), 5, 2)
    h2d_peak = big / (ms * 1e6)
    host_pool[:big].zero_()
    del big_d
    log("hipMemcpyAsync %d MiB pinned: D2H %.2f GB/s, H2D %.2f GB/s (link %.1f GB/s theoretical)" %
        (big >> 20, d2h_peak, h2d_peak, PCIE5_X16_GBPS))

    # ---- the timed steps: swap-out -------------------------------------------
    value = ms_per_step = kernel_ms_out = None
    spread_out = spread_in = spread_gather = None
    if "swap_out" in sections:
        spread_out = launch_spread(swap_out, min(args.steps, 10))
        wall, kernel_ms_out = timed(swap_out, args.steps, args.warmup)
        value = args.steps * payload / wall / 1e9
        ms_per_step = wall * 1e3 / args.steps
        log("swap-out: %.2f GB/s whole-job (%.3f ms/step wall, %.3f ms/launch by events)" %
            (value, ms_per_step, kernel_ms_out))
        # verify: host slots == device source blocks read back by an independent path (torch index + D2H copy)
        t0 = time.time()
        for p in range(planes):
            want = dev_bytes[p].index_select(0, ids_dev).cpu()
            assert torch.equal(host_planes[p].index_select(0, dst_ids), want), "swap-out mismatch in plane %d" % p
        untouched = torch.ones(cfg.host_blocks, dtype=torch.bool)
        untouched[dst_ids] = False
        for p in (0, planes // 2, planes - 1):
            assert int(host_planes[p][untouched].max()) == 0, "swap-out wrote outside its slots (plane %d)" % p
        log("swap-out verified bit-exact on all %d planes (%.1fs)" % (planes, time.time() - t0))
    else:   # later sections still need the host slots filled: do it with plain torch copies
        for p in range(planes):
            host_planes[p][dst_ids] = dev_bytes[p].index_select(0, ids_dev).cpu()

    # ---- swap-in (host slots -> other device slots) -----------------------------
    pairs_in = W.pairs_tensor(dst_ids, back_ids).to(dev)

    def swap_in():
        capi.check(capi.swap_blocks(dev_tab.data_ptr(), host_tab.data_ptr(), pairs_in.data_ptr(), planes, n, bb, bb, bb,
                                    cfg.host_blocks, cfg.dev_blocks, 0, stream, capi.SWAP_SRC_HOST), "hfk_swap_blocks(in)")

    swap_in_gbps = kernel_ms_in = None
    if "swap_in" in sections:
        expect_in = {p: host_planes[p].index_select(0, dst_ids).clone() for p in range(planes)}
        spread_in = launch_spread(swap_in, min(args.steps, 10))
        wall_in, kernel_ms_in = timed(swap_in, args.steps, args.warmup)
        for p in range(planes):
            got = dev_bytes[p].index_select(0, back_ids.to(dev)).cpu()
            assert torch.equal(got, expect_in[p]), "swap-in mismatch in plane %d" % p
        del expect_in
        swap_in_gbps = args.steps * payload / wall_in / 1e9
        log("swap-in: %.2f GB/s (%.3f ms/launch), verified" % (swap_in_gbps, kernel_ms_in))

    # ---- block gather, HBM -> HBM ------------------------------------------------
    gather_alg_bytes = 2 * payload + 8 * n             # read + write + the id list
    kernel_ms_g = gather_traffic_gbps = gather_payload_gbps = torch_gather_gbps = None
    if "gather" in sections:
        spread_gather = launch_spread(gather, min(args.steps, 10))
        wall_g, kernel_ms_g = timed(gather, args.steps, args.warmup)
        for p in range(planes):
            assert torch.equal(prefill[p], dev_bytes[p].index_select(0, ids_dev)), "gather mismatch %d" % p
        gather_traffic_gbps = gather_alg_bytes / (kernel_ms_g * 1e6)
        gather_payload_gbps = payload / (kernel_ms_g * 1e6)
        _, ms_t = timed(lambda: torch.index_select(dev_bytes[0], 0, ids_dev), args.steps, args.warmup)
        torch_gather_gbps = 2 * n * bb / (ms_t * 1e6)
        log("gather: %.1f GB/s of HBM traffic (%.1f payload GB/s, %.3f ms/launch), verified; torch.index_select on one "
            "plane: %.1f GB/s" % (gather_traffic_gbps, gather_payload_gbps, kernel_ms_g, torch_gather_gbps))

    # ---- both directions at once on two streams (the link is full duplex) -------------
    duplex = None
    if "duplex" in sections:
        gen = torch.Generator().manual_seed(cfg.base_seed + 77)
        free_dev = torch.ones(cfg.dev_blocks, dtype=torch.bool)
        free_dev[src_ids] = False
        free_dev[back_ids] = False
        free_host = torch.ones(cfg.host_blocks, dtype=torch.bool)
        free_host[dst_ids] = False
        dev_free, host_free = free_dev.nonzero().flatten(), free_host.nonzero().flatten()
        n2 = min(n, dev_free.numel(), host_free.numel())
        in_dev = dev_free[torch.randperm(dev_free.numel(), generator=gen)[:n2]]      # disjoint from the swap-out's blocks
        in_host = host_free[torch.randperm(host_free.numel(), generator=gen)[:n2]]
        for p in range(planes):                                                      # give the host slots known content
            host_planes[p][in_host] = dev_bytes[p].index_select(0, ids_dev[:n2]).cpu()
        pairs_in2 = W.pairs_tensor(in_host, in_dev).to(dev)
        s_out, s_in = stream_a, stream_b

        def both():
            with torch.cuda.stream(s_out):
                capi.check(capi.swap_blocks(host_tab.data_ptr(), dev_tab.data_ptr(), pairs_out.data_ptr(), planes, n, bb,
                                            bb, bb, cfg.dev_blocks, cfg.host_blocks, 0, s_out.cuda_stream))
            with torch.cuda.stream(s_in):
                capi.check(capi.swap_blocks(dev_tab.data_ptr(), host_tab.data_ptr(), pairs_in2.data_ptr(), planes, n2, bb,
                                            bb, bb, cfg.host_blocks, cfg.dev_blocks, 0, s_in.cuda_stream))

        both()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            both()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        for p in range(planes):
            assert torch.equal(host_planes[p].index_select(0, dst_ids), dev_bytes[p].index_select(0, ids_dev).cpu())
            assert torch.equal(dev_bytes[p].index_select(0, in_dev.to(dev)).cpu(), host_planes[p].index_select(0, in_host))
        total = args.steps * (n + n2) * planes * bb
        # ... and the same two block tables in ONE duplex launch
        om = capi.BlockMove(host_tab.data_ptr(), dev_tab.data_ptr(), pairs_out.data_ptr(), n, bb, bb, cfg.dev_blocks,
                            cfg.host_blocks)
        im = capi.BlockMove(dev_tab.data_ptr(), host_tab.data_ptr(), pairs_in2.data_ptr(), n2, bb, bb, cfg.host_blocks,
                            cfg.dev_blocks)
        for p in range(planes):                                          # make the launch prove itself: clear the targets
            host_planes[p][dst_ids] = 0
            dev_bytes[p].index_fill_(0, in_dev.to(dev), 0)

        def one_launch():
            capi.check(capi.swap_blocks_duplex(om, im, planes, bb, 0, stream), "hfk_swap_blocks_duplex")

        wall_d, ms_d = timed(one_launch, args.steps, args.warmup)
        for p in range(planes):
            assert torch.equal(host_planes[p].index_select(0, dst_ids), dev_bytes[p].index_select(0, ids_dev).cpu())
            assert torch.equal(dev_bytes[p].index_select(0, in_dev.to(dev)).cpu(), host_planes[p].index_select(0, in_host))
        duplex_kernel_gbps = (n + n2) * planes * bb / (ms_d * 1e6)
        # the copy engines doing the same thing: two opposite 512 MiB pinned copies on the two streams
        half = min(1 << 29, host_pool.numel() // 2)
        d_a = torch.empty(half, dtype=torch.int8, device=dev)
        d_b = torch.empty(half, dtype=torch.int8, device=dev)
        h_a, h_b = host_pool[-half:], host_pool[-2 * half:-half]
        keep = h_b.clone()                       # these bytes belong to the host cache: put them back afterwards

        def both_memcpy():
            with torch.cuda.stream(s_out):
                h_a.copy_(d_a, non_blocking=True)
            with torch.cuda.stream(s_in):
                d_b.copy_(h_b, non_blocking=True)

        keep_a = h_a.clone()
        both_memcpy()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(5):
            both_memcpy()
        torch.cuda.synchronize()
        dt_m = time.perf_counter() - t0
        h_a.copy_(keep_a)
        h_b.copy_(keep)
        del d_a, d_b, keep, keep_a
        duplex = {"one_launch_GBps_both_directions": duplex_kernel_gbps,
                  "one_launch_pct_of_2x_pcie5_x16": 100 * duplex_kernel_gbps / (2 * PCIE5_X16_GBPS),
                  "two_launches_two_streams_GBps_both_directions": total / dt / 1e9, "out_blocks": n, "in_blocks": n2,
                  "memcpy_both_directions_GBps": 5 * 2 * half / dt_m / 1e9}
        log("duplex, verified: swap_blocks_duplex (one launch) %.2f GB/s summed; swap-out + swap-in on two streams "
            "%.2f GB/s summed; two opposite hipMemcpyAsync %.2f GB/s summed" %
            (duplex_kernel_gbps, total / dt / 1e9, duplex["memcpy_both_directions_GBps"]))

    # ---- staged swap (gather kernel on HBM + DMA copies) and what each path costs a kernel beside it ----
    staged = beside = None
    if "staged" in sections:
        run_start = 0          # the earlier sections' results are verified by now: their host slots may be reused
        host_run = torch.arange(run_start, run_start + n)
        host_addrs = torch.tensor([t.data_ptr() for t in host_planes], dtype=torch.int64)
        staging_buf = torch.empty(planes, n, bb, dtype=torch.uint8, device=dev)

        def staged_out(st=None):
            capi.check(capi.swap_blocks_staged(dev_tab.data_ptr(), host_addrs.data_ptr(), ids_dev.data_ptr(),
                                               host_run.data_ptr(), planes, n, bb, bb, bb, cfg.dev_blocks,
                                               cfg.host_blocks, staging_buf.data_ptr(), True, 0,
                                               stream if st is None else st), "hfk_swap_blocks_staged(out)")

        back_dev = back_ids.to(dev)

        def staged_in():
            capi.check(capi.swap_blocks_staged(dev_tab.data_ptr(), host_addrs.data_ptr(), back_dev.data_ptr(),
                                               host_run.data_ptr(), planes, n, bb, bb, bb, cfg.dev_blocks,
                                               cfg.host_blocks, staging_buf.data_ptr(), False, 0, stream),
                       "hfk_swap_blocks_staged(in)")

        _, ms_so = timed(staged_out, args.steps, args.warmup)
        for p in range(planes):
            assert torch.equal(host_planes[p][run_start:run_start + n], dev_bytes[p].index_select(0, ids_dev).cpu())
        _, ms_si = timed(staged_in, args.steps, args.warmup)
        for p in range(planes):
            assert torch.equal(dev_bytes[p].index_select(0, back_dev).cpu(), host_planes[p][run_start:run_start + n])
        # both directions at once on two streams (two DMA engines); disjoint device blocks and host runs
        staging_b = torch.empty(planes, n, bb, dtype=torch.uint8, device=dev)
        run_b = torch.arange(run_start + n, run_start + 2 * n)

        def staged_both():
            capi.check(capi.swap_blocks_staged(dev_tab.data_ptr(), host_addrs.data_ptr(), ids_dev.data_ptr(),
                                               host_run.data_ptr(), planes, n, bb, bb, bb, cfg.dev_blocks,
                                               cfg.host_blocks, staging_buf.data_ptr(), True, 0, stream_a.cuda_stream))
            capi.check(capi.swap_blocks_staged(dev_tab.data_ptr(), host_addrs.data_ptr(), back_dev.data_ptr(),
                                               run_b.data_ptr(), planes, n, bb, bb, bb, cfg.dev_blocks,
                                               cfg.host_blocks, staging_b.data_ptr(), False, 0, stream_b.cuda_stream))

        staged_both()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            staged_both()
        torch.cuda.synchronize()
        staged_duplex_gbps = args.steps * 2 * payload / (time.perf_counter() - t0) / 1e9
        del staging_b
        # kernels on another stream: alone, and beside each way of swapping. Three neighbours: a compute-bound
        # GEMM, an HBM-bound 1 GiB device copy and an attention kernel (mixed).
        side, comp = stream_a, stream_b
        ga = torch.randn(8192, 8192, device=dev, dtype=torch.bfloat16)
        gb = torch.randn(8192, 8192, device=dev, dtype=torch.bfloat16)
        ca = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        cb = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
        qkv = torch.randn(8, 32, 2048, 128, device=dev, dtype=torch.bfloat16)
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

        beside_out_flags = capi.SWAP_DST_HOST | capi.SWAP_BESIDE_COMPUTE
        beside_in_flags = capi.SWAP_SRC_HOST | capi.SWAP_BESIDE_COMPUTE

        def direct(direction, flags):
            def call(st):
                if direction == "out":
                    capi.check(capi.swap_blocks(host_tab.data_ptr(), dev_tab.data_ptr(), pairs_out.data_ptr(), planes, n, bb,
                                                bb, bb, cfg.dev_blocks, cfg.host_blocks, 0, st, flags), "hfk_swap_blocks(out)")
                else:
                    capi.check(capi.swap_blocks(dev_tab.data_ptr(), host_tab.data_ptr(), pairs_in.data_ptr(), planes, n, bb,
                                                bb, bb, cfg.host_blocks, cfg.dev_blocks, 0, st, flags), "hfk_swap_blocks(in)")
            return call

        def staged_in_on(st):
            capi.check(capi.swap_blocks_staged(dev_tab.data_ptr(), host_addrs.data_ptr(), back_dev.data_ptr(),
                                               host_run.data_ptr(), planes, n, bb, bb, bb, cfg.dev_blocks,
                                               cfg.host_blocks, staging_buf.data_ptr(), False, 0, st),
                       "hfk_swap_blocks_staged(in)")

        ways = {"throughput_out": direct("out", args.out_flags), "throughput_in": direct("in", capi.SWAP_SRC_HOST),
                "beside_compute_out": direct("out", beside_out_flags), "beside_compute_in": direct("in", beside_in_flags),
                "staged_out": staged_out, "staged_in": staged_in_on}
        # own rate of the beside-compute launch shape, GPU otherwise idle; result checked like the plain swap-out's
        for p_ in range(planes):
            host_planes[p_][dst_ids] = 0
        _, ms_bo = timed(lambda: ways["beside_compute_out"](stream), args.steps, args.warmup)
        for p_ in range(planes):
            assert torch.equal(host_planes[p_].index_select(0, dst_ids), dev_bytes[p_].index_select(0, ids_dev).cpu()), \
                "beside-compute swap-out mismatch in plane %d" % p_
        _, ms_bi = timed(lambda: ways["beside_compute_in"](stream), args.steps, args.warmup)
        for p_ in range(planes):
            assert torch.equal(dev_bytes[p_].index_select(0, back_dev).cpu(), host_planes[p_].index_select(0, dst_ids)), \
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
        staged = {"swap_out_GBps": payload / (ms_so * 1e6), "swap_in_GBps": payload / (ms_si * 1e6),
                  "out_and_in_on_two_streams_GBps": staged_duplex_gbps,
                  "host_slots": "one run of %d consecutive slots per plane (%.1f MiB per plane, 2-D DMA copies over "
                                "evenly spaced planes)" % (n, n * bb / 2**20)}
        beside = {"swap_out_GBps": payload / (ms_bo * 1e6), "swap_in_GBps": payload / (ms_bi * 1e6),
                  "link_MBps_from_sysfs": capi.get_tuning(capi.KNOB_LINK_MBPS),
                  "neighbour_ms_alone": alone,
                  "neighbour_slowdown": slowdown,
                  "how": "each neighbour runs %s times on one stream while %d swaps of %d MiB are queued on another; "
                         "x = its time per call / its time alone; null = the swaps ended first" %
                         ("/".join(str(r) for _, r in neighbours.values()), side_reps, payload >> 20)}
        log("staged swap, verified: out %.2f GB/s, in %.2f GB/s, both on two streams %.2f GB/s summed" %
            (staged["swap_out_GBps"], staged["swap_in_GBps"], staged_duplex_gbps))
        log("swap with HFK_SWAP_BESIDE_COMPUTE, verified: out %.2f GB/s, in %.2f GB/s" % (beside["swap_out_GBps"], beside["swap_in_GBps"]))
        for way in ways:
            log("  neighbours beside %-19s %s" % (way + ":", ", ".join("%s x%s" % (k.split("_")[0], v) for k, v in slowdown[way].items())))

    # ---- plain device copy of known size: yardstick for reachable HBM bandwidth, and the
    # calibration row for the rocprofv3 FETCH_SIZE / WRITE_SIZE counters -----------------
    cal_bytes = 1 << 29
    cal_a = torch.empty(cal_bytes, dtype=torch.uint8, device=dev)
    cal_b = torch.full((cal_bytes,), 7, dtype=torch.uint8, device=dev)
    _, ms_c = timed(lambda: cal_a.copy_(cal_b), args.steps, args.warmup)
    d2d_copy_gbps = 2 * cal_bytes / (ms_c * 1e6)
    del cal_a, cal_b
    log("torch device copy of %d MiB: %.1f GB/s of HBM traffic" % (cal_bytes >> 20, d2d_copy_gbps))

    # ---- per-block hipMemcpyAsync loop ---------------------------------------------
    memcpy_loop = None
    if not args.skip_memcpy_loop:
        lib = ctypes.CDLL(_build.HFK_BENCH_SO)
        lib.hfkb_memcpy_block_loop.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_uint32] + [ctypes.c_uint64] * 4 + [
            ctypes.c_void_p]
        dst_addrs = np.array([t.data_ptr() for t in host_planes], dtype=np.uint64)
        src_addrs = np.array([t.data_ptr() for t in dev_planes], dtype=np.uint64)
        pairs_np = np.ascontiguousarray(W.pairs_tensor(src_ids, dst_ids).numpy())

        def loop():
            rc = lib.hfkb_memcpy_block_loop(dst_addrs.ctypes.data, src_addrs.ctypes.data, pairs_np.ctypes.data, planes,
                                            n, bb, bb, bb, stream)
            assert rc == 0, rc

        loop()
        torch.cuda.synchronize()
        reps = 2
        t0 = time.perf_counter()
        for _ in range(reps):
            loop()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / reps
        memcpy_loop = {"GBps": payload / dt / 1e9, "ms": dt * 1e3, "calls": planes * n}
        log("per-block hipMemcpyAsync loop (%d calls): %.2f GB/s" % (planes * n, memcpy_loop["GBps"]))

    # ---- CPU baseline: the torch CPU path on this box's host cores ----------------
    cpu_baseline = None
    if not args.skip_cpu_baseline:
        sample_planes = min(planes, 64)   # the whole block table where it fits: a few planes alone sit in the CPU's L3
        cpu_src = [dev_planes[p].cpu() for p in range(sample_planes)]
        if cfg.dtype == torch.float8_e4m3fn:      # CPU index ops on fp8 are not guaranteed: move its bytes
            cpu_src = [s.view(torch.uint8) for s in cpu_src]
        cpu_dst = [torch.zeros((cfg.host_blocks,) + tuple(cfg.block_shape), dtype=cpu_src[0].dtype)
                   for _ in range(sample_planes)]

        from oracle import oracle as O      # the checker, timed here as the CPU baseline; never on the GPU path

        def cpu_pass():
            for s, d in zip(cpu_src, cpu_dst):
                O.torch_swap_blocks(d, s, src_ids, dst_ids)   # dst.index_copy_(0, dst_ids, src.index_select(0, src_ids))

        cpu_pass()
        for p in range(sample_planes):      # the baseline computes the same bytes the GPU produced
            assert torch.equal(W.as_bytes(cpu_dst[p]).index_select(0, dst_ids),
                               W.as_bytes(cpu_src[p]).index_select(0, src_ids))
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
                O.torch_gather_rows(s, src_ids)
            gpasses += 1
        cpu_gather_gbps = gpasses * sample_planes * n * bb / (time.perf_counter() - t1) / 1e9
        cpu_model = ""
        try:
            with open("/proc/cpuinfo") as f:
                for line in f:
                    if line.startswith("model name"):
                        cpu_model = line.split(":", 1)[1].strip()
                        break
        except OSError:
            pass
        cpu_baseline = {
            "value": cpu_gbps, "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "torch CPU dst.index_copy_(0, dst_ids, src.index_select(0, src_ids)) per plane on %d of %d "
                      "planes of the same block table (%d blocks x %d B each), %d passes in %.1fs" %
                      (sample_planes, planes, n, bb, passes, dt),
            "gather_index_select_GBps": cpu_gather_gbps, "os_cpu_count": os.cpu_count(),
            "affinity": len(os.sched_getaffinity(0)), "cpu_model": cpu_model,
        }
        log("CPU baseline (torch, %d threads): swap %.2f GB/s, gather %.2f GB/s payload" %
            (torch.get_num_threads(), cpu_gbps, cpu_gather_gbps))

    # ---- HBM traffic measured offline with rocprofv3 --pmc, if recorded -------------
    traffic = {}
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            traffic = json.load(f).get(args.workload, {})
    except (OSError, ValueError):
        pass

    def rate(nbytes, ms):
        return None if ms is None else nbytes / (ms * 1e6)

    def frac(x, peak):
        return None if x is None else x / peak

    out_kernel_gbps = rate(payload, kernel_ms_out)
    in_kernel_gbps = rate(payload, kernel_ms_in)
    result = {
        "metric": "KV swap GB/s (% of PCIe5 x16 peak); block gather GB/s (% of HBM peak)",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": cfg.name, "planes": planes, "layers": cfg.layers, "block_bytes": bb,
                   "blocks_per_launch": n, "device_blocks": cfg.dev_blocks, "host_blocks": cfg.host_blocks,
                   "host_blocks_specified": CONFIG_HOST_BLOCKS,
                   "payload_bytes_per_step": payload, "cache_dtype": str(cfg.dtype).replace("torch.", ""),
                   "tuning_overrides": tuned},
        # Dominant kernel of the step. A swap never touches HBM twice; the resource it saturates is the
        # PCIe Gen5 x16 link, so that is the roofline it is priced against (theoretical link rate as
        # `peak`, the rate one large pinned hipMemcpyAsync reaches in this run as `peak_measured`).
        "roofline": {
            "kernel": ("swap_blocks_kernel<4, 3>, paced" if (args.out_flags & capi.SWAP_DST_HOST) and capi.get_tuning(capi.KNOB_LINK_MBPS) > 0
                       else "swap_blocks_kernel<8, 3>") + " via hfk_swap_blocks (swap-out, HBM -> pinned host)", "bound": "pcie",
            "achieved": out_kernel_gbps, "peak": PCIE5_X16_GBPS, "unit": "GB/s",
            "frac": frac(out_kernel_gbps, PCIE5_X16_GBPS),
            "traffic": traffic.get("swap_out_hbm_bytes_per_launch"),
            "peak_measured": d2h_peak, "frac_of_measured": frac(out_kernel_gbps, d2h_peak),
            "algorithmic_bytes_per_launch": payload, "avg_launch_ms": kernel_ms_out,
        },
        # The HBM-bound kernel of the path: the multi-plane block gather on the same cache.
        "roofline_gather": {
            "kernel": "gather_blocks_kernel<8, 3> via hfk_gather_blocks (HBM -> HBM)", "bound": "hbm",
            "achieved": gather_traffic_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": frac(gather_traffic_gbps, HBM_PEAK_GBPS), "traffic": traffic.get("gather_hbm_bytes_per_launch"),
            "algorithmic_bytes_per_launch": gather_alg_bytes, "avg_launch_ms": kernel_ms_g,
            "payload_GBps": gather_payload_gbps, "torch_index_select_GBps": torch_gather_gbps,
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
        "duplex": duplex,
        "staged": staged,
        "beside_compute": beside,
        "memcpy_block_loop": memcpy_loop,
        "cpu_baseline": cpu_baseline,
        "verified": "bit-exact on every plane: " + ", ".join(sorted(sections)),
    }
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
