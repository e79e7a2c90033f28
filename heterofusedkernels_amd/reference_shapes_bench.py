"""Re-runs the reference's own two benchmark tables (pcieThrough/tests/README.md) on MI355X.

* Embedding-row gather from a host-registered table, fp16 rows of 512 elements (1 KiB),
  batch sizes 16 ... 1024, one call per batch and "combined" (10 batches per call), timed
  end to end on the host like pcieThrough/tests/test_gather.py:50-61 and
  test_gather_combine.py:50-61; next to it the torch CPU index + H2D copy baseline of
  pcieThrough/tests/test_memcpy.py:18-27.
* One KV block [blockSize, layers, heads, headdim] int8, host -> per-layer device buffers
  with layout conversion, direct and staged, per-op event time like
  pcieThrough/tests/test_transfer_kernel.py:51-52,86-88.

Results are verified (seeded random data, byte compare) before they are printed.
Usage: python -m heterofusedkernels_amd.reference_shapes_bench [--rows N] [--runs N]
"""
import argparse
import json
import sys
import time

import torch

import heterofusedkernels_amd  # noqa: F401
import pcie_through  # noqa: F401
from heterofusedkernels import memory


PCIE5_X16_GBPS = 32.0 * 16 * (128.0 / 130.0) / 8.0


def gather_table(rows, runs, out, batch_sizes=(16, 32, 64, 128, 256, 512, 1024), fill="randn"):
    """fill: "randn" = N(0,1) rows like the reference's test; "bytes" = random 16-bit patterns, which fill
    a 4 GiB table in seconds (rows are compared as bytes either way)."""
    dev = "cuda"
    dim = 512
    embed = memory.alloc_numa_pinned_tensor(rows * dim * 2).view(torch.float16).view(rows, dim)
    gen = torch.Generator().manual_seed(0)
    chunk = 1 << 16
    for r0 in range(0, rows, chunk):        # every row distinct and non-zero
        r1 = min(rows, r0 + chunk)
        if fill == "randn":
            embed[r0:r1] = torch.randn(r1 - r0, dim, generator=gen).to(torch.float16)
        else:
            embed[r0:r1].view(torch.int16).random_(1, 32767, generator=gen)
    for bs in batch_sizes:
        row = {"bs": bs}
        # torch CPU advanced index + H2D copy (tests/test_memcpy.py:18,23)
        ids = torch.randint(0, rows, (runs, bs), dtype=torch.int64, generator=gen)
        for i in range(3):
            embed[ids[i % runs]].to(dev)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        cpu_runs = min(runs, 50)
        for i in range(cpu_runs):
            x = embed[ids[i]].to(dev)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / cpu_runs
        row["torch_cpu_index_h2d_ms"] = dt * 1e3
        row["torch_cpu_index_h2d_GBps"] = bs * dim * 2 / dt / 1e9
        # one call per batch
        ids_dev = ids.to(dev)
        dst = torch.empty(bs, dim, dtype=torch.float16, device=dev)
        for i in range(10):
            torch.ops.pcie_through.gather(embed, dst, ids_dev[i % runs], aiv=4)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(runs):
            torch.ops.pcie_through.gather(embed, dst, ids_dev[i], aiv=4)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / runs
        assert torch.equal(dst.cpu().view(torch.int16), embed[ids[runs - 1]].view(torch.int16)), "gather mismatch"
        row["gather_ms"] = dt * 1e3
        row["gather_GBps"] = bs * dim * 2 / dt / 1e9
        # combined: 10 batches in one call, default aiv (tests/test_gather_combine.py:47-56)
        ids10 = torch.randint(0, rows, (runs, bs * 10), dtype=torch.int64, generator=gen)
        ids10_dev = ids10.to(dev)
        dst10 = torch.empty(bs * 10, dim, dtype=torch.float16, device=dev)
        for i in range(10):
            torch.ops.pcie_through.gather(embed, dst10, ids10_dev[i % runs])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(runs):
            torch.ops.pcie_through.gather(embed, dst10, ids10_dev[i])
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / runs
        assert torch.equal(dst10.cpu().view(torch.int16), embed[ids10[runs - 1]].view(torch.int16)), "gather mismatch"
        row["gather_combined_ms_per_batch"] = dt * 1e3 / 10
        row["gather_combined_GBps"] = bs * 10 * dim * 2 / dt / 1e9
        row["gather_combined_frac_of_pcie5_x16"] = row["gather_combined_GBps"] / PCIE5_X16_GBPS
        out["gather"].append(row)
        print("gather bs=%4d: cpu+h2d %.3f ms (%.2f GB/s) | gather %.4f ms (%.2f GB/s) | combined %.4f ms/batch "
              "(%.2f GB/s)" % (bs, row["torch_cpu_index_h2d_ms"], row["torch_cpu_index_h2d_GBps"], row["gather_ms"],
                               row["gather_GBps"], row["gather_combined_ms_per_batch"], row["gather_combined_GBps"]),
              file=sys.stderr, flush=True)


def gather_hbm_table(out, rows=1 << 20, n_ids=1 << 18, launches=50):
    """The same row gather with the table in device memory: [rows, 512] fp16, n_ids random rows per call,
    timed by one HIP event pair around `launches` calls; GB/s of HBM traffic (rows read + rows written + ids)."""
    dev = "cuda"
    dim = 512
    gen = torch.Generator().manual_seed(1)
    table = torch.randint(1, 32767, (rows, dim), dtype=torch.int16, device=dev).view(torch.float16)
    ids = torch.randint(0, rows, (n_ids,), dtype=torch.int64, generator=gen).to(dev)
    dst = torch.empty(n_ids, dim, dtype=torch.float16, device=dev)
    for _ in range(3):
        torch.ops.pcie_through.gather(table, dst, ids)
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    s.record()
    for _ in range(launches):
        torch.ops.pcie_through.gather(table, dst, ids)
    e.record()
    torch.cuda.synchronize()
    ms = s.elapsed_time(e) / launches
    assert torch.equal(dst.view(torch.int16), table.view(torch.int16).index_select(0, ids)), "gather mismatch"
    traffic = 2 * n_ids * dim * 2 + 8 * n_ids
    out["gather_hbm_table"] = {"rows": rows, "ids_per_call": n_ids, "row_bytes": dim * 2, "ms": ms,
                               "traffic_GBps": traffic / (ms * 1e6), "frac_of_hbm_peak": traffic / (ms * 1e6) / 8000.0}
    print("gather from an HBM table [%d, %d] fp16, %d ids per call: %.4f ms, %.0f GB/s of HBM traffic" %
          (rows, dim, n_ids, ms, traffic / (ms * 1e6)), file=sys.stderr, flush=True)


README_TRANSFER_SHAPES = ((1024, 32, 1, 128), (1024, 32, 8, 128), (1024, 64, 1, 128), (1024, 64, 8, 128))


def transfer_table(out, blocks=8, shapes=README_TRANSFER_SHAPES):
    dev = "cuda"
    for (T, L, H, D) in shapes:
        nbytes = T * L * H * D
        pool = memory.alloc_numa_pinned_tensor(blocks * nbytes)
        pool.copy_(torch.randint(-128, 128, (blocks * nbytes,), dtype=torch.int8,
                                 generator=torch.Generator().manual_seed(L * 10 + H)))
        host_blocks = list(pool.view(blocks, T, L, H, D).unbind(0))
        dev_blocks = torch.zeros(blocks, L, H, T, D, dtype=torch.int8, device=dev)
        ptrs = [torch.tensor([dev_blocks[b, l].data_ptr() for l in range(L)], dtype=torch.int64).to(dev)
                for b in range(blocks)]
        staging = torch.empty(T, L, H, D, dtype=torch.int8, device=dev)
        row = {"shape": [T, L, H, D], "block_bytes": nbytes}
        # "memcpy": one hipMemcpyAsync of the same block, timed the same way (the yardstick for a transfer this short)
        for name, fused in (("direct", False), ("staged", True), ("memcpy", None)):
            def call(b):
                if fused is None:
                    staging.copy_(host_blocks[b], non_blocking=True)
                elif fused:
                    torch.ops.pcie_through.fused_memcpy_multi_layer_block_transfer(ptrs[b], host_blocks[b], staging, 4)
                else:
                    torch.ops.pcie_through.multi_layer_block_transfer(ptrs[b], host_blocks[b], 4)
            for b in range(blocks):
                call(b)
            torch.cuda.synchronize()
            times = []
            for rep in range(3):
                for b in range(blocks):
                    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    s.record()
                    call(b)
                    e.record()
                    times.append((s, e))
            torch.cuda.synchronize()
            ms = sum(s.elapsed_time(e) for s, e in times) / len(times)
            if fused is None:
                assert torch.equal(staging.cpu(), host_blocks[blocks - 1]), "memcpy mismatch"
            else:
                got = dev_blocks.cpu()
                for b in range(blocks):
                    assert torch.equal(got[b].permute(2, 0, 1, 3), host_blocks[b]), "transfer mismatch"
                dev_blocks.zero_()   # the next leg must move the bytes itself
            row[name + "_ms"] = ms
            row[name + "_GBps"] = nbytes / (ms * 1e6)
            row[name + "_frac_of_pcie5_x16"] = row[name + "_GBps"] / PCIE5_X16_GBPS
        # all blocks in one launch through the block table, host -> device and device -> host
        caches = torch.zeros(L, blocks, H, T, D, dtype=torch.int8, device=dev)
        lptrs = torch.tensor([caches[l].data_ptr() for l in range(L)], dtype=torch.int64).to(dev)
        pairs = torch.stack([torch.arange(blocks), torch.arange(blocks).flip(0)], 1).contiguous().to(dev)
        host_pool = pool.view(blocks, T, L, H, D)
        back_pool = memory.alloc_numa_pinned_tensor(blocks * nbytes).view(blocks, T, L, H, D)
        for name, to_host, hp in (("table_in", False, host_pool), ("table_out", True, back_pool)):
            def call_table():
                torch.ops.pcie_through.multi_layer_block_table_transfer(lptrs, hp, pairs, H * T * D, blocks, to_host)
            call_table()
            torch.cuda.synchronize()
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for _ in range(5):
                call_table()
            e.record()
            torch.cuda.synchronize()
            ms = s.elapsed_time(e) / 5
            row[name + "_ms"] = ms
            row[name + "_GBps"] = blocks * nbytes / (ms * 1e6)
            row[name + "_frac_of_pcie5_x16"] = row[name + "_GBps"] / PCIE5_X16_GBPS
        got = caches.cpu()
        for b in range(blocks):
            assert torch.equal(got[:, blocks - 1 - b].permute(2, 0, 1, 3), host_blocks[b]), "table transfer mismatch"
        assert torch.equal(back_pool, host_pool), "table transfer round trip mismatch"
        out["transfer"].append(row)
        print("transfer [%d,%d,%d,%d] int8: direct %.3f ms (%.2f GB/s) | staged %.3f ms (%.2f GB/s) | plain hipMemcpyAsync "
              "%.2f GB/s | %d blocks in one launch: in %.2f GB/s, out %.2f GB/s" %
              (T, L, H, D, row["direct_ms"], row["direct_GBps"], row["staged_ms"], row["staged_GBps"], row["memcpy_GBps"], blocks,
               row["table_in_GBps"], row["table_out_GBps"]), file=sys.stderr, flush=True)
        del back_pool, host_pool
        del pool, host_blocks


def config1_latency(out, runs=500):
    """Single-layer paged KV gather of the benchmark's first configuration: K and V caches
    [1024, 16, 8, 128] fp16, 32 block ids -> [32, 16, 8, 128] each. 1 MiB per call: launch latency."""
    from heterofusedkernels_amd import workloads as W
    cfg = W.C1_GATHER_FP16
    dev = "cuda"
    ids = W.gather_ids(cfg).to(dev)
    planes = [W.make_plane(cfg, 0, kv, cfg.dev_blocks).to(dev) for kv in range(2)]
    outs = [torch.empty((32,) + cfg.block_shape, dtype=cfg.dtype, device=dev) for _ in range(2)]

    def ours():
        for kv in range(2):
            torch.ops.pcie_through.gather(planes[kv], outs[kv], ids)

    def torch_path():
        for kv in range(2):
            torch.index_select(planes[kv], 0, ids, out=outs[kv])

    res = {}
    for name, fn in (("pcie_through.gather", ours), ("torch.index_select", torch_path)):
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(runs):
            fn()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / runs
        res[name] = {"us_per_K_and_V": dt * 1e6, "payload_GBps": 2 * 32 * cfg.block_bytes / dt / 1e9}
    for kv in range(2):
        torch.ops.pcie_through.gather(planes[kv], outs[kv], ids)
        torch.cuda.synchronize()
        assert torch.equal(outs[kv].view(torch.int16), planes[kv].index_select(0, ids).view(torch.int16))
    cpu_planes = [p.cpu() for p in planes]
    cpu_ids = ids.cpu()
    t0 = time.perf_counter()
    for _ in range(runs):
        for kv in range(2):
            cpu_planes[kv].index_select(0, cpu_ids)
    dt = (time.perf_counter() - t0) / runs
    res["torch CPU index_select (%d threads)" % torch.get_num_threads()] = {
        "us_per_K_and_V": dt * 1e6, "payload_GBps": 2 * 32 * cfg.block_bytes / dt / 1e9}
    out["config1"] = res
    for k, v in res.items():
        print("config 1 (K+V, 32 blocks of 32 KiB each): %-40s %.1f us, %.1f GB/s payload" %
              (k, v["us_per_K_and_V"], v["payload_GBps"]), file=sys.stderr, flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--rows", type=int, default=4000000, help="embedding rows (reference: 4 000 000)")
    ap.add_argument("--runs", type=int, default=200)
    ap.add_argument("--only", default="config1,gather,gather_hbm,transfer",
                    help="comma list of: config1, gather, gather_hbm, transfer")
    ap.add_argument("--fill", default="randn", choices=["randn", "bytes"], help="how the gather's host table is filled")
    ap.add_argument("--transfer-shape", default=None,
                    help="one T,L,H,D instead of the README's four shapes (e.g. 1024,64,8,128), for profiling")
    args = ap.parse_args()
    assert torch.cuda.is_available()
    parts = set(args.only.split(","))
    assert parts <= {"config1", "gather", "gather_hbm", "transfer"}, "unknown part in --only"
    out = {"gather": [], "transfer": [], "rows": args.rows, "runs": args.runs}
    if "config1" in parts:
        config1_latency(out)
    if "gather" in parts:
        gather_table(args.rows, args.runs, out, fill=args.fill)
    if "gather_hbm" in parts:
        gather_hbm_table(out)
    if "transfer" in parts:
        shapes = README_TRANSFER_SHAPES
        if args.transfer_shape:
            shapes = (tuple(int(x) for x in args.transfer_shape.split(",")),)
            assert len(shapes[0]) == 4, "--transfer-shape takes T,L,H,D"
        transfer_table(out, shapes=shapes)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
