"""The ops allocate nothing and launch on the current stream, so they can be recorded
into a HIP graph. Each graph is replayed several times with eager work and
synchronizations in between, with fresh inputs, and every replay is compared with the
eager result."""
import pytest
import torch

import heterofusedkernels_amd  # noqa: F401
import pcie_through
from heterofusedkernels import memory
from heterofusedkernels_amd import workloads as W

from gpu_helpers import announce

pytestmark = pytest.mark.gpu
DEV = "cuda"


def test_swap_and_gather_replay_in_a_hip_graph():
    cfg = W.C2_LLAMA8B_SWAP_OUT.scaled(layers=2, dev_blocks=64, host_blocks=64, n_blocks=16)
    announce("HIP graph: swap-out + swap-in + gather recorded once, replayed 4 times")
    bb = cfg.block_bytes
    dev = [torch.zeros(cfg.dev_blocks, bb, dtype=torch.uint8, device=DEV) for _ in range(cfg.planes)]
    back = [torch.zeros(cfg.dev_blocks, bb, dtype=torch.uint8, device=DEV) for _ in range(cfg.planes)]
    prefill = [torch.zeros(cfg.n_blocks, bb, dtype=torch.uint8, device=DEV) for _ in range(cfg.planes)]
    pool = memory.alloc_numa_pinned_tensor(cfg.planes * cfg.host_blocks * bb)
    host = list(pool.view(torch.uint8).view(cfg.planes, cfg.host_blocks, bb).unbind(0))
    dtab = pcie_through.plane_pointer_table(dev, DEV)
    btab = pcie_through.plane_pointer_table(back, DEV)
    ptab = pcie_through.plane_pointer_table(prefill, DEV)
    htab = pcie_through.plane_pointer_table(host, DEV)
    pairs_out = torch.zeros(cfg.n_blocks, 2, dtype=torch.int64, device=DEV)     # static buffers, refilled per replay
    pairs_in = torch.zeros(cfg.n_blocks, 2, dtype=torch.int64, device=DEV)
    ids = torch.zeros(cfg.n_blocks, dtype=torch.int64, device=DEV)

    def run():
        # swap-out in the paced beside-compute shape (its schedule restarts with every replay), swap-in with its side named
        torch.ops.pcie_through.swap_blocks(htab, dtab, pairs_out, bb, bb, bb, cfg.dev_blocks, cfg.host_blocks, None, 1 | 4)
        torch.ops.pcie_through.swap_blocks(btab, htab, pairs_in, bb, bb, bb, cfg.host_blocks, cfg.dev_blocks, None, 2)
        torch.ops.pcie_through.gather_blocks(ptab, dtab, ids, bb, bb, cfg.dev_blocks)

    def set_inputs(seed):
        gen = torch.Generator().manual_seed(seed)
        for p in range(cfg.planes):
            dev[p].copy_(torch.randint(0, 256, (cfg.dev_blocks, bb), dtype=torch.uint8, generator=gen))
            back[p].zero_()
        src = torch.randperm(cfg.dev_blocks, generator=gen)[:cfg.n_blocks]
        slot = torch.randperm(cfg.host_blocks, generator=gen)[:cfg.n_blocks]
        dst = torch.randperm(cfg.dev_blocks, generator=gen)[:cfg.n_blocks]
        pairs_out.copy_(torch.stack([src, slot], 1))
        pairs_in.copy_(torch.stack([slot, dst], 1))
        ids.copy_(src)
        return src, slot, dst

    def check(src, slot, dst, tag):
        for p in range(cfg.planes):
            d = dev[p].cpu()
            assert torch.equal(host[p][slot], d[src]), tag + " swap-out plane %d" % p
            assert torch.equal(back[p].cpu()[dst], d[src]), tag + " swap-in plane %d" % p
            assert torch.equal(prefill[p].cpu(), d[src]), tag + " gather plane %d" % p

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):                      # warm-up on a side stream, as graph capture wants
        set_inputs(0)
        run()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for replay in range(4):
        src, slot, dst = set_inputs(100 + replay)   # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        check(src, slot, dst, "replay %d" % replay)
        set_inputs(200 + replay)                     # same inputs eagerly: the eager result is the reference
        src2, slot2, dst2 = set_inputs(100 + replay)
        run()
        torch.cuda.synchronize()
        check(src2, slot2, dst2, "eager %d" % replay)


def test_duplex_staged_and_table_transfer_replay_in_a_hip_graph():
    """The newer entry points record as well: the duplex swap (one kernel), the staged swap (kernel +
    DMA copy nodes; its host slot list is read at capture time and therefore fixed for the graph), the same
    through the library's own staging array (the entry point made for callers that cannot allocate, such as
    this one; its first call, which asks the runtime for the array's address, is the eager run before the
    capture) and the block-table transfer in both directions."""
    announce("HIP graph: duplex swap + staged swap (caller's and library's staging) + block-table transfer, replayed 3 times")
    planes, blocks, bb, n = 4, 48, 32768, 10
    dev = [torch.zeros(blocks, bb, dtype=torch.uint8, device=DEV) for _ in range(planes)]
    pool = memory.alloc_numa_pinned_tensor(planes * blocks * bb)
    host = list(pool.view(torch.uint8).view(planes, blocks, bb).unbind(0))
    dtab, htab = pcie_through.plane_pointer_table(dev, DEV), pcie_through.plane_pointer_table(host, DEV)
    host_addrs = torch.tensor([h.data_ptr() for h in host], dtype=torch.int64)
    out_pairs = torch.zeros(n, 2, dtype=torch.int64, device=DEV)
    in_pairs = torch.zeros(n, 2, dtype=torch.int64, device=DEV)
    staged_ids = torch.zeros(n, dtype=torch.int64, device=DEV)
    staged_slots = torch.arange(30, 30 + n)                               # fixed at capture
    staging = torch.zeros(planes, n, bb, dtype=torch.uint8, device=DEV)
    n_static = 8
    static_ids = torch.zeros(n_static, dtype=torch.int64, device=DEV)
    static_slots = torch.arange(40, 40 + n_static)                         # fixed at capture, after the staged swap's slots
    T, L, H, D = 32, 3, 2, 64
    tpool = memory.alloc_numa_pinned_tensor(6 * T * L * H * D).view(6, T, L, H, D)
    tback = memory.alloc_numa_pinned_tensor(6 * T * L * H * D).view(6, T, L, H, D)
    caches = torch.zeros(L, 5, H, T, D, dtype=torch.int8, device=DEV)
    lptrs = torch.tensor([caches[l].data_ptr() for l in range(L)], dtype=torch.int64).to(DEV)
    tpairs = torch.zeros(4, 2, dtype=torch.int64, device=DEV)

    def run():
        torch.ops.pcie_through.swap_blocks_duplex(dtab, htab, out_pairs, in_pairs, bb, bb, bb, blocks, blocks)
        torch.ops.pcie_through.swap_blocks_staged(dtab, host_addrs, staged_ids, staged_slots, staging, bb, bb, bb, True,
                                                  blocks, blocks)
        torch.ops.pcie_through.swap_blocks_staged_static(dtab, host_addrs, static_ids, static_slots, bb, bb, bb, True,
                                                         blocks, blocks)
        torch.ops.pcie_through.multi_layer_block_table_transfer(lptrs, tpool, tpairs, H * T * D, 5, False)
        torch.ops.pcie_through.multi_layer_block_table_transfer(lptrs, tback, tpairs, H * T * D, 5, True)

    def set_inputs(seed):
        gen = torch.Generator().manual_seed(seed)
        state = {}
        for p in range(planes):
            dev[p].copy_(torch.randint(0, 256, (blocks, bb), dtype=torch.uint8, generator=gen))
            host[p].copy_(torch.randint(0, 256, (blocks, bb), dtype=torch.uint8, generator=gen))
        state["dev"] = [d.cpu() for d in dev]
        state["host"] = [h.clone() for h in host]
        dperm = torch.randperm(30, generator=gen)                       # device blocks 0..29, host slots 0..29 for the duplex
        hperm = torch.randperm(30, generator=gen)
        state["out"] = torch.stack([dperm[:n], hperm[:n]], 1)
        state["in"] = torch.stack([hperm[n:2 * n], dperm[n:2 * n]], 1)
        state["staged"] = 30 + torch.randperm(blocks - 30, generator=gen)[:n]   # device blocks 30.. -> host slots 30..
        out_pairs.copy_(state["out"])
        in_pairs.copy_(state["in"])
        staged_ids.copy_(state["staged"])
        state["static"] = 30 + torch.randperm(blocks - 30, generator=gen)[:n_static]
        static_ids.copy_(state["static"])
        tpool.copy_(torch.randint(-128, 128, tuple(tpool.shape), dtype=torch.int8, generator=gen))
        tback.zero_()
        state["tpairs"] = torch.stack([torch.randperm(6, generator=gen)[:4], torch.randperm(5, generator=gen)[:4]], 1)
        tpairs.copy_(state["tpairs"])
        return state

    def check(st, tag):
        for p in range(planes):
            h, d = host[p], dev[p].cpu()
            assert torch.equal(h[st["out"][:, 1]], st["dev"][p][st["out"][:, 0]]), tag + " duplex out"
            assert torch.equal(d[st["in"][:, 1]], st["host"][p][st["in"][:, 0]]), tag + " duplex in"
            assert torch.equal(h[30:30 + n], st["dev"][p][st["staged"]]), tag + " staged"
            assert torch.equal(h[40:40 + n_static], st["dev"][p][st["static"]]), tag + " staged through the library's array"
        for hb, _ in st["tpairs"].tolist():
            assert torch.equal(tback[hb], tpool[hb]), tag + " table transfer round trip"

    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        set_inputs(1)
        run()
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for replay in range(3):
        st = set_inputs(50 + replay)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        check(st, "replay %d" % replay)
        st = set_inputs(50 + replay)
        run()
        torch.cuda.synchronize()
        check(st, "eager %d" % replay)
