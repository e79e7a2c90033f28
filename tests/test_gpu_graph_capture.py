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
        torch.ops.pcie_through.swap_blocks(htab, dtab, pairs_out, bb, bb, bb, cfg.dev_blocks, cfg.host_blocks)
        torch.ops.pcie_through.swap_blocks(btab, htab, pairs_in, bb, bb, bb, cfg.host_blocks, cfg.dev_blocks)
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
