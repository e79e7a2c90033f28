"""GPU parity: the HIP kernels, called through the C-ABI (ctypes) and through the
torch ops, against the CPU oracle and the committed golden vectors, bit for bit.

Sizes here are ones the oracle finishes in seconds; the full-size configurations
are covered by tests/test_gpu_fullsize.py through size-independent properties.
"""
import glob
import os

import numpy as np
import pytest
import torch

import heterofusedkernels_amd  # noqa: F401  (puts the drop-in packages on sys.path)
import pcie_through  # noqa: F401  (registers torch.ops.pcie_through.*)
from heterofusedkernels_amd import capi
from heterofusedkernels_amd import workloads as W
from oracle import oracle as O

from gpu_helpers import (announce, bytes_np, gather_blocks, gather_rows, host_ptr_table, ptr_table, stream_handle,
                         swap)

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DEV = "cuda"


def _golden(prefix):
    return [(os.path.basename(f), f) for f in sorted(glob.glob(os.path.join(GOLDEN, prefix + "_*.npz")))]


@pytest.fixture(scope="module")
def memory():
    import heterofusedkernels_amd  # noqa: F401
    import pcie_through  # noqa: F401
    from heterofusedkernels import memory as m

    return m


def _pinned(memory, nbytes, fill=None):
    t = memory.alloc_numa_pinned_tensor(nbytes)
    assert t.is_pinned() and t.device.type == "cpu" and t.dtype == torch.int8 and t.dim() == 1
    if fill is not None:
        t.view(torch.uint8).fill_(fill)
    return t


# ---------------------------------------------------------------------------
# golden vectors through the C-ABI
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("name,path", _golden("gather"))
def test_golden_gather(name, path):
    announce("golden gather " + name)
    g = np.load(path)
    table = torch.from_numpy(g["table"]).to(DEV)
    ids = torch.from_numpy(g["ids"]).to(DEV)
    dst = torch.full(g["expected"].shape, 0xEE, dtype=torch.uint8, device=DEV)
    gather_rows(table, dst, ids, table.shape[1], table_rows=table.shape[0])
    torch.cuda.synchronize()
    assert np.array_equal(dst.cpu().numpy(), g["expected"])


@pytest.mark.parametrize("name,path", _golden("swap"))
def test_golden_swap(name, path):
    announce("golden swap " + name)
    g = np.load(path)
    planes, sblocks, bb = g["src"].shape
    dblocks = g["dst_before"].shape[1]
    src = [torch.from_numpy(np.ascontiguousarray(g["src"][p])).to(DEV) for p in range(planes)]
    dst = [torch.from_numpy(g["dst_before"][p].copy()).to(DEV) for p in range(planes)]
    pairs = torch.from_numpy(g["pairs"]).to(DEV)
    swap(ptr_table(dst), ptr_table(src), pairs, planes, bb, src_blocks=sblocks, dst_blocks=dblocks)
    torch.cuda.synchronize()
    got = np.stack([d.cpu().numpy() for d in dst])
    assert np.array_equal(got, g["expected"])


@pytest.mark.parametrize("name,path", _golden("transfer"))
def test_golden_transfer(name, path):
    announce("golden transfer " + name)
    g = np.load(path)
    T, L, H, D, e = (int(x) for x in g["geometry"])
    src = torch.from_numpy(g["src"]).to(DEV)
    layers = torch.full((L, H * T * D * e), 0xEE, dtype=torch.uint8, device=DEV)
    ptrs = ptr_table([layers[l] for l in range(L)])
    capi.check(capi.multi_layer_block_transfer(ptrs.data_ptr(), src.data_ptr(), T, L, H, D, e, 0, stream_handle()))
    torch.cuda.synchronize()
    assert np.array_equal(layers.cpu().numpy(), g["expected"])


# ---------------------------------------------------------------------------
# configuration 1: single-layer paged KV gather, exact sizes
# ---------------------------------------------------------------------------
def test_config1_gather_fp16_exact():
    cfg = W.C1_GATHER_FP16
    announce("config 1 gather K and V [1024,16,8,128] fp16, 32 ids")
    ids = W.gather_ids(cfg)
    assert ids.numel() == 32 and ids.unique().numel() == 32
    for kv in range(cfg.kv):
        plane = W.make_plane(cfg, 0, kv, cfg.dev_blocks)
        want = O.torch_gather_rows(plane, ids)                       # the CPU torch path
        out = torch.zeros((32,) + cfg.block_shape, dtype=cfg.dtype, device=DEV)
        gather_rows(plane.to(DEV), out, ids.to(DEV), cfg.block_bytes, table_rows=cfg.dev_blocks)
        torch.cuda.synchronize()
        assert np.array_equal(bytes_np(out), bytes_np(want))
        assert np.array_equal(bytes_np(out), O.c_gather_rows(bytes_np(plane), ids.numpy()))
        # same through the torch op, with the table viewed as [blocks, 16384] like an embedding table
        out2 = torch.zeros(32, cfg.block_elems, dtype=cfg.dtype, device=DEV)
        torch.ops.pcie_through.gather(plane.view(cfg.dev_blocks, -1).to(DEV), out2, ids.to(DEV), aiv=4)
        torch.cuda.synchronize()
        assert np.array_equal(bytes_np(out2), bytes_np(want))
        out3 = torch.zeros_like(out2)                                   # alias-annotated variant
        torch.ops.pcie_through.gather_into(plane.view(cfg.dev_blocks, -1).to(DEV), out3, ids.to(DEV))
        torch.cuda.synchronize()
        assert np.array_equal(bytes_np(out3), bytes_np(want))


# ---------------------------------------------------------------------------
# gather from host-registered memory (the reference's embedding use)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("bs", [1, 16, 256, 1024])
@pytest.mark.parametrize("id_dtype", [torch.int64, torch.int32])
def test_gather_from_registered_host_table(memory, bs, id_dtype):
    rows, dim = 20000, 512                                     # fp16 rows of 1 KiB (tests/test_gather.py:35-41)
    announce("host-table gather bs=%d ids=%s" % (bs, id_dtype))
    embed = _pinned(memory, rows * dim * 2).view(torch.float16).view(rows, dim)
    gen = torch.Generator().manual_seed(bs)
    embed.copy_(torch.randn(rows, dim, generator=gen).to(torch.float16))
    ids = torch.randint(0, rows, (bs,), generator=gen, dtype=torch.int64).to(id_dtype)
    dst = torch.zeros(bs, dim, dtype=torch.float16, device=DEV)
    torch.ops.pcie_through.gather(embed, dst, ids.to(DEV), aiv=4)        # keyword aiv (tests/test_gather.py:56)
    torch.cuda.synchronize()
    want = embed[ids.to(torch.int64)]                                    # tests/test_memcpy.py:18
    assert np.array_equal(bytes_np(dst), bytes_np(want))
    dst2 = torch.zeros_like(dst)
    torch.ops.pcie_through.gather(embed, dst2, ids.to(DEV))              # default aiv (test_gather_combine.py:51-55)
    torch.cuda.synchronize()
    assert torch.equal(dst2.cpu().view(torch.int16), dst.cpu().view(torch.int16))


def test_gather_from_reference_scale_host_table(memory):
    """The reference's own table: [4 000 000, 512] fp16 (4 GB) in registered host memory, int64 ids on
    the device, aiv=4 and default (pcieThrough/tests/test_gather.py:35-58), at batch sizes from its loop
    (8 .. 2040 in steps of 8), at the size of its combined call (ten batches of 2040 ids in one call,
    default aiv: pcieThrough/tests/test_gather_combine.py:47-56; 20 MiB per call, which takes the grid
    bound of a long gather out of host memory) and with random rows instead of its all-zero table."""
    rows, dim = 4000000, 512
    announce("host-table gather out of the reference's 4 000 000 x 512 fp16 table")
    embed = _pinned(memory, rows * dim * 2).view(torch.float16).view(rows, dim)
    part = 500000                                               # random bytes made on the device, copied over
    for first in range(0, rows, part):
        chunk = torch.randint(0, 256, (part, dim * 2), dtype=torch.uint8, device=DEV,
                              generator=torch.Generator(device=DEV).manual_seed(first))
        embed[first:first + part].view(torch.uint8).copy_(chunk)
    gen = torch.Generator().manual_seed(4000000)
    for bs in (8, 16, 128, 1024, 2040, 20400):
        ids = torch.randint(0, rows, (bs,), generator=gen, dtype=torch.int64)
        ids[0], ids[-1] = 0, rows - 1                           # both ends of the table
        for aiv in ((None,) if bs == 20400 else (4, None)):
            dst = torch.zeros(bs, dim, dtype=torch.float16, device=DEV)
            torch.ops.pcie_through.gather(embed, dst, ids.to(DEV), aiv=aiv)
            torch.cuda.synchronize()
            want = embed[ids]                                   # tests/test_memcpy.py:18
            assert np.array_equal(bytes_np(dst), bytes_np(want)), "bs %d aiv %s" % (bs, aiv)
        assert np.array_equal(bytes_np(dst), O.c_gather_rows(bytes_np(embed), ids.numpy())), "bs %d vs oracle" % bs


def test_gather_from_torch_pinned_table_without_registration(memory):
    """A tensor pinned by torch itself can be handed to the op directly; nothing is recorded for it."""
    announce("host-table gather from a torch.pin_memory() tensor, never registered")
    gen = torch.Generator().manual_seed(5)
    embed = torch.randn(3000, 512, generator=gen).to(torch.float16).pin_memory()
    ids = torch.randint(0, 3000, (77,), generator=gen)
    n0 = memory.record_count()
    dst = torch.zeros(77, 512, dtype=torch.float16, device=DEV)
    torch.ops.pcie_through.gather(embed, dst, ids.to(DEV))
    torch.cuda.synchronize()
    assert np.array_equal(bytes_np(dst), bytes_np(embed[ids]))
    assert memory.record_count() == n0
    sub = embed[1000:]                                          # interior view of the pinned block
    torch.ops.pcie_through.gather(sub, dst, ids.to(DEV) % 2000)
    torch.cuda.synchronize()
    assert np.array_equal(bytes_np(dst), bytes_np(sub[ids % 2000]))
    with pytest.raises(RuntimeError, match="neither registered"):
        torch.ops.pcie_through.gather(torch.zeros(8, 512, dtype=torch.float16), dst, ids.to(DEV))


# ---------------------------------------------------------------------------
# configurations 2-5, scaled: block-table swap against index_select / index_copy_
# ---------------------------------------------------------------------------
def _host_pool(memory, cfg, blocks, fill=0x5C):
    pool = _pinned(memory, cfg.planes * blocks * cfg.block_bytes, fill=fill)
    return pool, list(pool.view(torch.uint8).view(cfg.planes, blocks, cfg.block_bytes).unbind(0))


def _cpu_planes(cfg, blocks):
    return [W.make_plane(cfg, l, kv, blocks) for l in range(cfg.layers) for kv in range(cfg.kv)]


def test_config2_swap_out_scaled(memory):
    cfg = W.C2_LLAMA8B_SWAP_OUT.scaled(layers=4, dev_blocks=256, host_blocks=512, n_blocks=64)
    announce("config 2 scaled swap-out: %d planes, %d pairs, %d B blocks" % (cfg.planes, cfg.n_blocks, cfg.block_bytes))
    cpu = _cpu_planes(cfg, cfg.dev_blocks)
    dev = [p.to(DEV) for p in cpu]
    pool, host = _host_pool(memory, cfg, cfg.host_blocks)
    src_ids, dst_ids = W.block_table(cfg, src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
    pairs = W.pairs_tensor(src_ids, dst_ids)
    swap(host_ptr_table(host), ptr_table(dev), pairs.to(DEV), cfg.planes, cfg.block_bytes,
         src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want = torch.full((cfg.host_blocks, cfg.block_bytes), 0x5C, dtype=torch.uint8)
        O.torch_swap_blocks(want, W.as_bytes(cpu[p]), src_ids, dst_ids)      # index_copy_(index_select)
        assert torch.equal(host[p], want), "plane %d" % p                     # incl. every untouched slot
        assert torch.equal(W.as_bytes(dev[p].cpu()), W.as_bytes(cpu[p]))      # source unchanged
    # C restatement agrees as well
    want_c = [np.full((cfg.host_blocks, cfg.block_bytes), 0x5C, dtype=np.uint8) for _ in range(cfg.planes)]
    O.c_swap_blocks(want_c, [bytes_np(p) for p in cpu], pairs.numpy())
    for p in range(cfg.planes):
        assert np.array_equal(host[p].numpy(), want_c[p])


def test_config3_swap_in_scaled(memory):
    cfg = W.C3_LLAMA70B_SWAP_IN.scaled(layers=5, dev_blocks=256, host_blocks=512, n_blocks=96)
    announce("config 3 scaled swap-in: %d planes, %d pairs" % (cfg.planes, cfg.n_blocks))
    pool, host = _host_pool(memory, cfg, cfg.host_blocks, fill=None)
    cpu_host = _cpu_planes(cfg, cfg.host_blocks)
    for p in range(cfg.planes):
        host[p].copy_(W.as_bytes(cpu_host[p]))
    dev = [torch.full((cfg.dev_blocks, cfg.block_bytes), 0x6D, dtype=torch.uint8, device=DEV) for _ in range(cfg.planes)]
    gen = torch.Generator().manual_seed(33)
    perm = torch.randperm(cfg.host_blocks, generator=gen)             # block table as a permutation slice
    src_ids = perm[:cfg.n_blocks].contiguous()
    dst_ids = torch.randperm(cfg.dev_blocks, generator=gen)[:cfg.n_blocks].contiguous()
    swap(ptr_table(dev), host_ptr_table(host), W.pairs_tensor(src_ids, dst_ids).to(DEV), cfg.planes, cfg.block_bytes,
         src_blocks=cfg.host_blocks, dst_blocks=cfg.dev_blocks)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want = torch.full((cfg.dev_blocks, cfg.block_bytes), 0x6D, dtype=torch.uint8)
        O.torch_swap_blocks(want, W.as_bytes(cpu_host[p]), src_ids, dst_ids)
        assert torch.equal(dev[p].cpu(), want), "plane %d" % p
        assert torch.equal(host[p], W.as_bytes(cpu_host[p]))


def test_config4_mla_round_trip_scaled(memory):
    cfg = W.C4_MLA_ROUNDTRIP.scaled(layers=7, dev_blocks=64, host_blocks=64, n_blocks=16)
    assert cfg.block_bytes == 73728
    announce("config 4 scaled MLA round trip: %d planes, block %d B" % (cfg.planes, cfg.block_bytes))
    cpu = _cpu_planes(cfg, cfg.dev_blocks)
    dev = [p.to(DEV) for p in cpu]
    pool, host = _host_pool(memory, cfg, cfg.host_blocks, fill=0)
    gen = torch.Generator().manual_seed(44)
    out_src = torch.randperm(cfg.dev_blocks, generator=gen)[:cfg.n_blocks]
    host_slots = torch.randperm(cfg.host_blocks, generator=gen)[:cfg.n_blocks]
    free = torch.tensor([b for b in range(cfg.dev_blocks) if b not in set(out_src.tolist())])
    in_dst = free[torch.randperm(len(free), generator=gen)[:cfg.n_blocks]]   # different slots
    dtab, htab = ptr_table(dev), host_ptr_table(host)
    swap(htab, dtab, W.pairs_tensor(out_src, host_slots).to(DEV), cfg.planes, cfg.block_bytes,
         src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
    swap(dtab, htab, W.pairs_tensor(host_slots, in_dst).to(DEV), cfg.planes, cfg.block_bytes,
         src_blocks=cfg.host_blocks, dst_blocks=cfg.dev_blocks)               # same stream: ordered after swap-out
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        got = W.as_bytes(dev[p].cpu())
        orig = W.as_bytes(cpu[p])
        assert torch.equal(got[in_dst], orig[out_src]), "plane %d round trip" % p
        untouched = torch.ones(cfg.dev_blocks, dtype=torch.bool)
        untouched[in_dst] = False
        assert torch.equal(got[untouched], orig[untouched])


def test_config5_fp8_fragmented_scaled(memory):
    cfg = W.C5_FP8_FRAGMENTED.scaled(layers=3, dev_blocks=512, host_blocks=512, n_blocks=256)
    announce("config 5 scaled fp8 fragmented gather + swap-out: %d planes, %d ids" % (cfg.planes, cfg.n_blocks))
    ids = W.fragmented_ids(cfg.dev_blocks, cfg.n_blocks)
    cpu = _cpu_planes(cfg, cfg.dev_blocks)
    dev = [p.to(DEV) for p in cpu]
    prefill = [torch.zeros(cfg.n_blocks, cfg.block_bytes, dtype=torch.uint8, device=DEV) for _ in range(cfg.planes)]
    gather_blocks(ptr_table(prefill), ptr_table(dev), ids.to(DEV), cfg.planes, cfg.block_bytes,
                  src_blocks=cfg.dev_blocks)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want = O.torch_gather_rows(W.as_bytes(cpu[p]), ids)
        assert torch.equal(prefill[p].cpu(), want), "plane %d" % p
    # matching swap-out of the same ids to host slots 0..n-1
    pool, host = _host_pool(memory, cfg, cfg.host_blocks, fill=0x11)
    pairs = W.pairs_tensor(ids, torch.arange(cfg.n_blocks))
    swap(host_ptr_table(host), ptr_table(dev), pairs.to(DEV), cfg.planes, cfg.block_bytes,
         src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        assert torch.equal(host[p][:cfg.n_blocks], prefill[p].cpu())
        assert (host[p][cfg.n_blocks:] == 0x11).all()
    # through the torch op too
    prefill2 = [torch.zeros_like(x) for x in prefill]
    torch.ops.pcie_through.gather_blocks(ptr_table(prefill2), ptr_table(dev), ids.to(DEV), cfg.block_bytes,
                                         cfg.block_bytes, cfg.dev_blocks)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        assert torch.equal(prefill2[p], prefill[p])


@pytest.mark.parametrize("cfg,n_out,n_in", [
    (W.C2_LLAMA8B_SWAP_OUT.scaled(layers=3, dev_blocks=128, host_blocks=192), 40, 40),
    (W.C2_LLAMA8B_SWAP_OUT.scaled(layers=2, dev_blocks=128, host_blocks=192), 50, 7),
    (W.C4_MLA_ROUNDTRIP.scaled(layers=5, dev_blocks=48, host_blocks=48), 9, 20),
    (W.C5_FP8_FRAGMENTED.scaled(layers=2, dev_blocks=256, host_blocks=256), 0, 60),
    (W.C5_FP8_FRAGMENTED.scaled(layers=2, dev_blocks=256, host_blocks=256), 60, 0),
])
def test_duplex_swap_equals_two_swaps(memory, cfg, n_out, n_in):
    """One duplex launch == swap-out then swap-in through index_select / index_copy_ on disjoint blocks."""
    announce("duplex swap %s: %d out, %d in, %d planes" % (cfg.name, n_out, n_in, cfg.planes))
    bb = cfg.block_bytes
    cpu_dev = [W.as_bytes(p).clone() for p in _cpu_planes(cfg, cfg.dev_blocks)]
    dev = [p.to(DEV) for p in cpu_dev]
    pool, host = _host_pool(memory, cfg, cfg.host_blocks, fill=None)
    gen = torch.Generator().manual_seed(n_out * 100 + n_in)
    cpu_host = [torch.randint(0, 256, (cfg.host_blocks, bb), dtype=torch.uint8, generator=gen) for _ in range(cfg.planes)]
    for p in range(cfg.planes):
        host[p].copy_(cpu_host[p])
    dperm = torch.randperm(cfg.dev_blocks, generator=gen)
    hperm = torch.randperm(cfg.host_blocks, generator=gen)
    out_pairs = W.pairs_tensor(dperm[:n_out], hperm[:n_out])                          # device block -> host block
    in_pairs = W.pairs_tensor(hperm[n_out:n_out + n_in], dperm[n_out:n_out + n_in])   # host block -> device block
    dtab, htab = ptr_table(dev), host_ptr_table(host)
    torch.ops.pcie_through.swap_blocks_duplex(dtab, htab, out_pairs.to(DEV), in_pairs.to(DEV), bb, bb, bb,
                                              cfg.dev_blocks, cfg.host_blocks)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want_host, want_dev = cpu_host[p].clone(), cpu_dev[p].clone()
        if n_out:
            O.torch_swap_blocks(want_host, cpu_dev[p], out_pairs[:, 0], out_pairs[:, 1])
        if n_in:
            O.torch_swap_blocks(want_dev, cpu_host[p], in_pairs[:, 0], in_pairs[:, 1])
        assert torch.equal(host[p], want_host), "plane %d host side" % p
        assert torch.equal(dev[p].cpu(), want_dev), "plane %d device side" % p
    # the C-ABI with explicit structs and a tiny grid gives the same bytes
    dev2 = [p.to(DEV) for p in cpu_dev]
    for p in range(cfg.planes):
        host[p].copy_(cpu_host[p])
    dtab2 = ptr_table(dev2)
    po, pi = out_pairs.to(DEV), in_pairs.to(DEV)
    om = capi.BlockMove(htab.data_ptr(), dtab2.data_ptr(), po.data_ptr() if n_out else None, n_out, bb, bb,
                        cfg.dev_blocks, cfg.host_blocks)
    im = capi.BlockMove(dtab2.data_ptr(), htab.data_ptr(), pi.data_ptr() if n_in else None, n_in, bb, bb,
                        cfg.host_blocks, cfg.dev_blocks)
    capi.check(capi.swap_blocks_duplex(om, im, cfg.planes, bb, 3, stream_handle()))
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        assert torch.equal(dev2[p], dev[p]), "plane %d" % p


@pytest.mark.parametrize("cfg,n,pattern", [
    (W.C2_LLAMA8B_SWAP_OUT.scaled(layers=3, dev_blocks=128, host_blocks=192), 48, "run"),
    (W.C2_LLAMA8B_SWAP_OUT.scaled(layers=2, dev_blocks=128, host_blocks=192), 40, "runs"),
    (W.C4_MLA_ROUNDTRIP.scaled(layers=3, dev_blocks=48, host_blocks=64), 17, "scattered"),
    (W.C5_FP8_FRAGMENTED.scaled(layers=2, dev_blocks=256, host_blocks=256), 100, "runs"),
])
def test_staged_swap_equals_direct_swap(memory, cfg, n, pattern):
    """Staged swap-out then staged swap-in (kernel on HBM + DMA copies) == index_select / index_copy_,
    and the staging buffer holds the moved blocks (as the reference's staged op leaves its staging block)."""
    announce("staged swap %s: %d blocks, host slots %s" % (cfg.name, n, pattern))
    bb = cfg.block_bytes
    cpu_dev = [W.as_bytes(p).clone() for p in _cpu_planes(cfg, cfg.dev_blocks)]
    dev = [p.to(DEV) for p in cpu_dev]
    pool, host = _host_pool(memory, cfg, cfg.host_blocks, fill=0x2B)
    gen = torch.Generator().manual_seed(n)
    dev_ids = torch.randperm(cfg.dev_blocks, generator=gen)[:n].contiguous()
    if pattern == "run":
        host_ids = torch.arange(5, 5 + n)
    elif pattern == "runs":
        host_ids = W.fragmented_ids(cfg.host_blocks, n, seed=n)
    else:
        host_ids = torch.randperm(cfg.host_blocks, generator=gen)[:n].contiguous()
    dtab = ptr_table(dev)
    host_addrs = torch.tensor([t.data_ptr() for t in host], dtype=torch.int64)          # host addresses, CPU tensor
    staging = torch.zeros(cfg.planes, n, bb, dtype=torch.uint8, device=DEV)
    torch.ops.pcie_through.swap_blocks_staged(dtab, host_addrs, dev_ids.to(DEV), host_ids, staging, bb, bb, bb, True,
                                              cfg.dev_blocks, cfg.host_blocks)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want = torch.full((cfg.host_blocks, bb), 0x2B, dtype=torch.uint8)
        O.torch_swap_blocks(want, cpu_dev[p], dev_ids, host_ids)
        assert torch.equal(host[p], want), "plane %d host side" % p
        assert torch.equal(staging[p].cpu(), cpu_dev[p][dev_ids]), "plane %d staging" % p
        assert torch.equal(dev[p].cpu(), cpu_dev[p]), "plane %d source changed" % p
    # back in, to other device blocks
    back_ids = torch.roll(dev_ids, 3)
    fresh = [torch.full((cfg.dev_blocks, bb), 0x4D, dtype=torch.uint8, device=DEV) for _ in range(cfg.planes)]
    staging.zero_()
    torch.ops.pcie_through.swap_blocks_staged(ptr_table(fresh), host_addrs, back_ids.to(DEV), host_ids, staging, bb, bb,
                                              bb, False, cfg.dev_blocks, cfg.host_blocks)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want = torch.full((cfg.dev_blocks, bb), 0x4D, dtype=torch.uint8)
        O.torch_swap_blocks(want, host[p], host_ids, back_ids)
        assert torch.equal(fresh[p].cpu(), want), "plane %d device side" % p
    # host planes that are NOT evenly spaced (reversed order) take the per-plane copy path: same bytes
    for p in range(cfg.planes):
        host[p].fill_(0x2B)
    rev = list(reversed(range(cfg.planes)))
    host_addrs_rev = torch.tensor([host[p].data_ptr() for p in rev], dtype=torch.int64)
    dtab_rev = ptr_table([dev[p] for p in rev])
    torch.ops.pcie_through.swap_blocks_staged(dtab_rev, host_addrs_rev, dev_ids.to(DEV), host_ids, staging, bb, bb, bb,
                                              True, cfg.dev_blocks, cfg.host_blocks)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want = torch.full((cfg.host_blocks, bb), 0x2B, dtype=torch.uint8)
        O.torch_swap_blocks(want, cpu_dev[p], dev_ids, host_ids)
        assert torch.equal(host[p], want), "plane %d host side (per-plane copies)" % p
    # a host slot out of range rejects the call before anything is enqueued
    bad = host_ids.clone()
    bad[0] = cfg.host_blocks
    with pytest.raises(RuntimeError, match="hfk_swap_blocks_staged"):
        torch.ops.pcie_through.swap_blocks_staged(dtab, host_addrs, dev_ids.to(DEV), bad, staging, bb, bb, bb, True,
                                                  cfg.dev_blocks, cfg.host_blocks)


@pytest.mark.parametrize("cfg", [
    W.C2_LLAMA8B_SWAP_OUT.scaled(layers=4, dev_blocks=256, host_blocks=256, n_blocks=96),
    W.C4_MLA_ROUNDTRIP.scaled(layers=5, dev_blocks=96, host_blocks=96, n_blocks=40),       # 72 KiB blocks: 4.5 chunks
    W.C5_FP8_FRAGMENTED.scaled(layers=2, dev_blocks=512, host_blocks=512, n_blocks=200),
], ids=lambda c: c.name)
def test_swap_beside_compute_moves_the_same_bytes(memory, cfg):
    """HFK_SWAP_BESIDE_COMPUTE only changes the launch shape (8-24 workgroups, paced toward the host):
    swap-out then swap-in with the flags == index_select / index_copy_, untouched blocks included."""
    announce("swap beside compute %s: %d planes, %d pairs, %d B blocks, link %d MB/s"
             % (cfg.name, cfg.planes, cfg.n_blocks, cfg.block_bytes, capi.get_tuning(capi.KNOB_LINK_MBPS)))
    bb = cfg.block_bytes
    cpu = [W.as_bytes(p).clone() for p in _cpu_planes(cfg, cfg.dev_blocks)]
    dev = [p.to(DEV) for p in cpu]
    pool, host = _host_pool(memory, cfg, cfg.host_blocks, fill=0x33)
    src_ids, dst_ids = W.block_table(cfg, src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
    dtab, htab = ptr_table(dev), host_ptr_table(host)
    out_pairs = W.pairs_tensor(src_ids, dst_ids).to(DEV)
    capi.check(capi.swap_blocks(htab.data_ptr(), dtab.data_ptr(), out_pairs.data_ptr(), cfg.planes, src_ids.numel(), bb, bb, bb,
                                cfg.dev_blocks, cfg.host_blocks, 0, stream_handle(),
                                capi.SWAP_DST_HOST | capi.SWAP_BESIDE_COMPUTE), "hfk_swap_blocks(out, beside compute)")
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want = torch.full((cfg.host_blocks, bb), 0x33, dtype=torch.uint8)
        O.torch_swap_blocks(want, cpu[p], src_ids, dst_ids)
        assert torch.equal(host[p], want), "plane %d host side" % p
    back = torch.roll(src_ids, 5)
    fresh = [torch.full((cfg.dev_blocks, bb), 0x77, dtype=torch.uint8, device=DEV) for _ in range(cfg.planes)]
    in_pairs = W.pairs_tensor(dst_ids, back).to(DEV)
    capi.check(capi.swap_blocks(ptr_table(fresh).data_ptr(), htab.data_ptr(), in_pairs.data_ptr(), cfg.planes, back.numel(), bb, bb,
                                bb, cfg.host_blocks, cfg.dev_blocks, 0, stream_handle(),
                                capi.SWAP_SRC_HOST | capi.SWAP_BESIDE_COMPUTE), "hfk_swap_blocks(in, beside compute)")
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want = torch.full((cfg.dev_blocks, bb), 0x77, dtype=torch.uint8)
        O.torch_swap_blocks(want, host[p], dst_ids, back)
        assert torch.equal(fresh[p].cpu(), want), "plane %d device side" % p
    # and through the torch op
    for p in range(cfg.planes):
        host[p].fill_(0x33)
    torch.ops.pcie_through.swap_blocks(htab, dtab, out_pairs, bb, bb, bb, cfg.dev_blocks, cfg.host_blocks, None,
                                       capi.SWAP_DST_HOST | capi.SWAP_BESIDE_COMPUTE)
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want = torch.full((cfg.host_blocks, bb), 0x33, dtype=torch.uint8)
        O.torch_swap_blocks(want, cpu[p], src_ids, dst_ids)
        assert torch.equal(host[p], want), "plane %d host side (op)" % p
    with pytest.raises(RuntimeError, match="flag"):
        torch.ops.pcie_through.swap_blocks(htab, dtab, out_pairs, bb, bb, bb, cfg.dev_blocks, cfg.host_blocks, None, 64)


def test_paced_swap_ends_when_its_rate_is_unreachably_low(memory):
    """The pacing wait is bounded: at an offered rate of 1 MB/s every chunk's wait runs into its spin limit
    (a few milliseconds) and the swap still completes with the right bytes; an unknown link rate
    (0) simply runs unpaced."""
    cfg = W.C2_LLAMA8B_SWAP_OUT.scaled(layers=1, dev_blocks=16, host_blocks=16, n_blocks=8)
    bb = cfg.block_bytes
    cpu = [W.as_bytes(p).clone() for p in _cpu_planes(cfg, cfg.dev_blocks)]
    dev = [p.to(DEV) for p in cpu]
    src_ids, dst_ids = W.block_table(cfg, src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
    pairs = W.pairs_tensor(src_ids, dst_ids).to(DEV)
    dtab = ptr_table(dev)
    for what, knob, value in (("1 MB/s", capi.KNOB_SWAP_PACE_MBPS, 1), ("unknown link", capi.KNOB_LINK_MBPS, 0)):
        announce("paced swap, %s: %d planes x %d blocks" % (what, cfg.planes, src_ids.numel()))
        pool, host = _host_pool(memory, cfg, cfg.host_blocks, fill=0x11)
        with capi.thread_tuning({knob: value}):      # this thread's calls only; the process-wide knobs stay
            capi.check(capi.swap_blocks(host_ptr_table(host).data_ptr(), dtab.data_ptr(), pairs.data_ptr(), cfg.planes,
                                        src_ids.numel(), bb, bb, bb, cfg.dev_blocks, cfg.host_blocks, 0, stream_handle(),
                                        capi.SWAP_DST_HOST | capi.SWAP_BESIDE_COMPUTE))
        torch.cuda.synchronize()
        for p in range(cfg.planes):
            want = torch.full((cfg.host_blocks, bb), 0x11, dtype=torch.uint8)
            O.torch_swap_blocks(want, cpu[p], src_ids, dst_ids)
            assert torch.equal(host[p], want), "%s plane %d" % (what, p)
    assert capi.get_tuning(capi.KNOB_SWAP_PACE_MBPS) == 0
    announce("PCIe link rate read from sysfs: %d MB/s (0 = unreadable: paced swaps run unpaced)" % capi.get_tuning(capi.KNOB_LINK_MBPS))


def test_pace_report_accounts_for_every_turn(memory):
    """HFK_KNOB_PACE_REPORT: every workgroup of a paced swap leaves its account (ticks run, ticks allotted, turns,
    late turns, largest delay, interval). The turns add up to the launch's work items, the interval is the same
    in every row and matches the offered rate, and a launch paced far below the link's rate keeps its schedule:
    it runs no longer than allotted (plus its last item) and almost no turn begins late."""
    cfg = W.C2_LLAMA8B_SWAP_OUT.scaled(layers=4, dev_blocks=64, host_blocks=64, n_blocks=48)
    bb = cfg.block_bytes
    cpu = [W.as_bytes(p).clone() for p in _cpu_planes(cfg, cfg.dev_blocks)]
    dev = [p.to(DEV) for p in cpu]
    src_ids, dst_ids = W.block_table(cfg, src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
    pairs = W.pairs_tensor(src_ids, dst_ids).to(DEV)
    dtab = ptr_table(dev)
    pool, host = _host_pool(memory, cfg, cfg.host_blocks, fill=0x22)
    grid, pace_mbps = 12, 20000                       # the beside-compute shape: 12 workgroups x 1 vector per lane, at 20 GB/s
    report = torch.full((grid, 8), -1, dtype=torch.int64, device=DEV)
    announce("pace report: %d planes x %d blocks paced at %d MB/s" % (cfg.planes, src_ids.numel(), pace_mbps))
    with capi.thread_tuning({capi.KNOB_SWAP_PACE_MBPS: pace_mbps, capi.KNOB_PACE_REPORT: report.data_ptr()}):
        capi.check(capi.swap_blocks(host_ptr_table(host).data_ptr(), dtab.data_ptr(), pairs.data_ptr(), cfg.planes,
                                    src_ids.numel(), bb, bb, bb, cfg.dev_blocks, cfg.host_blocks, 0, stream_handle(),
                                    capi.SWAP_DST_HOST | capi.SWAP_BESIDE_COMPUTE))
    torch.cuda.synchronize()
    for p in range(cfg.planes):
        want = torch.full((cfg.host_blocks, bb), 0x22, dtype=torch.uint8)
        O.torch_swap_blocks(want, cpu[p], src_ids, dst_ids)
        assert torch.equal(host[p], want), "plane %d" % p
    rows = report.cpu()
    ran, allotted, turns, late, worst, interval_q8 = (rows[:, i] for i in range(6))
    items = cfg.planes * src_ids.numel() * (bb // 4096)            # one 4 KiB chunk per work item
    assert int(turns.sum()) == items, (int(turns.sum()), items)
    assert bool((rows[:, 6:] == 0).all())
    assert int(interval_q8.min()) == int(interval_q8.max()) > 0
    ticks_per_item = float(interval_q8[0]) / 256.0 / grid          # 100 MHz ticks the launch allots to one item
    assert abs(ticks_per_item - 4096 / (pace_mbps * 1e6) * 1e8) < 0.05 * ticks_per_item, ticks_per_item
    # a third of the link's rate leaves room for whatever else the machine does meanwhile: the bounds are generous
    assert bool((ran <= allotted + allotted // 10 + 2 * interval_q8 // 256).all()), (ran.tolist(), allotted.tolist())
    assert int(late.sum()) <= items // 10, (int(late.sum()), items)
    assert capi.get_tuning(capi.KNOB_PACE_REPORT) == 0             # the override ended with the block


def test_pace_set_between_launches_keeps_its_account(memory):
    """A paced throughput-mode swap-out (HFK_KNOB_THROUGHPUT_PACE_PERMILLE != 0) ends by settling, in eight words the
    library keeps on the device, the factor the next such launch applies to its interval. Every launch is counted,
    the account of a finished launch is cleared, the factor stays within its bounds and moves the way the late turns
    say; with HFK_KNOB_ADAPTIVE_PACE off, and for a swap marked HFK_SWAP_BESIDE_COMPUTE, the words are left alone.
    The bytes are right throughout."""
    cfg = W.C2_LLAMA8B_SWAP_OUT.scaled(layers=8, dev_blocks=160, host_blocks=160, n_blocks=128)   # 64 MiB per launch
    bb = cfg.block_bytes
    cpu = [W.as_bytes(p).clone() for p in _cpu_planes(cfg, cfg.dev_blocks)]
    dev = [p.to(DEV) for p in cpu]
    src_ids, dst_ids = W.block_table(cfg, src_blocks=cfg.dev_blocks, dst_blocks=cfg.host_blocks)
    pairs = W.pairs_tensor(src_ids, dst_ids).to(DEV)
    dtab = ptr_table(dev)
    pool, host = _host_pool(memory, cfg, cfg.host_blocks, fill=0x33)
    htab = host_ptr_table(host)
    assert cfg.planes * src_ids.numel() * bb >= 64 << 20
    announce("pace set between launches: %d planes x %d blocks = %d MiB per launch" % (cfg.planes, src_ids.numel(),
                                                                                      cfg.planes * src_ids.numel() * bb >> 20))

    def launch(flags):
        capi.check(capi.swap_blocks(htab.data_ptr(), dtab.data_ptr(), pairs.data_ptr(), cfg.planes, src_ids.numel(), bb, bb, bb,
                                    cfg.dev_blocks, cfg.host_blocks, 0, stream_handle(), flags))

    before = capi.pace_state()
    with capi.thread_tuning({capi.KNOB_THROUGHPUT_PACE_PERMILLE: 500}):      # far under the link's limit: no turn is late
        for _ in range(6):
            launch(capi.SWAP_DST_HOST)
        after = capi.pace_state()
        assert after[5] == before[5] + 6, (before, after)
        assert after[1:5] == [0, 0, 0, 0], after
        assert 61000 <= after[0] <= 68157, after
        assert after[0] < (before[0] or 65536) or after[0] == 61000, (before, after)    # few late turns: the next interval is shorter
        assert after[6] < 3604, after
        launch(capi.SWAP_DST_HOST | capi.SWAP_BESIDE_COMPUTE)                # its pace is fixed: no account kept
        with capi.thread_tuning({capi.KNOB_THROUGHPUT_PACE_PERMILLE: 500, capi.KNOB_ADAPTIVE_PACE: 0}):
            launch(capi.SWAP_DST_HOST)
        assert capi.pace_state() == after
    launch(capi.SWAP_DST_HOST)                                                # the default is unpaced: nothing to settle
    assert capi.pace_state() == after
    # Paced launches of different grids that overlap on two streams may settle on each other's counts: the account
    # stays bounded and keeps being cleared, the factor stays within its bounds, and the bytes depend on none of it.
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    for _ in range(4):
        with capi.thread_tuning({capi.KNOB_THROUGHPUT_PACE_PERMILLE: 700}):
            launch(capi.SWAP_DST_HOST)
        with torch.cuda.stream(side), capi.thread_tuning({capi.KNOB_THROUGHPUT_PACE_PERMILLE: 700,
                                                          capi.KNOB_PACED_WORKGROUPS: 12}):
            launch(capi.SWAP_DST_HOST)
    torch.cuda.current_stream().wait_stream(side)
    with capi.thread_tuning({capi.KNOB_THROUGHPUT_PACE_PERMILLE: 700}):
        launch(capi.SWAP_DST_HOST)
    mixed = capi.pace_state()
    assert mixed[3] < 12 and mixed[5] > after[5] and 61000 <= mixed[0] <= 68157, (after, mixed)
    for p in range(cfg.planes):
        want = torch.full((cfg.host_blocks, bb), 0x33, dtype=torch.uint8)
        O.torch_swap_blocks(want, cpu[p], src_ids, dst_ids)
        assert torch.equal(host[p], want), "plane %d" % p


# ---------------------------------------------------------------------------
# edge cases
# ---------------------------------------------------------------------------
def test_empty_and_out_of_range():
    announce("edge: empty inputs and out-of-range ids")
    table = torch.arange(64 * 32, dtype=torch.int32, device=DEV).view(64, 32)        # 128-byte rows
    dst = torch.full((6, 32), -1, dtype=torch.int32, device=DEV)
    ids = torch.tensor([5, -1, 63, 64, 0, 1 << 40], dtype=torch.int64, device=DEV)
    gather_rows(table, dst, ids, 128, table_rows=64)
    torch.cuda.synchronize()
    got = dst.cpu()
    assert torch.equal(got[0], table[5].cpu()) and torch.equal(got[2], table[63].cpu()) and torch.equal(got[4], table[0].cpu())
    assert (got[1] == -1).all() and (got[3] == -1).all() and (got[5] == -1).all()
    empty = torch.zeros(0, dtype=torch.int64, device=DEV)
    assert capi.gather_rows(table.data_ptr(), dst.data_ptr(), empty.data_ptr(), True, 0, 128, 64, 0, stream_handle()) == 0
    torch.ops.pcie_through.gather(table, dst, empty)
    # swap: pairs with an out-of-range side are skipped, the rest copied
    src = [torch.randint(0, 255, (8, 4096), dtype=torch.uint8, device=DEV)]
    dstp = [torch.zeros(8, 4096, dtype=torch.uint8, device=DEV)]
    pairs = torch.tensor([[1, 2], [8, 3], [2, -1], [3, 8], [4, 5]], dtype=torch.int64, device=DEV)
    swap(ptr_table(dstp), ptr_table(src), pairs, 1, 4096, src_blocks=8, dst_blocks=8)
    torch.cuda.synchronize()
    d, s = dstp[0].cpu(), src[0].cpu()
    assert torch.equal(d[2], s[1]) and torch.equal(d[5], s[4])
    assert (d[[0, 1, 3, 4, 6, 7]] == 0).all()


@pytest.mark.parametrize("row_bytes", [1, 7, 33, 100, 1000, 4095, 4099, 8212, 65536 + 4])
def test_ragged_row_sizes(row_bytes):
    announce("edge: ragged rows of %d bytes" % row_bytes)
    rs = np.random.RandomState(row_bytes)
    table = rs.randint(0, 256, size=(97, row_bytes)).astype(np.uint8)
    ids = rs.randint(0, 97, size=53).astype(np.int64)
    t_dev, i_dev = torch.from_numpy(table).to(DEV), torch.from_numpy(ids).to(DEV)
    dst = torch.zeros(53, row_bytes, dtype=torch.uint8, device=DEV)
    gather_rows(t_dev, dst, i_dev, row_bytes, table_rows=97)
    torch.cuda.synchronize()
    assert np.array_equal(dst.cpu().numpy(), O.c_gather_rows(table, ids))


def test_results_independent_of_tuning_and_grid():
    announce("edge: every unroll / non-temporal / grid setting gives the same bytes")
    cfg = W.C4_MLA_ROUNDTRIP.scaled(layers=2, dev_blocks=16, host_blocks=16, n_blocks=9)
    cpu = _cpu_planes(cfg, cfg.dev_blocks)
    dev = [p.to(DEV) for p in cpu]
    src_ids, dst_ids = W.block_table(cfg, src_blocks=16, dst_blocks=16)
    pairs = W.pairs_tensor(src_ids, dst_ids).to(DEV)
    want = []
    for p in range(cfg.planes):
        w = torch.zeros(16, cfg.block_bytes, dtype=torch.uint8)
        O.torch_swap_blocks(w, W.as_bytes(cpu[p]), src_ids, dst_ids)
        want.append(w)
    for unroll in (1, 2, 4, 8, 16):
        for nt in (0, 1, 2, 3):
            for wgs in (0, 1, 5, 100000):
                out = [torch.zeros(16, cfg.block_bytes, dtype=torch.uint8, device=DEV) for _ in range(cfg.planes)]
                with capi.thread_tuning({capi.KNOB_SWAP_UNROLL: unroll, capi.KNOB_UNROLL: unroll, capi.KNOB_NONTEMPORAL: nt}):
                    swap(ptr_table(out), ptr_table(dev), pairs, cfg.planes, cfg.block_bytes, workgroups=wgs)
                torch.cuda.synchronize()
                for p in range(cfg.planes):
                    assert torch.equal(out[p].cpu(), want[p]), (unroll, nt, wgs, p)
    assert capi.get_tuning(capi.KNOB_NONTEMPORAL) == 3


def test_strided_planes():
    announce("edge: block stride larger than block bytes on both sides")
    src = torch.randint(0, 255, (10, 3, 2048), dtype=torch.uint8, device=DEV)    # use [:, 0, :] -> stride 6144
    dst = torch.zeros(12, 2, 2048, dtype=torch.uint8, device=DEV)                # use [:, 1, :] -> stride 4096
    pairs = torch.tensor([[0, 11], [9, 0], [4, 4]], dtype=torch.int64, device=DEV)
    dst_tab = torch.tensor([dst[0, 1].data_ptr()], dtype=torch.int64, device=DEV)
    src_tab = torch.tensor([src[0, 0].data_ptr()], dtype=torch.int64, device=DEV)
    swap(dst_tab, src_tab, pairs, 1, 2048, src_stride=6144, dst_stride=4096, src_blocks=10, dst_blocks=12)
    torch.cuda.synchronize()
    d, s = dst.cpu(), src.cpu()
    assert torch.equal(d[11, 1], s[0, 0]) and torch.equal(d[0, 1], s[9, 0]) and torch.equal(d[4, 1], s[4, 0])
    assert (d[:, 0] == 0).all() and d[:, 1].sum() == s[[0, 9, 4], 0].sum()


def test_python_swap_wrapper_names_the_host_side_by_itself(memory):
    """pcie_through.swap_blocks: the op with its flags read off tables that plane_pointer_table built."""
    announce("pcie_through.swap_blocks wrapper: out and back, flags inferred from the tables")
    planes, blocks, bb, n = 3, 40, 32768, 12
    gen = torch.Generator().manual_seed(321)
    dev = [torch.randint(0, 256, (blocks, bb), dtype=torch.uint8, generator=gen).to(DEV) for _ in range(planes)]
    pool = memory.alloc_numa_pinned_tensor(planes * blocks * bb)
    host = list(pool.view(torch.uint8).view(planes, blocks, bb).unbind(0))
    dtab, htab = pcie_through.plane_pointer_table(dev, DEV), pcie_through.plane_pointer_table(host, DEV)
    assert htab.hfk_planes_in_host is True and dtab.hfk_planes_in_host is False
    src, dst = torch.randperm(blocks, generator=gen)[:n], torch.randperm(blocks, generator=gen)[:n]
    before = [d.cpu() for d in dev]
    pcie_through.swap_blocks(htab, dtab, torch.stack([src, dst], 1).to(DEV), bb, bb, bb, blocks, blocks)
    back = torch.roll(src, 1)
    pcie_through.swap_blocks(dtab, htab, torch.stack([dst, back], 1).to(DEV), bb, bb, bb, blocks, blocks,
                             beside_compute=True)
    torch.cuda.synchronize()
    for p in range(planes):
        assert torch.equal(host[p][dst], before[p][src]), "swap-out through the wrapper"
        want = before[p].clone()
        want[back] = before[p][src]
        assert torch.equal(dev[p].cpu(), want), "swap-in through the wrapper"
    # the note belongs to the table object: another tensor over the same storage carries none, and names no side
    alias = htab.view(-1)
    assert getattr(alias, "hfk_planes_in_host", None) is None
    for p in range(planes):
        host[p][dst] = 0
    pcie_through.swap_blocks(alias, dtab, torch.stack([back, dst], 1).to(DEV), bb, bb, bb, blocks, blocks)
    torch.cuda.synchronize()
    for p in range(planes):
        assert torch.equal(host[p][dst], dev[p].cpu()[back]), "swap-out through a table without a note"


@pytest.mark.parametrize("args", [(), ("3", "40", "4112", "20"), ("64", "128", "32768", "64")],
                         ids=["defaults", "odd_block_size", "config2_planes"])
def test_plain_c_client_runs_the_swap_path(args):
    """The C-ABI bound from C99 with no torch in the process: swap-out, swap-in, staged swap and gather,
    each checked byte for byte inside the client against the pattern it wrote."""
    import subprocess
    from heterofusedkernels_amd import _build

    announce("plain-C client %s" % (" ".join(args) or "(defaults)"))
    proc = subprocess.run([_build.C_CLIENT, *args], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=100)
    assert proc.returncode == 0, (proc.returncode, proc.stdout[-2000:], proc.stderr[-2000:])
    assert proc.stdout.strip().endswith("hfk_c_client: OK")
