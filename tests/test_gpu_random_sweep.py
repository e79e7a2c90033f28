"""Seeded random sweep of every C-ABI entry point against the C oracle: odd block sizes,
strides larger than a block, bases off every alignment, planes on either side of the PCIe
link, int32 and int64 ids, out-of-range entries, random grid bounds. Each case checks the
whole destination buffer, gaps between strided blocks included."""
import ctypes
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
DEV = "cuda"
BLOCK_BYTES = [1, 3, 16, 48, 100, 528, 4096, 4112, 12288, 32768, 33001]
PADS = [0, 0, 16, 5, 4096]
OFFSETS = [0, 0, 16, 4, 1, 7]
CASES = 40
# HFK_SWEEP_SEED_OFFSET=k shifts every seed by k: other cases of the same sweep, for longer one-off runs.
SEED_OFFSET = int(os.environ.get("HFK_SWEEP_SEED_OFFSET", "0"))


class Arena:
    """A byte buffer on one side of the link, its numpy mirror and the address a kernel uses."""

    def __init__(self, nbytes, on_host, rng, fill=None):
        nbytes = max(int(nbytes), 1)
        init = rng.integers(0, 256, nbytes, dtype=np.uint8) if fill is None else np.full(nbytes, fill, np.uint8)
        self.on_host = on_host
        if on_host:
            self.t = memory.alloc_numa_pinned_tensor(nbytes).view(torch.uint8)
            self.t.copy_(torch.from_numpy(init))
            self.addr = memory.get_device_ptr(self.t.data_ptr())
            self.host_addr = self.t.data_ptr()
            assert self.addr != 0
        else:
            self.t = torch.from_numpy(init).to(DEV)
            self.addr = self.t.data_ptr()
        self.before = init

    def now(self):
        return self.t.cpu().numpy().copy()


def _planes(base, offset, n_planes, blocks, stride):
    """addresses of n_planes strided planes laid out back to back from base + offset"""
    return [base + offset + p * blocks * stride for p in range(n_planes)]


def _view(buf, offset, plane, blocks, stride, bb):
    """[blocks, bb] strided numpy view of one plane inside a flat byte buffer"""
    start = offset + plane * blocks * stride
    return np.lib.stride_tricks.as_strided(buf[start:], shape=(blocks, bb), strides=(stride, 1), writeable=True)


def _table(addresses):
    return torch.tensor(addresses, dtype=torch.int64).to(DEV)


def _pairs(rng, n, src_blocks, dst_blocks, with_bad):
    """n (src, dst) pairs with distinct in-range destinations, plus out-of-range rows when asked"""
    dst = rng.permutation(dst_blocks)[:n]
    src = rng.integers(0, src_blocks, dst.shape[0])
    pairs = np.stack([src, dst], 1).astype(np.int64).reshape(-1, 2)
    if with_bad:
        bad = np.array([[-1, 0], [src_blocks, 0], [0, dst_blocks], [0, -3], [2 ** 40, 0]], dtype=np.int64)
        pairs = np.concatenate([pairs, bad[rng.integers(0, len(bad), 3)]])
        pairs = pairs[rng.permutation(pairs.shape[0])]
    ok = (pairs[:, 0] >= 0) & (pairs[:, 0] < src_blocks) & (pairs[:, 1] >= 0) & (pairs[:, 1] < dst_blocks)
    return pairs, pairs[ok]


def _expect_swap(dst_buf, src_buf, doff, soff, n_planes, dst_blocks, src_blocks, dstride, sstride, bb, valid):
    want = dst_buf.copy()
    for p in range(n_planes):
        d = np.ascontiguousarray(_view(want, doff, p, dst_blocks, dstride, bb))
        s = np.ascontiguousarray(_view(src_buf, soff, p, src_blocks, sstride, bb))
        O.c_swap_blocks([d], [s], valid)
        _view(want, doff, p, dst_blocks, dstride, bb)[:] = d
    return want


@pytest.mark.parametrize("seed", range(4))
def test_random_swap_blocks(seed):
    rng = np.random.default_rng(1000 + seed + 17 * SEED_OFFSET)
    for case in range(CASES):
        n_planes = int(rng.integers(1, 9))
        src_blocks, dst_blocks = int(rng.integers(1, 40)), int(rng.integers(1, 40))
        bb = int(rng.choice(BLOCK_BYTES))
        sstride, dstride = bb + int(rng.choice(PADS)), bb + int(rng.choice(PADS))
        soff, doff = int(rng.choice(OFFSETS)), int(rng.choice(OFFSETS))
        src_host, dst_host = [(False, False), (False, True), (True, False)][int(rng.integers(0, 3))]
        n = int(rng.integers(0, dst_blocks + 1))
        with_bad = bool(rng.integers(0, 2))
        wg = int(rng.choice([0, 0, 1, 3, 1000]))
        # the flags only choose the launch shape (grid, pacing): any value gives the same bytes
        flags = int(rng.choice([0, capi.SWAP_BESIDE_COMPUTE, capi.SWAP_BESIDE_COMPUTE | capi.SWAP_DST_HOST,
                                capi.SWAP_BESIDE_COMPUTE | capi.SWAP_SRC_HOST, capi.SWAP_DST_HOST, capi.SWAP_SRC_HOST]))
        announce("random swap seed %d case %d: planes %d, blocks %d->%d, %d B (strides %d/%d, offsets %d/%d), "
                 "src_host %s dst_host %s, %d pairs, bad %s, workgroups %d, flags %d"
                 % (seed, case, n_planes, src_blocks, dst_blocks, bb, sstride, dstride, soff, doff, src_host, dst_host,
                    n, with_bad, wg, flags))
        src = Arena(soff + n_planes * src_blocks * sstride, src_host, rng)
        dst = Arena(doff + n_planes * dst_blocks * dstride, dst_host, rng)
        pairs, valid = _pairs(rng, n, src_blocks, dst_blocks, with_bad)
        pairs_d = torch.from_numpy(pairs).to(DEV)
        stab = _table(_planes(src.addr, soff, n_planes, src_blocks, sstride))
        dtab = _table(_planes(dst.addr, doff, n_planes, dst_blocks, dstride))
        capi.check(capi.swap_blocks(dtab.data_ptr(), stab.data_ptr(), pairs_d.data_ptr() if pairs.shape[0] else None,
                                    n_planes, pairs.shape[0], bb, sstride, dstride, src_blocks, dst_blocks, wg,
                                    stream_handle(), flags), "hfk_swap_blocks")
        torch.cuda.synchronize()
        want = _expect_swap(dst.before, src.before, doff, soff, n_planes, dst_blocks, src_blocks, dstride, sstride, bb, valid)
        assert np.array_equal(dst.now(), want)
        assert np.array_equal(src.now(), src.before), "source changed"


def _pool_side(to_packed, packed_host):
    """The flag that says, truthfully, where the packed pool of a table transfer lives."""
    if to_packed:
        return capi.SWAP_DST_HOST if packed_host else capi.SWAP_DST_DEVICE
    return capi.SWAP_SRC_HOST if packed_host else capi.SWAP_SRC_DEVICE


@pytest.mark.parametrize("seed", range(4))
def test_random_gather_rows_and_blocks(seed):
    rng = np.random.default_rng(2000 + seed + 17 * SEED_OFFSET)
    for case in range(CASES):
        rows = int(rng.integers(1, 200))
        rb = int(rng.choice(BLOCK_BYTES + [7, 1000, 8212]))
        toff, doff = int(rng.choice(OFFSETS)), int(rng.choice(OFFSETS))
        table_host = bool(rng.integers(0, 2))
        n = int(rng.integers(0, 300))
        id_dtype = np.int64 if rng.integers(0, 2) else np.int32
        with_bad = bool(rng.integers(0, 2))
        wg = int(rng.choice([0, 0, 1, 5]))
        announce("random gather_rows seed %d case %d: %d rows of %d B (offsets %d/%d), host table %s, %d ids %s, bad %s, "
                 "workgroups %d" % (seed, case, rows, rb, toff, doff, table_host, n, id_dtype.__name__, with_bad, wg))
        table = Arena(toff + rows * rb, table_host, rng)
        dst = Arena(doff + n * rb, False, rng)
        ids = rng.integers(0, rows, n).astype(id_dtype)
        if with_bad and n:
            ids[rng.integers(0, n, 3)] = np.array([-1, rows, rows + 5], dtype=id_dtype)
        ids_d = torch.from_numpy(ids).to(DEV) if n else torch.zeros(1, dtype=torch.int64, device=DEV)
        # what the caller may say about the table: nothing, or the truth (the launch shape follows, never the bytes)
        side = int(rng.choice([0, capi.SWAP_SRC_HOST if table_host else capi.SWAP_SRC_DEVICE]))
        capi.check(capi.gather_rows(table.addr + toff, dst.addr + doff, ids_d.data_ptr(), id_dtype is np.int64, n, rb,
                                    rows, wg, stream_handle(), side), "hfk_gather_rows")
        torch.cuda.synchronize()
        want = dst.before.copy()
        ok = (ids >= 0) & (ids < rows)
        got_rows = O.c_gather_rows(table.before[toff:toff + rows * rb].reshape(rows, rb), ids[ok])
        want[doff:doff + n * rb].reshape(n, rb)[ok] = got_rows
        assert np.array_equal(dst.now(), want)

        # the same ids over several strided planes: hfk_gather_blocks
        n_planes = int(rng.integers(1, 7))
        stride = rb + int(rng.choice(PADS))
        announce("random gather_blocks seed %d case %d: %d planes, stride %d" % (seed, case, n_planes, stride))
        src = Arena(toff + n_planes * rows * stride, table_host, rng)
        out = Arena(doff + n_planes * n * rb, False, rng)
        ids64 = torch.from_numpy(ids.astype(np.int64)).to(DEV) if n else torch.zeros(1, dtype=torch.int64, device=DEV)
        stab = _table(_planes(src.addr, toff, n_planes, rows, stride))
        dtab = _table(_planes(out.addr, doff, n_planes, n, rb))
        gflags = int(rng.choice([0, 0, capi.SWAP_SRC_HOST, capi.SWAP_SRC_HOST | capi.SWAP_BESIDE_COMPUTE]))   # launch shape only
        capi.check(capi.gather_blocks(dtab.data_ptr(), stab.data_ptr(), ids64.data_ptr(), n_planes, n, rb, stride, rows,
                                      wg, stream_handle(), gflags), "hfk_gather_blocks")
        torch.cuda.synchronize()
        want = out.before.copy()
        for p in range(n_planes):
            plane = np.ascontiguousarray(_view(src.before, toff, p, rows, stride, rb))
            start = doff + p * n * rb
            want[start:start + n * rb].reshape(n, rb)[ok] = O.c_gather_rows(plane, ids[ok])
        assert np.array_equal(out.now(), want)


@pytest.mark.parametrize("seed", range(4))
def test_random_block_table_transfer(seed):
    rng = np.random.default_rng(3000 + seed + 17 * SEED_OFFSET)
    for case in range(CASES):
        T, L, H = int(rng.integers(1, 40)), int(rng.integers(1, 6)), int(rng.integers(1, 5))
        D, e = int(rng.choice([1, 3, 8, 16, 24, 64, 128])), int(rng.choice([1, 2, 4]))
        packed_blocks, dev_blocks = int(rng.integers(1, 12)), int(rng.integers(1, 12))
        to_packed = bool(rng.integers(0, 2))
        packed_host = bool(rng.integers(0, 2))
        poff = int(rng.choice(OFFSETS))
        wg = int(rng.choice([0, 0, 1, 7]))
        layer_bytes, block_bytes = H * T * D * e, T * L * H * D * e
        n_dst = packed_blocks if to_packed else dev_blocks
        n = int(rng.integers(0, n_dst + 1))
        announce("random table transfer seed %d case %d: T%d L%d H%d D%d e%d, blocks %d/%d, to_packed %s, host pool %s, "
                 "offset %d, %d pairs, workgroups %d"
                 % (seed, case, T, L, H, D, e, packed_blocks, dev_blocks, to_packed, packed_host, poff, n, wg))
        packed = Arena(poff + packed_blocks * block_bytes, packed_host, rng)
        layers = Arena(L * dev_blocks * layer_bytes, False, rng)
        if to_packed:      # pairs are (packed_block, dev_block); the destination side must be distinct
            pb, db = rng.permutation(packed_blocks)[:n], rng.integers(0, dev_blocks, n)
        else:
            pb, db = rng.integers(0, packed_blocks, n), rng.permutation(dev_blocks)[:n]
        pairs = np.stack([pb, db], 1).astype(np.int64).reshape(-1, 2)
        bad = np.array([[-1, 0], [packed_blocks, 0], [0, dev_blocks]], dtype=np.int64)
        pairs_all = np.concatenate([pairs, bad[rng.integers(0, 3, 2)]]) if rng.integers(0, 2) else pairs
        pairs_d = torch.from_numpy(pairs_all).to(DEV) if pairs_all.shape[0] else None
        lptrs = _table([layers.addr + l * dev_blocks * layer_bytes for l in range(L)])
        capi.check(capi.multi_layer_block_table_transfer(
            lptrs.data_ptr(), layer_bytes, packed.addr + poff, block_bytes, pairs_d.data_ptr() if pairs_d is not None else None,
            pairs_all.shape[0], packed_blocks, dev_blocks, T, L, H, D, e, int(to_packed), wg, stream_handle(),
            int(rng.choice([0, capi.SWAP_BESIDE_COMPUTE])) | int(rng.choice([0, _pool_side(to_packed, packed_host)]))),
            "hfk_multi_layer_block_table_transfer")
        torch.cuda.synchronize()
        want_layers = layers.before.copy().reshape(L, dev_blocks, layer_bytes)
        want_packed = packed.before.copy()
        pk = np.ascontiguousarray(want_packed[poff:poff + packed_blocks * block_bytes].reshape(packed_blocks, block_bytes))
        O.c_multi_layer_block_table_transfer(want_layers, pk, pairs, T, L, H, D, e, to_packed)
        want_packed[poff:poff + packed_blocks * block_bytes] = pk.reshape(-1)
        assert np.array_equal(layers.now(), want_layers.reshape(-1))
        assert np.array_equal(packed.now(), want_packed)


@pytest.mark.parametrize("seed", range(3))
def test_random_duplex_and_staged(seed):
    rng = np.random.default_rng(4000 + seed + 17 * SEED_OFFSET)
    for case in range(CASES):
        n_planes = int(rng.integers(1, 7))
        dev_blocks, host_blocks = int(rng.integers(4, 40)), int(rng.integers(4, 40))
        bb = int(rng.choice(BLOCK_BYTES))
        dstride, hstride = bb + int(rng.choice(PADS)), bb + int(rng.choice(PADS))
        doff, hoff = int(rng.choice(OFFSETS)), int(rng.choice(OFFSETS))
        wg = int(rng.choice([0, 0, 1, 3]))
        most = min(dev_blocks, host_blocks) // 2
        n_out, n_in = int(rng.integers(0, most + 1)), int(rng.integers(0, most + 1))
        announce("random duplex seed %d case %d: %d planes, blocks %d/%d, %d B (strides %d/%d, offsets %d/%d), out %d in %d, "
                 "workgroups %d" % (seed, case, n_planes, dev_blocks, host_blocks, bb, dstride, hstride, doff, hoff, n_out,
                                    n_in, wg))
        dev = Arena(doff + n_planes * dev_blocks * dstride, False, rng)
        host = Arena(hoff + n_planes * host_blocks * hstride, True, rng)
        dperm, hperm = rng.permutation(dev_blocks), rng.permutation(host_blocks)
        out_pairs = np.stack([dperm[:n_out], hperm[:n_out]], 1).astype(np.int64).reshape(-1, 2)
        in_pairs = np.stack([hperm[n_out:n_out + n_in], dperm[n_out:n_out + n_in]], 1).astype(np.int64).reshape(-1, 2)
        po = torch.from_numpy(out_pairs).to(DEV) if n_out else None
        pi = torch.from_numpy(in_pairs).to(DEV) if n_in else None
        dtab = _table(_planes(dev.addr, doff, n_planes, dev_blocks, dstride))
        htab = _table(_planes(host.addr, hoff, n_planes, host_blocks, hstride))
        om = capi.BlockMove(htab.data_ptr(), dtab.data_ptr(), po.data_ptr() if n_out else None, n_out, dstride, hstride,
                            dev_blocks, host_blocks)
        im = capi.BlockMove(dtab.data_ptr(), htab.data_ptr(), pi.data_ptr() if n_in else None, n_in, hstride, dstride,
                            host_blocks, dev_blocks)
        capi.check(capi.swap_blocks_duplex(om, im, n_planes, bb, wg, stream_handle(),
                                           int(rng.choice([0, capi.SWAP_BESIDE_COMPUTE]))), "hfk_swap_blocks_duplex")
        torch.cuda.synchronize()
        want_host = _expect_swap(host.before, dev.before, hoff, doff, n_planes, host_blocks, dev_blocks, hstride, dstride, bb,
                                 out_pairs)
        want_dev = _expect_swap(dev.before, host.before, doff, hoff, n_planes, dev_blocks, host_blocks, dstride, hstride, bb,
                                in_pairs)
        assert np.array_equal(host.now(), want_host), "host side"
        assert np.array_equal(dev.now(), want_dev), "device side"

        # staged, both directions, on fresh buffers of the same geometry
        n = int(rng.integers(1, min(dev_blocks, host_blocks) + 1))
        dev_ids = rng.permutation(dev_blocks)[:n].astype(np.int64)
        first = int(rng.integers(0, host_blocks - n + 1))
        host_ids = np.arange(first, first + n, dtype=np.int64)
        if rng.integers(0, 2):
            host_ids = rng.permutation(host_blocks)[:n].astype(np.int64)          # scattered slots
        to_host = bool(rng.integers(0, 2))
        bad_dev = bool(rng.integers(0, 2))
        if bad_dev:         # a device id out of range: skipped on the way in, zeros in the host slot on the way out
            dev_ids[rng.integers(0, n, 2)] = np.array([-1, dev_blocks], dtype=np.int64)[rng.integers(0, 2, 2)]
        ok = (dev_ids >= 0) & (dev_ids < dev_blocks)
        static = bool(rng.integers(0, 2)) and n_planes * n * bb <= capi.STATIC_STAGING_BYTES
        announce("random staged seed %d case %d: %d blocks, to_host %s, bad device ids %s, library staging %s"
                 % (seed, case, n, to_host, bad_dev, static))
        dev2 = Arena(doff + n_planes * dev_blocks * dstride, False, rng)
        host2 = Arena(hoff + n_planes * host_blocks * hstride, True, rng)
        staging = torch.full((n_planes * n * bb,), 0xC3, dtype=torch.uint8, device=DEV)
        dtab2 = _table(_planes(dev2.addr, doff, n_planes, dev_blocks, dstride))
        host_addrs = (ctypes.c_void_p * n_planes)(*_planes(host2.host_addr, hoff, n_planes, host_blocks, hstride))
        ids_d = torch.from_numpy(dev_ids).to(DEV)
        if static:
            capi.check(capi.swap_blocks_staged_static(dtab2.data_ptr(), host_addrs, ids_d.data_ptr(), host_ids.ctypes.data,
                                                      n_planes, n, bb, dstride, hstride, dev_blocks, host_blocks,
                                                      int(to_host), wg, stream_handle()), "hfk_swap_blocks_staged_static")
        else:
            capi.check(capi.swap_blocks_staged(dtab2.data_ptr(), host_addrs, ids_d.data_ptr(), host_ids.ctypes.data,
                                               n_planes, n, bb, dstride, hstride, dev_blocks, host_blocks,
                                               staging.data_ptr(), int(to_host), wg, stream_handle()),
                       "hfk_swap_blocks_staged")
        torch.cuda.synchronize()
        if to_host:
            want = _expect_swap(host2.before, dev2.before, hoff, doff, n_planes, host_blocks, dev_blocks, hstride, dstride,
                                bb, np.stack([dev_ids, host_ids], 1)[ok])
            for p in range(n_planes):
                _view(want, hoff, p, host_blocks, hstride, bb)[host_ids[~ok]] = 0
            assert np.array_equal(host2.now(), want), "staged host side"
            assert np.array_equal(dev2.now(), dev2.before)
        else:
            want = _expect_swap(dev2.before, host2.before, doff, hoff, n_planes, dev_blocks, host_blocks, dstride, hstride,
                                bb, np.stack([host_ids, dev_ids], 1)[ok])
            assert np.array_equal(dev2.now(), want), "staged device side"
            assert np.array_equal(host2.now(), host2.before)


def _run_table(rng, n, blocks):
    """n distinct slots out of `blocks`: runs of 1-6 consecutive slots, in random order."""
    runs, at = [], 0
    while at < blocks:
        length = int(rng.integers(1, 7))
        if at + length > blocks:
            break
        runs.append(np.arange(at, at + length, dtype=np.int64))
        at += length + int(rng.integers(1, 3))      # a gap keeps neighbouring runs from joining up
    order = rng.permutation(len(runs))
    ids = np.concatenate([runs[i] for i in order]) if runs else np.zeros(0, dtype=np.int64)
    return ids[:n]


@pytest.mark.parametrize("seed", range(3))
def test_random_swap_blocks_auto(seed):
    """The run-splitting swap against the oracle: fragmented host slots, every threshold from "stage
    everything" to "stage nothing", with and without a staging buffer, with a buffer that holds the long runs
    only, padded strides (2-D copies per plane), planes that are not evenly spaced on the host, bad device ids."""
    rng = np.random.default_rng(5000 + seed + 17 * SEED_OFFSET)
    for case in range(CASES):
        n_planes = int(rng.integers(1, 7))
        dev_blocks, host_blocks = int(rng.integers(4, 40)), int(rng.integers(8, 60))
        bb = int(rng.choice(BLOCK_BYTES))
        dstride, hstride = bb + int(rng.choice(PADS)), bb + int(rng.choice(PADS))
        doff, hoff = int(rng.choice(OFFSETS)), int(rng.choice(OFFSETS))
        host_ids = _run_table(rng, int(rng.integers(1, min(dev_blocks, host_blocks) + 1)), host_blocks)
        n = host_ids.shape[0]
        dev_ids = rng.permutation(dev_blocks)[:n].astype(np.int64)
        to_host = bool(rng.integers(0, 2))
        bad_dev = bool(rng.integers(0, 2))
        if bad_dev:
            dev_ids[rng.integers(0, n, 2)] = np.array([-1, dev_blocks], dtype=np.int64)[rng.integers(0, 2, 2)]
        ok = (dev_ids >= 0) & (dev_ids < dev_blocks)
        min_run = int(rng.choice([0, 1, 2, 3, 4, 7, 5000]))
        # 0: full arguments, 1: no staging, 2: staging one byte short of the whole table (used compactly if the long
        # runs and their slot table fit), 3: no host arrays, 4: staging of exactly the compact size
        how = int(rng.integers(0, 5))
        if how == 4:
            min_run = int(rng.choice([2, 3, 4]))
        flags = int(rng.choice([0, capi.SWAP_BESIDE_COMPUTE]))
        plane_gap = int(rng.choice([0, 0, 64]))       # != 0: the last plane sits off the even spacing
        announce("random auto seed %d case %d: %d planes, blocks %d/%d, %d B (strides %d/%d, offsets %d/%d), %d pairs, "
                 "to_host %s, bad device ids %s, min_run %d, how %d, flags %d, plane gap %d"
                 % (seed, case, n_planes, dev_blocks, host_blocks, bb, dstride, hstride, doff, hoff, n, to_host, bad_dev,
                    min_run, how, flags, plane_gap))
        dev = Arena(doff + n_planes * dev_blocks * dstride, False, rng)
        host = Arena(hoff + n_planes * host_blocks * hstride + plane_gap, True, rng)
        dev_addrs = _planes(dev.addr, doff, n_planes, dev_blocks, dstride)
        host_offsets = [hoff + p * host_blocks * hstride + (plane_gap if p == n_planes - 1 and p > 0 else 0)
                        for p in range(n_planes)]
        dtab = _table(dev_addrs)
        htab = _table([host.addr + o for o in host_offsets])
        host_addrs = (ctypes.c_void_p * n_planes)(*[host.host_addr + o for o in host_offsets])
        pairs = np.stack([dev_ids, host_ids] if to_host else [host_ids, dev_ids], 1).astype(np.int64)
        pairs_d = torch.from_numpy(pairs).to(DEV)
        guard = 4096
        staging = torch.full((max(n_planes * n * bb, 1) + 16 * n + 256 + guard,), 0xC3, dtype=torch.uint8, device=DEV)
        staging_bytes = n_planes * n * bb if how != 2 else max(n_planes * n * bb - 1, 0)
        if how == 4:      # the blocks of the long runs, rounded up to 256 bytes, and 16 bytes per pair for their slots
            run_len = np.ones(n, dtype=np.int64)
            starts = np.flatnonzero(np.r_[True, host_ids[1:] != host_ids[:-1] + 1])
            for first, last in zip(starts, np.r_[starts[1:], n]):
                run_len[first:last] = last - first
            long_blocks = int((run_len >= min_run).sum())
            staging_bytes = (n_planes * long_blocks * bb + 255) // 256 * 256 + 16 * n
        # every other case with the debugging check that compares the table's host column with the host array
        with capi.thread_tuning({capi.KNOB_CHECK_HOST_COLUMN: case % 2}):
            capi.check(capi.swap_blocks_auto(dtab.data_ptr(), htab.data_ptr(), host_addrs if how != 3 else None,
                                             pairs_d.data_ptr(), host_ids.ctypes.data if how != 3 else None, n_planes, n, bb,
                                             dstride, hstride, dev_blocks, host_blocks,
                                             staging.data_ptr() if how != 1 else None, staging_bytes if how != 1 else 0,
                                             int(to_host), min_run, flags, stream_handle()), "hfk_swap_blocks_auto")
        torch.cuda.synchronize()
        assert bool((staging[staging_bytes:] == 0xC3).all()), "staging was written beyond the size given"
        if how == 4 and 0 < long_blocks < n:      # the compact buffer was used, not passed over for the direct way
            assert not bool((staging[:n_planes * long_blocks * bb] == 0xC3).all()), "compact staging went unused"

        def host_view(buf, p):
            return np.lib.stride_tricks.as_strided(buf[host_offsets[p]:], shape=(host_blocks, bb), strides=(hstride, 1),
                                                   writeable=True)

        want_host, want_dev = host.before.copy(), dev.before.copy()
        for p in range(n_planes):
            d = _view(want_dev if not to_host else dev.before, doff, p, dev_blocks, dstride, bb)
            h = host_view(want_host if to_host else host.before, p)
            if to_host:
                h[host_ids[ok]] = d[dev_ids[ok]]
                h[host_ids[~ok]] = 0
            else:
                d[dev_ids[ok]] = h[host_ids[ok]]
        # the same planes through the C oracle (contiguous copies of the strided views)
        for p in range(n_planes):
            if to_host:
                chk = np.ascontiguousarray(host_view(host.before, p))
                O.c_swap_blocks([chk], [np.ascontiguousarray(_view(dev.before, doff, p, dev_blocks, dstride, bb))], pairs[ok])
                chk[host_ids[~ok]] = 0
                assert np.array_equal(chk, host_view(want_host, p))
            else:
                chk = np.ascontiguousarray(_view(dev.before, doff, p, dev_blocks, dstride, bb))
                O.c_swap_blocks([chk], [np.ascontiguousarray(host_view(host.before, p))], pairs[ok])
                assert np.array_equal(chk, _view(want_dev, doff, p, dev_blocks, dstride, bb))
        assert np.array_equal(host.now(), want_host), "host side"
        assert np.array_equal(dev.now(), want_dev), "device side"


def _pair_lists(host_ids, min_run):
    """What hfk::fill_pair_lists states: table indices of the pairs in runs of at least min_run consecutive ids,
    and of all others, each in table order and padded with -1 to the table's length."""
    n = host_ids.shape[0]
    starts = np.flatnonzero(np.r_[True, host_ids[1:] != host_ids[:-1] + 1])
    run_len = np.ones(n, dtype=np.int64)
    for first, last in zip(starts, np.r_[starts[1:], n]):
        run_len[first:last] = last - first
    is_long = run_len >= min_run
    pad = lambda a: np.r_[a, np.full(n - a.shape[0], -1)].astype(np.int64)      # noqa: E731
    return pad(np.flatnonzero(is_long)), pad(np.flatnonzero(~is_long))


@pytest.mark.parametrize("min_run", [2, 7, 64, 300, 1024])
def test_run_splitting_swap_on_a_long_table(min_run):
    """A table of 1500 pairs (six batches of the list kernel's 256) whose runs of host slots are 1 to 700 long, split
    at thresholds from 2 to 1024, out and back: the bytes against the oracle, and the two lists the call leaves
    behind its compact staging against their sequential statement."""
    rng = np.random.default_rng(9100 + min_run + 17 * SEED_OFFSET)
    n_planes, bb, dev_blocks, host_blocks = 2, 512, 2048, 6000
    lengths = [700, 1, 1, 299, 300, 2, 63, 64, 65, 1, 3]
    runs, at = [], 0
    for length in lengths:
        runs.append(np.arange(at, at + length, dtype=np.int64))
        at += length + 1 + int(rng.integers(0, 3))
    host_ids = np.concatenate([runs[i] for i in rng.permutation(len(runs))])
    n = host_ids.shape[0]
    assert n == sum(lengths) == 1499 and at <= host_blocks
    dev_ids = rng.permutation(dev_blocks)[:n].astype(np.int64)
    long_list, short_list = _pair_lists(host_ids, min_run)
    long_blocks = int((long_list >= 0).sum())
    lists_offset = (n_planes * long_blocks * bb + 255) // 256 * 256
    staging_bytes = lists_offset + 16 * n
    for to_host in (True, False):
        announce("long table, min_run %d, to_host %s: %d pairs, %d in long runs" % (min_run, to_host, n, long_blocks))
        dev = Arena(n_planes * dev_blocks * bb, False, rng)
        host = Arena(n_planes * host_blocks * bb, True, rng)
        dtab = _table(_planes(dev.addr, 0, n_planes, dev_blocks, bb))
        htab = _table(_planes(host.addr, 0, n_planes, host_blocks, bb))
        host_addrs = (ctypes.c_void_p * n_planes)(*_planes(host.host_addr, 0, n_planes, host_blocks, bb))
        pairs = np.stack([dev_ids, host_ids] if to_host else [host_ids, dev_ids], 1).astype(np.int64)
        pairs_d = torch.from_numpy(pairs).to(DEV)
        staging = torch.full((staging_bytes + 4096,), 0xC3, dtype=torch.uint8, device=DEV)
        capi.check(capi.swap_blocks_auto(dtab.data_ptr(), htab.data_ptr(), host_addrs, pairs_d.data_ptr(), host_ids.ctypes.data,
                                         n_planes, n, bb, bb, bb, dev_blocks, host_blocks, staging.data_ptr(), staging_bytes,
                                         int(to_host), min_run, capi.SWAP_BESIDE_COMPUTE, stream_handle()), "hfk_swap_blocks_auto")
        torch.cuda.synchronize()
        assert bool((staging[staging_bytes:] == 0xC3).all()), "staging was written beyond the size given"
        if 0 < long_blocks < n:      # the table is split: the call wrote its lists
            lists = staging[lists_offset:staging_bytes].cpu().numpy().view(np.int64)
            assert np.array_equal(lists[:n], long_list), "list of the pairs in long runs"
            assert np.array_equal(lists[n:], short_list), "list of the other pairs"
        want_host, want_dev = host.before.copy(), dev.before.copy()
        for p in range(n_planes):
            d = _view(want_dev if not to_host else dev.before, 0, p, dev_blocks, bb, bb)
            h = _view(want_host if to_host else host.before, 0, p, host_blocks, bb, bb)
            if to_host:
                h[host_ids] = d[dev_ids]
            else:
                d[dev_ids] = h[host_ids]
        for p in range(n_planes):      # the same planes through the C oracle
            src_buf, dst_buf = (dev.before, host.before) if to_host else (host.before, dev.before)
            sb, db = (dev_blocks, host_blocks) if to_host else (host_blocks, dev_blocks)
            chk = np.ascontiguousarray(_view(dst_buf, 0, p, db, bb, bb))
            O.c_swap_blocks([chk], [np.ascontiguousarray(_view(src_buf, 0, p, sb, bb, bb))], pairs)
            assert np.array_equal(chk, _view(want_host if to_host else want_dev, 0, p, db, bb, bb))
        assert np.array_equal(host.now(), want_host), "host side"
        assert np.array_equal(dev.now(), want_dev), "device side"


@pytest.mark.parametrize("to_host", [True, False])
def test_auto_swap_refuses_a_host_array_that_differs_from_the_table(to_host):
    """HFK_KNOB_CHECK_HOST_COLUMN: the host array of host slots and the device table's host column are two
    copies of one thing; with the check on, a call whose copies differ returns HFK_ERR_TABLE_MISMATCH and
    moves nothing; with it off (the default) the same call is accepted."""
    rng = np.random.default_rng(99)
    n_planes, dev_blocks, host_blocks, bb, n = 2, 12, 16, 4096, 8
    announce("auto swap with the host-column check, to_host %s" % to_host)
    dev = Arena(n_planes * dev_blocks * bb, False, rng)
    host = Arena(n_planes * host_blocks * bb, True, rng)
    dtab = _table(_planes(dev.addr, 0, n_planes, dev_blocks, bb))
    htab = _table(_planes(host.addr, 0, n_planes, host_blocks, bb))
    host_addrs = (ctypes.c_void_p * n_planes)(*[host.host_addr + p * host_blocks * bb for p in range(n_planes)])
    host_ids = np.arange(4, 4 + n, dtype=np.int64)
    dev_ids = rng.permutation(dev_blocks)[:n].astype(np.int64)
    pairs_d = torch.from_numpy(np.stack([dev_ids, host_ids] if to_host else [host_ids, dev_ids], 1).astype(np.int64)).to(DEV)
    staging = torch.zeros(n_planes * n * bb, dtype=torch.uint8, device=DEV)
    wrong = host_ids.copy()
    wrong[3] = 0                    # breaks the run the copy engines would take

    def call(ids):
        return capi.swap_blocks_auto(dtab.data_ptr(), htab.data_ptr(), host_addrs, pairs_d.data_ptr(), ids.ctypes.data, n_planes,
                                     n, bb, bb, bb, dev_blocks, host_blocks, staging.data_ptr(), staging.numel(), int(to_host),
                                     2, 0, stream_handle())

    with capi.thread_tuning({capi.KNOB_CHECK_HOST_COLUMN: 1}):
        rc = call(wrong)
        assert rc == capi.ERR_TABLE_MISMATCH, rc
        assert "host_block_ids" in capi.status_string(rc)
        torch.cuda.synchronize()
        assert np.array_equal(host.now(), host.before) and np.array_equal(dev.now(), dev.before), "a refused call moved bytes"
        assert call(host_ids) == 0
    torch.cuda.synchronize()
    moved = dev.now() if not to_host else host.now()
    assert not np.array_equal(moved, dev.before if not to_host else host.before)
