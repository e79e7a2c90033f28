"""CPU oracle for the pcieThrough path: checker only, never the product.

TEST INFRASTRUCTURE. Only ``tests/``, the smoke check and the benchmark's CPU
baseline may import this module. Three independent statements of each operation
live here so that they can pin one another:

* ``c_*``      - ctypes calls into ``libhfk_oracle.so`` (``hfk_oracle.c``, the plain-C
                 restatement that keeps the reference's per-core work split),
* ``torch_*``  - the torch CPU path the reference's tests and baseline use
                 (``embed[ids]``, pcieThrough/tests/test_memcpy.py:18,23; the
                 permute-compare of pcieThrough/tests/test_transfer_kernel.py:77-83;
                 ``index_select`` / ``index_copy_`` for the block table),
* ``brute_*``  - pure-Python element loops written straight from the index formulas
                 (pcieThrough/csrc/kernel/multi_layer_block_transfer_kernel.h:47,63-67;
                 pcieThrough/csrc/kernel/gather.h:106-122), for tiny shapes only.

Everything works on bytes: callers pass ``numpy.uint8`` arrays (or torch tensors
viewed as uint8), so bf16 / fp8 payloads with NaN bit patterns compare exactly.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhfk_oracle.so")
_lib = None


def build(force=False):
    """Compile hfk_oracle.c with gcc (seconds)."""
    if force or not os.path.exists(_LIB_PATH) or (
        os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "hfk_oracle.c"))
    ):
        subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libhfk_oracle.so"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        u64, u32, vp, ci = ctypes.c_uint64, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_int
        L.oracle_gather_rows.argtypes = [vp, vp, vp, ci, u64, u64, u32]
        L.oracle_gather_rows.restype = ci
        L.oracle_multi_layer_block_transfer.argtypes = [vp, vp, u32, u32, u32, u32, u32, u32]
        L.oracle_multi_layer_block_transfer.restype = ci
        L.oracle_multi_layer_block_table_transfer.argtypes = [vp, u64, vp, u64, vp, u64, u32, u32, u32, u32, u32, ci, u32]
        L.oracle_multi_layer_block_table_transfer.restype = ci
        L.oracle_swap_blocks.argtypes = [vp, vp, vp, u32, u64, u64, u64, u64]
        L.oracle_swap_blocks.restype = ci
        _lib = L
    return _lib


def _u8(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint8).reshape(a.shape[0], -1) if a.ndim > 1 else a.view(np.uint8)


# ----------------------------------------------------------------------------
# C restatement
# ----------------------------------------------------------------------------
def c_gather_rows(table_u8, ids, cores=2):
    """table_u8: [rows, row_bytes] uint8; ids: int64 or int32 1-D. Returns [n, row_bytes]."""
    table_u8 = np.ascontiguousarray(table_u8)
    assert table_u8.dtype == np.uint8 and table_u8.ndim == 2
    ids = np.ascontiguousarray(ids)
    assert ids.dtype in (np.int64, np.int32)
    out = np.zeros((ids.shape[0], table_u8.shape[1]), dtype=np.uint8)
    rc = lib().oracle_gather_rows(
        table_u8.ctypes.data, out.ctypes.data, ids.ctypes.data, int(ids.dtype == np.int64),
        ids.shape[0], table_u8.shape[1], cores)
    assert rc == 0, rc
    return out


def c_multi_layer_block_transfer(src_u8, T, L, H, D, elem_bytes, cores=2, fill=0):
    """src_u8: flat uint8 of T*L*H*D*elem_bytes bytes ([T,L,H,D] order).
    Returns uint8 [L, H*T*D*elem_bytes]: the L per-layer [H,T,D] buffers."""
    src_u8 = np.ascontiguousarray(src_u8).reshape(-1)
    assert src_u8.dtype == np.uint8 and src_u8.size == T * L * H * D * elem_bytes
    out = np.full((L, H * T * D * elem_bytes), fill, dtype=np.uint8)
    ptrs = (ctypes.c_void_p * max(L, 1))(*[out[l].ctypes.data for l in range(L)])
    rc = lib().oracle_multi_layer_block_transfer(ptrs, src_u8.ctypes.data, T, L, H, D, elem_bytes, cores)
    assert rc == 0, rc
    return out


def c_multi_layer_block_table_transfer(layers_u8, packed_u8, pairs, T, L, H, D, elem_bytes, to_packed, cores=2):
    """layers_u8: uint8 [L, dev_blocks, H*T*D*e] (per-layer caches); packed_u8: uint8
    [packed_blocks, T*L*H*D*e]; pairs int64 [n,2] = (packed_block, layered_block).
    Mutates layers_u8 (to_packed False) or packed_u8 (to_packed True) in place."""
    assert layers_u8.dtype == np.uint8 and packed_u8.dtype == np.uint8
    assert layers_u8.flags.c_contiguous and packed_u8.flags.c_contiguous
    assert layers_u8.shape[0] == L and layers_u8.shape[2] == H * T * D * elem_bytes
    assert packed_u8.shape[1] == T * L * H * D * elem_bytes
    pairs = np.ascontiguousarray(pairs, dtype=np.int64).reshape(-1, 2)
    ptrs = (ctypes.c_void_p * max(L, 1))(*[layers_u8[l].ctypes.data for l in range(L)])
    rc = lib().oracle_multi_layer_block_table_transfer(
        ptrs, layers_u8.shape[2], packed_u8.ctypes.data, packed_u8.shape[1], pairs.ctypes.data, pairs.shape[0],
        T, L, H, D, elem_bytes, int(bool(to_packed)), cores)
    assert rc == 0, rc


def c_swap_blocks(dst_planes_u8, src_planes_u8, pairs):
    """dst/src_planes_u8: lists of [blocks, block_bytes] uint8 arrays (dst mutated in place).
    pairs: int64 [n, 2] = (src_block, dst_block)."""
    pairs = np.ascontiguousarray(pairs, dtype=np.int64).reshape(-1, 2)
    n_planes = len(dst_planes_u8)
    assert n_planes == len(src_planes_u8)
    if n_planes == 0 or pairs.shape[0] == 0:
        return dst_planes_u8
    bb = src_planes_u8[0].shape[1]
    for d, s in zip(dst_planes_u8, src_planes_u8):
        assert d.dtype == np.uint8 and s.dtype == np.uint8
        assert d.flags.c_contiguous and s.flags.c_contiguous and d.shape[1] == bb and s.shape[1] == bb
    dp = (ctypes.c_void_p * n_planes)(*[d.ctypes.data for d in dst_planes_u8])
    sp = (ctypes.c_void_p * n_planes)(*[s.ctypes.data for s in src_planes_u8])
    rc = lib().oracle_swap_blocks(dp, sp, pairs.ctypes.data, n_planes, pairs.shape[0], bb, bb, bb)
    assert rc == 0, rc
    return dst_planes_u8


# ----------------------------------------------------------------------------
# torch CPU path (index_select / index_copy_ over the same block table; also the timed CPU baseline)
# ----------------------------------------------------------------------------
def torch_gather_rows(table, ids):
    """dst = table.index_select(0, ids) == table[ids] (tests/test_memcpy.py:18)."""
    import torch
    return torch.index_select(table, 0, ids.to(torch.int64))


def torch_swap_blocks(dst_plane, src_plane, src_ids, dst_ids):
    """In place on dst_plane: dst.index_copy_(0, dst_ids, src.index_select(0, src_ids))."""
    return dst_plane.index_copy_(0, dst_ids, src_plane.index_select(0, src_ids))


def torch_multi_layer_block_transfer(host_block):
    """host_block [T,L,H,D] -> list of L contiguous [H,T,D] tensors.
    Inverse of the check in tests/test_transfer_kernel.py:77-83, where the device
    block [L,H,T,D] permuted by (2,0,1,3) must equal the host block [T,L,H,D]."""
    L = host_block.shape[1]
    return [host_block[:, l].permute(1, 0, 2).contiguous() for l in range(L)]


# ----------------------------------------------------------------------------
# brute force (tiny shapes only)
# ----------------------------------------------------------------------------
def brute_gather_rows(table_u8, ids):
    rows, rb = table_u8.shape
    out = np.zeros((len(ids), rb), dtype=np.uint8)
    for i in range(len(ids)):
        for b in range(rb):
            out[i, b] = table_u8[int(ids[i]), b]
    return out


def brute_multi_layer_block_transfer(src_u8, T, L, H, D, elem_bytes):
    src = np.asarray(src_u8).reshape(-1)
    out = np.zeros((L, H * T * D * elem_bytes), dtype=np.uint8)
    for t in range(T):
        for l in range(L):
            for h in range(H):
                for d in range(D):
                    for b in range(elem_bytes):
                        s = (((t * L + l) * H + h) * D + d) * elem_bytes + b
                        o = ((h * T + t) * D + d) * elem_bytes + b
                        out[l, o] = src[s]
    return out


def brute_block_table_transfer(layers_u8, packed_u8, pairs, T, L, H, D, elem_bytes, to_packed):
    """Element loops for the block-table transfer in either direction (in place)."""
    for (pb, db) in np.asarray(pairs).reshape(-1, 2):
        for t in range(T):
            for l in range(L):
                for h in range(H):
                    for d in range(D * elem_bytes):
                        po = ((t * L + l) * H + h) * D * elem_bytes + d
                        lo = (h * T + t) * D * elem_bytes + d
                        if to_packed:
                            packed_u8[int(pb), po] = layers_u8[l, int(db), lo]
                        else:
                            layers_u8[l, int(db), lo] = packed_u8[int(pb), po]


def brute_swap_blocks(dst_planes_u8, src_planes_u8, pairs):
    for p in range(len(dst_planes_u8)):
        for (sb, db) in np.asarray(pairs).reshape(-1, 2):
            for b in range(src_planes_u8[p].shape[1]):
                dst_planes_u8[p][int(db), b] = src_planes_u8[p][int(sb), b]
    return dst_planes_u8
