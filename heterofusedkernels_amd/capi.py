"""ctypes binding of the C-ABI in include/hfk.h (libhfk_hip.so).

Thin by design: arguments are raw addresses and sizes, exactly what a C caller
passes. ``check`` turns a non-zero status into ``RuntimeError``. torch is used by
callers for device memory and streams only; nothing here touches tensors.
"""
import ctypes
import os

from . import _build

_lib = None

KNOB_UNROLL = 0
KNOB_NONTEMPORAL = 1
KNOB_WORKGROUPS_PER_CU = 2
KNOB_SWAP_WORKGROUPS = 3
KNOB_DUPLEX_UNROLL = 4
KNOB_SWAP_UNROLL = 5
KNOB_SWAP_PACE_MBPS = 6
KNOB_LINK_MBPS = 7
KNOB_DUPLEX_WORKGROUPS = 8
KNOB_THROUGHPUT_PACE_PERMILLE = 9
KNOB_HBM_LDS_BYTES = 10
KNOB_PACED_UNROLL = 11
KNOB_PACED_WORKGROUPS = 12
KNOB_PACE_REPORT = 13
KNOB_DUPLEX_PACE_PERMILLE = 14
KNOB_TRANSFER_PACE_PERMILLE = 15
KNOB_TRANSFER_UNROLL = 16
KNOB_CHECK_HOST_COLUMN = 17
KNOB_TRANSFER_TILED = 18
KNOB_ADAPTIVE_PACE = 19
KNOB_FUSED_COPY_ENGINE = 20
SWAP_DST_HOST = 1
SWAP_SRC_HOST = 2
SWAP_BESIDE_COMPUTE = 4
SWAP_SRC_DEVICE = 8
SWAP_DST_DEVICE = 16
STATIC_STAGING_BYTES = 64 << 20
ERR_STAGING_TOO_SMALL = -7
ERR_TABLE_MISMATCH = -8
ERR_STAGING_BUSY = -9


class KnobValue(ctypes.Structure):
    """struct hfk_knob_value."""
    _fields_ = [("knob", ctypes.c_int), ("value", ctypes.c_int64)]


class BlockMove(ctypes.Structure):
    """struct hfk_block_move."""
    _fields_ = [("dst_plane_ptrs", ctypes.c_void_p), ("src_plane_ptrs", ctypes.c_void_p),
                ("block_pairs", ctypes.c_void_p), ("n_pairs", ctypes.c_uint64),
                ("src_block_stride", ctypes.c_uint64), ("dst_block_stride", ctypes.c_uint64),
                ("src_blocks", ctypes.c_uint64), ("dst_blocks", ctypes.c_uint64)]

ENTRY_POINTS = (
    "hfk_version",
    "hfk_status_string",
    "hfk_gather_rows",
    "hfk_multi_layer_block_transfer",
    "hfk_fused_memcpy_multi_layer_block_transfer",
    "hfk_multi_layer_block_table_transfer",
    "hfk_swap_blocks",
    "hfk_swap_blocks_duplex",
    "hfk_swap_blocks_staged",
    "hfk_swap_blocks_staged_static",
    "hfk_swap_blocks_auto",
    "hfk_gather_blocks",
    "hfk_set_tuning",
    "hfk_get_tuning",
    "hfk_pace_state",
    "hfk_thread_tuning_begin",
    "hfk_thread_tuning_end",
)


def library_path():
    """In-tree build output, or the copy installed next to libpcie_through.so."""
    if os.path.exists(_build.HFK_HIP_SO):
        return _build.HFK_HIP_SO
    try:
        import importlib.util

        spec = importlib.util.find_spec("pcie_through")
        if spec is not None and spec.submodule_search_locations:
            installed = os.path.join(list(spec.submodule_search_locations)[0], "lib", "libhfk_hip.so")
            if os.path.exists(installed):
                return installed
    except (ImportError, ValueError):
        pass
    return _build.HFK_HIP_SO


def load():
    """Load libhfk_hip.so (built in-tree). Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not os.path.exists(path):
        raise RuntimeError(
            "libhfk_hip.so is not built (%s); run `python -m heterofusedkernels_amd._build`" % path
        )
    L = ctypes.CDLL(path)
    vp, u64, u32, ci, i64 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_uint32, ctypes.c_int, ctypes.c_int64
    L.hfk_version.argtypes = []
    L.hfk_version.restype = ci
    L.hfk_status_string.argtypes = [ci]
    L.hfk_status_string.restype = ctypes.c_char_p
    L.hfk_gather_rows.argtypes = [vp, vp, vp, ci, u64, u64, u64, u32, u32, vp]
    L.hfk_gather_rows.restype = ci
    L.hfk_multi_layer_block_transfer.argtypes = [vp, vp, u32, u32, u32, u32, u32, u32, u32, vp]
    L.hfk_multi_layer_block_transfer.restype = ci
    L.hfk_fused_memcpy_multi_layer_block_transfer.argtypes = [vp, vp, vp, u32, u32, u32, u32, u32, u32, vp]
    L.hfk_fused_memcpy_multi_layer_block_transfer.restype = ci
    L.hfk_multi_layer_block_table_transfer.argtypes = [vp, u64, vp, u64, vp, u64, u64, u64, u32, u32, u32, u32, u32, ci,
                                                       u32, u32, vp]
    L.hfk_multi_layer_block_table_transfer.restype = ci
    L.hfk_swap_blocks.argtypes = [vp, vp, vp, u32, u64, u64, u64, u64, u64, u64, u32, u32, vp]
    L.hfk_swap_blocks.restype = ci
    L.hfk_swap_blocks_duplex.argtypes = [ctypes.POINTER(BlockMove), ctypes.POINTER(BlockMove), u32, u64, u32, u32, vp]
    L.hfk_swap_blocks_duplex.restype = ci
    L.hfk_swap_blocks_staged.argtypes = [vp, vp, vp, vp, u32, u64, u64, u64, u64, u64, u64, vp, ci, u32, vp]
    L.hfk_swap_blocks_staged.restype = ci
    L.hfk_swap_blocks_staged_static.argtypes = [vp, vp, vp, vp, u32, u64, u64, u64, u64, u64, u64, ci, u32, vp]
    L.hfk_swap_blocks_staged_static.restype = ci
    L.hfk_swap_blocks_auto.argtypes = [vp, vp, vp, vp, vp, u32, u64, u64, u64, u64, u64, u64, vp, u64, ci, u32, u32, vp]
    L.hfk_swap_blocks_auto.restype = ci
    L.hfk_gather_blocks.argtypes = [vp, vp, vp, u32, u64, u64, u64, u64, u32, u32, vp]
    L.hfk_gather_blocks.restype = ci
    L.hfk_set_tuning.argtypes = [ci, i64]
    L.hfk_set_tuning.restype = ci
    L.hfk_get_tuning.argtypes = [ci]
    L.hfk_get_tuning.restype = i64
    L.hfk_pace_state.argtypes = [ctypes.POINTER(ctypes.c_uint32)]
    L.hfk_pace_state.restype = ci
    L.hfk_thread_tuning_begin.argtypes = [ctypes.POINTER(KnobValue), u32]
    L.hfk_thread_tuning_begin.restype = ci
    L.hfk_thread_tuning_end.argtypes = []
    L.hfk_thread_tuning_end.restype = None
    _lib = L
    return L


def status_string(rc):
    return load().hfk_status_string(rc).decode()


def check(rc, what="hfk call"):
    if rc != 0:
        raise RuntimeError("%s failed: %s (%d)" % (what, status_string(rc), rc))


def gather_rows(table, dst, ids, ids_are_i64, n_ids, row_bytes, table_rows=0, workgroups=0, stream=0, flags=0):
    return load().hfk_gather_rows(table, dst, ids, int(ids_are_i64), n_ids, row_bytes, table_rows, flags, workgroups,
                                  stream)


def multi_layer_block_transfer(layer_ptrs, src, T, L, H, D, elem_bytes, workgroups=0, stream=0, flags=0):
    return load().hfk_multi_layer_block_transfer(layer_ptrs, src, T, L, H, D, elem_bytes, flags, workgroups, stream)


def fused_memcpy_multi_layer_block_transfer(layer_ptrs, host_block, staging, T, L, H, D, elem_bytes,
                                            workgroups=0, stream=0):
    return load().hfk_fused_memcpy_multi_layer_block_transfer(layer_ptrs, host_block, staging, T, L, H, D,
                                                              elem_bytes, workgroups, stream)


def multi_layer_block_table_transfer(layer_ptrs, dev_block_stride, packed_blocks, packed_block_stride, pairs, n_pairs,
                                     n_packed_blocks, n_dev_blocks, T, L, H, D, elem_bytes, to_packed, workgroups=0,
                                     stream=0, flags=0):
    return load().hfk_multi_layer_block_table_transfer(layer_ptrs, dev_block_stride, packed_blocks,
                                                       packed_block_stride, pairs, n_pairs, n_packed_blocks,
                                                       n_dev_blocks, T, L, H, D, elem_bytes, int(bool(to_packed)),
                                                       flags, workgroups, stream)


def swap_blocks(dst_planes, src_planes, pairs, n_planes, n_pairs, block_bytes, src_stride, dst_stride,
                src_blocks=0, dst_blocks=0, workgroups=0, stream=0, flags=0):
    return load().hfk_swap_blocks(dst_planes, src_planes, pairs, n_planes, n_pairs, block_bytes, src_stride,
                                  dst_stride, src_blocks, dst_blocks, flags, workgroups, stream)


def swap_blocks_duplex(out_move, in_move, n_planes, block_bytes, workgroups=0, stream=0, flags=0):
    """out_move / in_move: BlockMove instances or None."""
    return load().hfk_swap_blocks_duplex(ctypes.byref(out_move) if out_move is not None else None,
                                         ctypes.byref(in_move) if in_move is not None else None, n_planes, block_bytes,
                                         flags, workgroups, stream)


def swap_blocks_staged(dev_planes, host_plane_addrs, dev_ids, host_ids, n_planes, n_blocks, block_bytes, dev_stride,
                       host_stride, dev_blocks, host_blocks, staging, to_host, workgroups=0, stream=0):
    """host_plane_addrs / host_ids: addresses of HOST arrays (e.g. numpy .ctypes.data)."""
    return load().hfk_swap_blocks_staged(dev_planes, host_plane_addrs, dev_ids, host_ids, n_planes, n_blocks,
                                         block_bytes, dev_stride, host_stride, dev_blocks, host_blocks, staging,
                                         int(bool(to_host)), workgroups, stream)


def swap_blocks_staged_static(dev_planes, host_plane_addrs, dev_ids, host_ids, n_planes, n_blocks, block_bytes,
                              dev_stride, host_stride, dev_blocks, host_blocks, to_host, workgroups=0, stream=0):
    """hfk_swap_blocks_staged through the library's own staging array (no staging argument, no allocation)."""
    return load().hfk_swap_blocks_staged_static(dev_planes, host_plane_addrs, dev_ids, host_ids, n_planes, n_blocks,
                                                block_bytes, dev_stride, host_stride, dev_blocks, host_blocks,
                                                int(bool(to_host)), workgroups, stream)


def swap_blocks_auto(dev_planes, host_planes_mapped, host_plane_addrs, pairs, host_ids, n_planes, n_pairs, block_bytes,
                     dev_stride, host_stride, dev_blocks, host_blocks, staging, staging_bytes, to_host,
                     min_run_blocks=0, flags=0, stream=0):
    """host_plane_addrs / host_ids: addresses of HOST arrays or None; pairs: device [n, 2] (src, dst)."""
    return load().hfk_swap_blocks_auto(dev_planes, host_planes_mapped, host_plane_addrs, pairs, host_ids, n_planes,
                                       n_pairs, block_bytes, dev_stride, host_stride, dev_blocks, host_blocks, staging,
                                       staging_bytes, int(bool(to_host)), min_run_blocks, flags, stream)


def gather_blocks(dst_planes, src_planes, ids, n_planes, n_ids, block_bytes, src_stride, src_blocks=0,
                  workgroups=0, stream=0, flags=0):
    return load().hfk_gather_blocks(dst_planes, src_planes, ids, n_planes, n_ids, block_bytes, src_stride,
                                    src_blocks, flags, workgroups, stream)


def set_tuning(knob, value):
    return load().hfk_set_tuning(knob, value)


def get_tuning(knob):
    return load().hfk_get_tuning(knob)


def pace_state():
    """The eight words of hfk_pace_state for the current device (waits for the device)."""
    out = (ctypes.c_uint32 * 8)()
    check(load().hfk_pace_state(out), "hfk_pace_state")
    return list(out)


class thread_tuning:
    """``with capi.thread_tuning({capi.KNOB_UNROLL: 4, ...}):`` -- knob values for the calls this thread
    makes inside the block (hfk_thread_tuning_begin / _end); the process-wide values stay as they are."""

    def __init__(self, overrides):
        self.overrides = dict(overrides)

    def __enter__(self):
        items = (KnobValue * max(1, len(self.overrides)))(*[KnobValue(k, v) for k, v in self.overrides.items()])
        check(load().hfk_thread_tuning_begin(items, len(self.overrides)), "hfk_thread_tuning_begin")
        return self

    def __exit__(self, *exc):
        load().hfk_thread_tuning_end()
        return False
