"""Helpers for the GPU parity tests: raw-address plumbing between torch tensors and
the C-ABI. torch provides device memory and streams only."""
import sys

import torch

from heterofusedkernels_amd import capi


def announce(msg):
    """Name the case before touching the GPU, so a fault can be attributed."""
    print("[gpu-case] " + msg, flush=True)
    sys.stdout.flush()


def stream_handle():
    return torch.cuda.current_stream().cuda_stream


def ptr_table(tensors, device="cuda"):
    return torch.tensor([t.data_ptr() for t in tensors], dtype=torch.int64).to(device)


def host_ptr_table(host_tensors, device="cuda"):
    from heterofusedkernels import memory

    addrs = []
    for t in host_tensors:
        a = memory.get_device_ptr(t.data_ptr())
        assert a != 0, "host plane is not registered"
        addrs.append(a)
    return torch.tensor(addrs, dtype=torch.int64).to(device)


def bytes_np(t):
    """uint8 numpy view [dim0, -1] of a (CPU or device) tensor."""
    t = t.detach().cpu().contiguous()
    return t.view(torch.uint8).reshape(t.shape[0], -1).numpy() if t.dim() > 1 else t.view(torch.uint8).numpy()


def swap(dst_tab, src_tab, pairs_dev, n_planes, block_bytes, src_stride=None, dst_stride=None, src_blocks=0,
         dst_blocks=0, workgroups=0, flags=0):
    """flags: capi.SWAP_DST_HOST / SWAP_SRC_HOST / SWAP_BESIDE_COMPUTE; they pick the launch shape only."""
    rc = capi.swap_blocks(dst_tab.data_ptr(), src_tab.data_ptr(), pairs_dev.data_ptr(), n_planes,
                          pairs_dev.shape[0], block_bytes, src_stride or block_bytes, dst_stride or block_bytes,
                          src_blocks, dst_blocks, workgroups, stream_handle(), flags)
    capi.check(rc, "hfk_swap_blocks")


def gather_rows(table, dst, ids, row_bytes, table_rows=0, workgroups=0):
    rc = capi.gather_rows(table.data_ptr() if hasattr(table, "data_ptr") else table, dst.data_ptr(), ids.data_ptr(),
                          ids.dtype == torch.int64, ids.shape[0], row_bytes, table_rows, workgroups,
                          stream_handle())
    capi.check(rc, "hfk_gather_rows")


def gather_blocks(dst_tab, src_tab, ids_dev, n_planes, block_bytes, src_stride=None, src_blocks=0, workgroups=0,
                  flags=0):
    rc = capi.gather_blocks(dst_tab.data_ptr(), src_tab.data_ptr(), ids_dev.data_ptr(), n_planes, ids_dev.shape[0],
                            block_bytes, src_stride or block_bytes, src_blocks, workgroups, stream_handle(), flags)
    capi.check(rc, "hfk_gather_blocks")


def oracle_swap_planes(dst_before, src_planes, pairs, plane_ids):
    """What the C oracle makes of planes `plane_ids`: dst_before / src_planes are lists of CPU uint8
    tensors [blocks, block_bytes] (one per entry of plane_ids), pairs an int64 [n, 2] tensor.
    Returns the expected destination planes as numpy arrays."""
    from oracle import oracle as O

    want = [d.numpy().copy() for d in dst_before]
    O.c_swap_blocks(want, [s.numpy() for s in src_planes], pairs.cpu().numpy())
    return want
