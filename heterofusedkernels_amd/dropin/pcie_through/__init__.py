from ._load import _load_opextension_so

_load_opextension_so()

# plane_pointer_table() notes on the table it returns whether its planes are host memory, as an attribute
# of that tensor object: the note lives and dies with the object, and a tensor that merely sits at the
# same address later (or another view of the same storage) carries none.
_SIDE_ATTR = "hfk_planes_in_host"

# flags of torch.ops.pcie_through.swap_blocks (hfk.h: HFK_SWAP_*)
SWAP_DST_HOST = 1        # the destination planes are host memory (swap-out)
SWAP_SRC_HOST = 2        # the source planes are host memory (swap-in)
SWAP_BESIDE_COMPUTE = 4  # other kernels run at the same time: small, paced launch
SWAP_SRC_DEVICE = 8      # the source is device memory (saves the library a question to the runtime)
SWAP_DST_DEVICE = 16     # the destination is device memory


def plane_pointer_table(planes, device):
    """int64 device tensor of kernel-usable base addresses, one per plane.

    Device tensors contribute ``data_ptr()``; pinned host tensors contribute their
    mapped address from ``heterofusedkernels.memory`` (registering them first if
    needed). Build it once per cache and reuse it for every swap_blocks /
    gather_blocks call, like the per-layer pointer tensor of
    multi_layer_block_transfer.
    """
    import torch
    from heterofusedkernels import memory

    planes = list(planes)
    addrs = []
    for t in planes:
        if t.is_cuda:
            addrs.append(t.data_ptr())
        else:
            dev = memory.get_device_ptr(t.data_ptr())
            if dev == 0:
                memory.host_register(t)
                dev = memory.get_device_ptr(t.data_ptr())
            if dev == 0:
                raise RuntimeError("plane is not device-visible host memory")
            addrs.append(dev)
    table = torch.tensor(addrs, dtype=torch.int64).to(device)
    kinds = {bool(t.is_cuda) for t in planes}
    if len(kinds) == 1:   # remembered for swap_blocks() below, on the table itself
        setattr(table, _SIDE_ATTR, not kinds.pop())
    return table


def swap_blocks(dst_table, src_table, block_pairs, block_bytes, src_block_stride, dst_block_stride, src_blocks=0,
                dst_blocks=0, workgroups=None, flags=None, beside_compute=False):
    """``torch.ops.pcie_through.swap_blocks`` with the flags filled in: for tables that came from
    ``plane_pointer_table`` the side that is host memory is known and named, so the launch is sized
    for the PCIe link instead of guessing. ``flags`` given explicitly are passed through."""
    import torch
    if flags is None:
        flags = SWAP_BESIDE_COMPUTE if beside_compute else 0
        if getattr(dst_table, _SIDE_ATTR, None) is True:     # a table that carries no note names no side
            flags |= SWAP_DST_HOST
        if getattr(src_table, _SIDE_ATTR, None) is True:
            flags |= SWAP_SRC_HOST
    torch.ops.pcie_through.swap_blocks(dst_table, src_table, block_pairs, block_bytes, src_block_stride,
                                       dst_block_stride, src_blocks, dst_blocks, workgroups, flags)


def swap_flags(dst_planes, src_planes, beside_compute=False):
    """The ``flags`` argument of ``swap_blocks`` for these two plane lists: names the side that is
    host memory (so the launch is sized for the PCIe link instead of guessing) and, with
    ``beside_compute``, says that other kernels run meanwhile and matter. Planes of one side must all
    live on the same kind of memory."""
    def side(planes, what):
        kinds = {bool(t.is_cuda) for t in planes}
        if len(kinds) != 1:
            raise ValueError("%s planes mix device and host memory" % what)
        return kinds.pop()
    flags = SWAP_BESIDE_COMPUTE if beside_compute else 0
    if not side(dst_planes, "destination"):
        flags |= SWAP_DST_HOST
    if not side(src_planes, "source"):
        flags |= SWAP_SRC_HOST
    return flags
