from ._load import _load_opextension_so

_load_opextension_so()


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
    return torch.tensor(addrs, dtype=torch.int64).to(device)
