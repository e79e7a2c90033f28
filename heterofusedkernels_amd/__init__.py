"""MI355X-native implementation of HeteroFusedKernels' pcieThrough path.

The drop-in Python packages keep the reference's names and live under
``dropin/``: ``pcie_through`` (importing it loads ``lib/libpcie_through.so`` and
with it ``torch.ops.pcie_through.*``) and ``heterofusedkernels`` (``.memory``).
Importing this package puts that directory on ``sys.path`` so that
``import pcie_through`` / ``from heterofusedkernels import memory`` resolve to
this build; an installation that copies ``dropin/*`` into site-packages needs
nothing from here.

``capi`` binds the C-ABI of ``libhfk_hip.so`` with ctypes (what the tests and the
benchmark call). There is no CPU implementation: every entry point needs the
built HIP library and raises if it is missing.
"""
import os
import sys

DROPIN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "dropin")


def enable_dropin():
    """Make ``pcie_through`` and ``heterofusedkernels`` importable from this tree."""
    if DROPIN_DIR not in sys.path:
        sys.path.insert(0, DROPIN_DIR)
    return DROPIN_DIR


enable_dropin()
