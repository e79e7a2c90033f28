import os
import pathlib

import torch


def _load_opextension_so():
    """Load <package>/lib/libpcie_through.so and thereby register torch.ops.pcie_through.*
    (same side effect and location as the reference's pcieThrough/pcie_through/_load.py:8-11).
    A missing library is an error: there is no fallback implementation."""
    pkg_path = pathlib.Path(__file__).parents[0]
    so_path = os.path.join(pkg_path, "lib", "libpcie_through.so")
    if not os.path.exists(so_path):
        raise ImportError(
            "pcie_through: %s has not been built (python -m heterofusedkernels_amd._build)" % so_path
        )
    torch.ops.load_library(so_path)
