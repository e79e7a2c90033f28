"""Installs the two drop-in packages (`pcie_through`, `heterofusedkernels`) with their
in-tree built libraries, so that `import pcie_through` works without this checkout on
sys.path. Build first: `python -m heterofusedkernels_amd._build` (hipcc for gfx950 + g++).
Mirrors what the reference's two setup scripts install (common/setup.py:176-195,
pcieThrough/setup.py:220-232): the op library under `pcie_through/lib/`, the registry
library, its headers and the `memory` extension module under `heterofusedkernels/`.
"""
import os

from setuptools import setup

ROOT = os.path.dirname(os.path.abspath(__file__))
DROPIN = os.path.join("heterofusedkernels_amd", "dropin")

missing = [p for p in (os.path.join(ROOT, DROPIN, "pcie_through", "lib", "libpcie_through.so"),
                       os.path.join(ROOT, DROPIN, "pcie_through", "lib", "libhfk_hip.so"),
                       os.path.join(ROOT, DROPIN, "heterofusedkernels", "libmanaged_memory.so"))
           if not os.path.exists(p)]
if missing:
    raise SystemExit("native libraries are not built (python -m heterofusedkernels_amd._build): " + ", ".join(missing))

setup(
    name="pcie-through-mi355x",
    version="0.1.0",
    description="MI355X-native pcieThrough path: KV-cache block swap, block gather, layout-converting block transfer",
    packages=["pcie_through", "heterofusedkernels", "heterofusedkernels_amd"],
    package_dir={"pcie_through": os.path.join(DROPIN, "pcie_through"),
                 "heterofusedkernels": os.path.join(DROPIN, "heterofusedkernels"),
                 "heterofusedkernels_amd": "heterofusedkernels_amd"},
    package_data={"pcie_through": ["lib/*.so"],
                  "heterofusedkernels": ["*.so", "include/*.h"]},
    python_requires=">=3.9",
    zip_safe=False,
)
