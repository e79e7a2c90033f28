"""Build recipe: explicit compiler command lines, no build system.

Artefacts (all in-tree, git-ignored):

    dropin/pcie_through/lib/libhfk_hip.so        gfx950 kernels + C-ABI (hipcc)
    dropin/pcie_through/lib/libpcie_through.so   torch dispatcher ops
    dropin/heterofusedkernels/libmanaged_memory.so   host-memory registry + allocator
    dropin/heterofusedkernels/memory*.so         Python module heterofusedkernels.memory
    dropin/heterofusedkernels/include/*.h        headers shipped for native users
    bin/hfk_c_client                             plain-C99 client of the C-ABI (csrc/examples)
    bin/libhfk_bench.so                          benchmark-only comparison paths and yardstick kernels
                                                 (outside the packages: never installed)

Run as ``python -m heterofusedkernels_amd._build`` or through ``build_all()``.
"""
import os
import shutil
import subprocess
import sysconfig
import time

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
INCLUDE = os.path.join(ROOT, "include")
DROPIN = os.path.join(PKG, "dropin")
PCIE_LIB = os.path.join(DROPIN, "pcie_through", "lib")
COMMON = os.path.join(DROPIN, "heterofusedkernels")
ROCM = os.environ.get("ROCM_PATH", "/opt/rocm")
GPU_ARCH = "gfx950"

HFK_HIP_SO = os.path.join(PCIE_LIB, "libhfk_hip.so")
PCIE_THROUGH_SO = os.path.join(PCIE_LIB, "libpcie_through.so")
HFK_BENCH_SO = os.path.join(PKG, "bin", "libhfk_bench.so")
MANAGED_MEMORY_SO = os.path.join(COMMON, "libmanaged_memory.so")
MEMORY_EXT_SO = os.path.join(COMMON, "memory" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))
C_CLIENT = os.path.join(PKG, "bin", "hfk_c_client")


def _run(cmd, quiet_patterns=()):
    t0 = time.time()
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines() if not any(p in line for p in quiet_patterns)
    )
    if proc.returncode != 0:
        raise RuntimeError("command failed (%d): %s\n%s" % (proc.returncode, " ".join(cmd), out))
    if out.strip():
        print(out)
    print("[build] %-28s %.1fs" % (os.path.basename(cmd[cmd.index("-o") + 1]), time.time() - t0), flush=True)


def build_hfk_hip():
    os.makedirs(PCIE_LIB, exist_ok=True)
    _run(
        [
            os.path.join(ROCM, "bin", "hipcc"), "--offload-arch=" + GPU_ARCH, "-O3", "-std=c++17", "-fPIC",
            "-shared", "-fvisibility=hidden", "-Wall",
            # hipcc -O3 turns float code into packed-fp32 instructions on its own; keep them off.
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-I" + INCLUDE, "-I" + CSRC, os.path.join(CSRC, "hfk_capi.hip"), "-o", HFK_HIP_SO,
        ],
        quiet_patterns=("packed-fp32-ops' is not a recognized feature",),
    )


def build_bench_support():
    """Comparison paths used by bench.py only (per-block hipMemcpyAsync loop, HBM read / write / copy
    yardstick kernels of the gather's shape). Built beside the C client, not into a package."""
    os.makedirs(os.path.dirname(HFK_BENCH_SO), exist_ok=True)
    _run(
        [
            os.path.join(ROCM, "bin", "hipcc"), "--offload-arch=" + GPU_ARCH, "-O3", "-std=c++17", "-fPIC",
            "-shared", "-fvisibility=hidden", "-Wall",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-I" + INCLUDE, "-I" + CSRC, os.path.join(CSRC, "bench_support.hip"), "-o", HFK_BENCH_SO,
        ],
        quiet_patterns=("packed-fp32-ops' is not a recognized feature",),
    )


def build_managed_memory():
    os.makedirs(COMMON, exist_ok=True)
    _run(
        [
            "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__=1",
            "-DHFK_MANAGED_MEM_NO_TORCH=1",   # the library itself is torch-free; its header serves both kinds of caller
            "-I" + os.path.join(ROCM, "include"), "-I" + INCLUDE, "-I" + CSRC,
            os.path.join(CSRC, "managed_mem.cpp"), "-o", MANAGED_MEMORY_SO,
            "-L" + os.path.join(ROCM, "lib"), "-lamdhip64", "-pthread",
        ]
    )
    inc = os.path.join(COMMON, "include")
    os.makedirs(inc, exist_ok=True)
    shutil.copy2(os.path.join(CSRC, "managed_mem.h"), inc)
    shutil.copy2(os.path.join(INCLUDE, "hfk_managed_memory.h"), inc)


def _torch_flags():
    import torch
    from torch.utils import cpp_extension

    tdir = os.path.dirname(torch.__file__)
    incs = ["-I" + p for p in cpp_extension.include_paths("cuda")]
    incs.append("-I" + sysconfig.get_paths()["include"])
    cxx = [
        "-O2", "-std=c++17", "-fPIC", "-shared", "-DUSE_ROCM=1", "-D__HIP_PLATFORM_AMD__=1",
        "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-Wno-deprecated-declarations",
    ]
    tlib = os.path.join(tdir, "lib")
    link = ["-L" + tlib, "-lc10", "-ltorch_cpu", "-ltorch", "-lc10_hip", "-ltorch_hip",
            "-L" + os.path.join(ROCM, "lib"), "-lamdhip64"]
    return cxx, incs, link, tlib


def build_memory_ext():
    cxx, incs, link, tlib = _torch_flags()
    _run(
        ["g++"] + cxx + ["-DTORCH_EXTENSION_NAME=memory", "-DTORCH_API_INCLUDE_EXTENSION_H"] + incs
        + ["-I" + INCLUDE, "-I" + CSRC, os.path.join(CSRC, "memory_pybind.cpp"), "-o", MEMORY_EXT_SO]
        + link + ["-ltorch_python", "-L" + COMMON, "-lmanaged_memory", "-Wl,-rpath,$ORIGIN"]
    )


def build_pcie_through():
    cxx, incs, link, tlib = _torch_flags()
    os.makedirs(PCIE_LIB, exist_ok=True)
    _run(
        ["g++"] + cxx + incs
        + ["-I" + INCLUDE, "-I" + CSRC, os.path.join(CSRC, "pcie_through_ops.cpp"), "-o", PCIE_THROUGH_SO]
        + link + ["-L" + PCIE_LIB, "-lhfk_hip", "-L" + COMMON, "-lmanaged_memory",
                  "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,$ORIGIN/../../heterofusedkernels", "-Wl,-z,defs"]
    )


def build_c_client():
    """The C-ABI as a foreign runtime sees it: C99, the two public headers, the HIP runtime's C API."""
    os.makedirs(os.path.dirname(C_CLIENT), exist_ok=True)
    _run(
        [
            "gcc", "-std=c99", "-O2", "-Wall", "-Wextra", "-Werror", "-D__HIP_PLATFORM_AMD__=1",
            "-I" + os.path.join(ROCM, "include"), "-I" + INCLUDE,
            os.path.join(CSRC, "examples", "hfk_c_client.c"), "-o", C_CLIENT,
            "-L" + PCIE_LIB, "-lhfk_hip", "-L" + COMMON, "-lmanaged_memory",
            "-L" + os.path.join(ROCM, "lib"), "-lamdhip64",
            "-Wl,-rpath,$ORIGIN/../dropin/pcie_through/lib", "-Wl,-rpath,$ORIGIN/../dropin/heterofusedkernels",
            "-Wl,-rpath," + os.path.join(ROCM, "lib"),
        ]
    )


def build_all():
    """Compile everything, every time it is called."""
    build_hfk_hip()
    build_bench_support()
    build_managed_memory()
    build_memory_ext()
    build_pcie_through()
    build_c_client()


def artefacts():
    return [HFK_HIP_SO, HFK_BENCH_SO, PCIE_THROUGH_SO, MANAGED_MEMORY_SO, MEMORY_EXT_SO, C_CLIENT]


if __name__ == "__main__":
    build_all()
    for a in artefacts():
        print(a, os.path.getsize(a))
