"""Drop-in boundary checks that need no GPU: the shared libraries load, export every
symbol the public headers declare, the torch op schemas are the reference's, and the
host-memory registry behaves like the reference's manager."""
import ctypes
import os
import re
import subprocess
import threading

import pytest
import torch

import heterofusedkernels_amd
from heterofusedkernels_amd import _build, capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header, macro):
    text = open(os.path.join(ROOT, "include", header)).read()
    return sorted(set(re.findall(macro + r"\s+[\w\s\*]+?\b(hfk_\w+)\s*\(", text)))


def _exported(so):
    out = subprocess.check_output(["nm", "-D", "--defined-only", so], text=True)
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


def test_artefacts_exist():
    for a in _build.artefacts():
        assert os.path.exists(a), a + " missing: run python -m heterofusedkernels_amd._build"


def test_hfk_hip_exports_every_declared_symbol():
    names = _declared("hfk.h", "HFK_API")
    assert sorted(names) == sorted(capi.ENTRY_POINTS)
    assert set(names) <= _exported(_build.HFK_HIP_SO)


def test_managed_memory_exports_every_declared_symbol():
    names = _declared("hfk_managed_memory.h", "HFK_MM_API")
    assert len(names) == 11
    assert set(names) <= _exported(_build.MANAGED_MEMORY_SO)
    # ... and the reference's C++ free functions, under their own (mangled) names
    cxx = subprocess.check_output(["nm", "-D", "-C", "--defined-only", _build.MANAGED_MEMORY_SO], text=True)
    for name in ("register_ptr(void*, unsigned long)", "unregister_ptr(void*)", "get_device_ptr(unsigned long)",
                 "alloc_pinned_numa_ptr(unsigned long, int)", "free_pinned_numa_ptr(void*)"):
        assert name in cxx, name


def test_reference_style_native_consumer_compiles():
    """A C++ file that uses the registry header exactly as the reference's sources do (same include,
    same calls, same types) compiles against the header shipped in the heterofusedkernels package."""
    from torch.utils import cpp_extension
    import sysconfig

    shipped = os.path.join(heterofusedkernels_amd.DROPIN_DIR, "heterofusedkernels", "include")
    assert os.path.exists(os.path.join(shipped, "managed_mem.h"))
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-Werror", "-Wno-deprecated-declarations", "-DUSE_ROCM=1",
           "-D__HIP_PLATFORM_AMD__=1", "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI), "-I" + shipped]
    cmd += ["-I" + p for p in cpp_extension.include_paths("cuda")] + ["-I" + sysconfig.get_paths()["include"]]
    cmd.append(os.path.join(ROOT, "tests", "compat", "reference_style_consumer.cpp"))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert proc.returncode == 0, proc.stdout[-3000:]


def test_capi_loads_and_reports():
    L = capi.load()
    assert L.hfk_version() == 3
    assert capi.status_string(0) == "ok"
    assert "NULL" in capi.status_string(-1)
    assert capi.get_tuning(capi.KNOB_UNROLL) in (1, 2, 4, 8, 16)
    assert capi.set_tuning(capi.KNOB_UNROLL, 3) == -4
    assert capi.set_tuning(99, 1) == -4
    assert "flag" in capi.status_string(-6)
    assert "static staging" in capi.status_string(capi.ERR_STAGING_TOO_SMALL)
    # the PCIe link rate: an override is reported back, -1 returns to auto-detection (0 = unknown without a device)
    assert capi.set_tuning(capi.KNOB_LINK_MBPS, 31500) == 0
    assert capi.get_tuning(capi.KNOB_LINK_MBPS) == 31500
    assert capi.set_tuning(capi.KNOB_LINK_MBPS, -1) == 0
    assert capi.get_tuning(capi.KNOB_LINK_MBPS) >= 0
    assert capi.set_tuning(capi.KNOB_LINK_MBPS, -2) == -4
    assert capi.set_tuning(capi.KNOB_SWAP_PACE_MBPS, 0) == 0


def test_thread_tuning_is_seen_by_the_calling_thread_only():
    """hfk_thread_tuning_begin / _end: the overrides are this thread's view, another thread keeps the
    process-wide values, a bad list is rejected whole, and _end restores the process-wide view."""
    import threading

    base = capi.get_tuning(capi.KNOB_SWAP_WORKGROUPS)
    seen = {}
    with capi.thread_tuning({capi.KNOB_SWAP_WORKGROUPS: base + 5, capi.KNOB_UNROLL: 4}):
        assert capi.get_tuning(capi.KNOB_SWAP_WORKGROUPS) == base + 5
        assert capi.get_tuning(capi.KNOB_UNROLL) == 4
        t = threading.Thread(target=lambda: seen.update(other=capi.get_tuning(capi.KNOB_SWAP_WORKGROUPS)))
        t.start()
        t.join()
        assert seen["other"] == base
        # a list with one bad entry changes nothing
        bad = (capi.KnobValue * 2)(capi.KnobValue(capi.KNOB_UNROLL, 2), capi.KnobValue(capi.KNOB_UNROLL, 3))
        assert capi.load().hfk_thread_tuning_begin(bad, 2) == -4
        assert capi.get_tuning(capi.KNOB_UNROLL) == 4
        assert capi.load().hfk_thread_tuning_begin(None, 1) == -1
        # the process-wide value can change underneath; the override still wins here
        assert capi.set_tuning(capi.KNOB_SWAP_WORKGROUPS, base + 1) == 0
        assert capi.get_tuning(capi.KNOB_SWAP_WORKGROUPS) == base + 5
    assert capi.get_tuning(capi.KNOB_SWAP_WORKGROUPS) == base + 1
    assert capi.set_tuning(capi.KNOB_SWAP_WORKGROUPS, base) == 0
    assert capi.get_tuning(capi.KNOB_UNROLL) == 1


def test_argument_errors_are_reported_before_any_gpu_work():
    # None of these reach a launch, so they are safe without a device.
    assert capi.gather_rows(0, 0, 0, True, 0, 16) == 0                 # n_ids == 0: no-op
    assert capi.gather_rows(0, 8, 8, True, 4, 16) == -1                # null table
    assert capi.gather_rows(8, 8, 8, True, 4, 0) == -2                 # empty rows
    assert capi.swap_blocks(0, 0, 0, 0, 0, 16, 16, 16) == 0            # nothing to do
    assert capi.swap_blocks(0, 8, 8, 2, 2, 16, 16, 16) == -1
    assert capi.swap_blocks(8, 8, 8, 2, 2, 32, 16, 32) == -2           # stride < block
    assert capi.swap_blocks(8, 8, 8, 2, 2, 0, 16, 32) == -2
    assert capi.swap_blocks(8, 8, 8, 2, 1 << 33, 16, 16, 16) == -3
    assert capi.swap_blocks(8, 8, 8, 2, 2, 16, 16, 16, flags=8) == -6  # a flag this entry point does not take
    assert capi.gather_rows(8, 8, 8, True, 4, 16, flags=capi.SWAP_DST_HOST) == -6
    assert capi.gather_rows(8, 8, 8, True, 4, 16, flags=capi.SWAP_SRC_HOST | capi.SWAP_SRC_DEVICE) == -6
    assert capi.gather_rows(0, 0, 0, True, 0, 16, flags=capi.SWAP_SRC_HOST) == 0
    assert capi.multi_layer_block_transfer(8, 8, 4, 4, 4, 4, 2, flags=capi.SWAP_BESIDE_COMPUTE) == -6
    assert capi.swap_blocks(0, 0, 0, 0, 0, 16, 16, 16, flags=capi.SWAP_DST_HOST | capi.SWAP_BESIDE_COMPUTE) == 0
    assert capi.gather_blocks(8, 8, 0, 2, 2, 16, 16) == -1
    assert capi.gather_blocks(8, 8, 8, 2, 2, 32, 16) == -2
    assert capi.multi_layer_block_transfer(0, 8, 4, 4, 4, 4, 2) == -1
    assert capi.multi_layer_block_transfer(8, 8, 4, 4, 4, 4, 0) == -2
    assert capi.multi_layer_block_transfer(8, 8, 0, 4, 4, 4, 2) == 0   # empty block
    assert capi.multi_layer_block_transfer(8, 8, 1 << 20, 1 << 10, 8, 128, 2) == -3
    assert capi.fused_memcpy_multi_layer_block_transfer(8, 8, 0, 4, 4, 4, 4, 2) == -1
    # staged swap: host-side arrays are validated on the host before anything is enqueued
    import numpy as np
    planes = np.array([4096, 8192], dtype=np.uint64)
    ids = np.array([0, 1, 9], dtype=np.int64)
    args = (8, planes.ctypes.data, 8, ids.ctypes.data, 2, 3, 64, 64, 64, 0, 8, 8, True)
    assert capi.swap_blocks_staged(*args) == -5                        # host id 9 >= 8 host blocks
    assert capi.swap_blocks_staged(8, 0, 8, ids.ctypes.data, 2, 3, 64, 64, 64, 0, 8, 8, True) == -1
    assert capi.swap_blocks_staged(8, planes.ctypes.data, 8, ids.ctypes.data, 2, 3, 64, 64, 32, 0, 0, 8, True) == -2
    assert capi.swap_blocks_staged(8, planes.ctypes.data, 8, ids.ctypes.data, 2, 0, 64, 64, 64, 0, 0, 8, True) == 0
    assert capi.swap_blocks_duplex(None, None, 4, 4096) == 0           # both sides empty
    assert capi.swap_blocks_duplex(None, None, 4, 0) == -2
    bad = capi.BlockMove(8, 8, None, 3, 4096, 4096, 0, 0)              # pairs missing
    assert capi.swap_blocks_duplex(bad, None, 4, 4096) == -1
    assert capi.multi_layer_block_table_transfer(8, 64, 8, 64, 0, 3, 0, 0, 2, 2, 2, 8, 1, False) == -1
    assert capi.multi_layer_block_table_transfer(8, 8, 8, 64, 8, 3, 0, 0, 2, 2, 2, 8, 1, False) == -2   # stride < block
    # flags are checked first, on every entry point that takes them
    assert capi.multi_layer_block_table_transfer(8, 64, 8, 64, 8, 3, 0, 0, 2, 2, 2, 8, 1, False, flags=1) == -6
    assert capi.swap_blocks_duplex(None, None, 4, 4096, flags=capi.SWAP_DST_HOST) == -6
    assert capi.swap_blocks_duplex(None, None, 4, 4096, flags=capi.SWAP_BESIDE_COMPUTE) == 0
    assert capi.gather_blocks(8, 8, 8, 2, 2, 16, 16, flags=capi.SWAP_DST_HOST) == -6
    assert capi.gather_blocks(0, 0, 0, 0, 0, 16, 16, flags=capi.SWAP_SRC_HOST | capi.SWAP_BESIDE_COMPUTE) == 0
    # the staged swap through the library's own staging array: size limit and host arrays, before any GPU call
    big = (8, planes.ctypes.data, 8, ids.ctypes.data, 2, 3, capi.STATIC_STAGING_BYTES // 4, 1 << 30, 1 << 30, 0, 8, True)
    assert capi.swap_blocks_staged_static(*big) == capi.ERR_STAGING_TOO_SMALL      # 2 * 3 * 16 MiB > 64 MiB
    assert capi.swap_blocks_staged_static(8, planes.ctypes.data, 8, ids.ctypes.data, 2, 0, 64, 64, 64, 0, 8, True) == 0
    assert capi.swap_blocks_staged_static(8, planes.ctypes.data, 8, ids.ctypes.data, 2, 3, 0, 64, 64, 0, 8, True) == -2
    assert capi.swap_blocks_staged_static(8, planes.ctypes.data, 8, ids.ctypes.data, 1 << 31, 1 << 40, 1 << 20, 1 << 20,
                                          1 << 20, 0, 0, True) == capi.ERR_STAGING_TOO_SMALL   # no overflow on the way
    # the run-splitting swap: flags, sizes and host slots are validated on the host
    auto = dict(dev_planes=8, host_planes_mapped=8, host_plane_addrs=planes.ctypes.data, pairs=8,
                host_ids=ids.ctypes.data, n_planes=2, n_pairs=3, block_bytes=64, dev_stride=64, host_stride=64,
                dev_blocks=0, host_blocks=8, staging=8, staging_bytes=2 * 3 * 64, to_host=True)
    assert capi.swap_blocks_auto(**auto) == -5                                      # host id 9 >= 8 host blocks
    assert capi.swap_blocks_auto(**dict(auto, flags=capi.SWAP_SRC_HOST)) == -6
    assert capi.swap_blocks_auto(**dict(auto, n_pairs=0)) == 0
    assert capi.swap_blocks_auto(**dict(auto, block_bytes=0)) == -2
    assert capi.swap_blocks_auto(**dict(auto, pairs=0)) == -1


# ---- torch ops: schemas are the reference's ---------------------------------
def test_op_schemas_match_reference():
    import pcie_through  # noqa: F401  (import side effect registers the ops)

    want = {
        # pcieThrough/csrc/host/gather_torch.cpp:60
        "gather": "pcie_through::gather(Tensor gmEmbed, Tensor gmEmbedDst, Tensor gmIds, int? aiv=None) -> ()",
        # pcieThrough/csrc/host/multi_layer_block_transfer_torch.cpp:113-114
        "multi_layer_block_transfer": "pcie_through::multi_layer_block_transfer(Tensor deviceBlockCachePtrs, "
                                      "Tensor hostBlockCache, int? aiv=None) -> ()",
        "fused_memcpy_multi_layer_block_transfer": "pcie_through::fused_memcpy_multi_layer_block_transfer(Tensor "
                                                   "deviceBlockCachePtrs, Tensor hostBlockCache, Tensor "
                                                   "stagingBlockCache, int? aiv=None) -> ()",
    }
    for name, schema in want.items():
        op = getattr(torch.ops.pcie_through, name)
        assert str(op.default._schema) == schema
    assert hasattr(torch.ops.pcie_through, "swap_blocks") and hasattr(torch.ops.pcie_through, "gather_blocks")


def test_flag_constants_match_the_header():
    import pcie_through
    text = open(os.path.join(ROOT, "include", "hfk.h")).read()
    for name in ("SWAP_DST_HOST", "SWAP_SRC_HOST", "SWAP_BESIDE_COMPUTE", "SWAP_SRC_DEVICE", "SWAP_DST_DEVICE"):
        value = int(re.search(r"#define HFK_%s (\d+)u" % name, text).group(1))
        assert getattr(pcie_through, name) == value == getattr(capi, name)


def test_swap_flags_helper_reads_the_sides_off_the_planes():
    import pcie_through
    host = [torch.zeros(4), torch.zeros(4)]

    class Dev:                                         # stands for a device plane: is_cuda is all the helper reads
        is_cuda = True
    assert pcie_through.swap_flags(host, [Dev(), Dev()]) == pcie_through.SWAP_DST_HOST
    assert pcie_through.swap_flags([Dev()], host) == pcie_through.SWAP_SRC_HOST
    assert pcie_through.swap_flags([Dev()], [Dev()]) == 0
    assert pcie_through.swap_flags(host, [Dev()], beside_compute=True) == \
        pcie_through.SWAP_DST_HOST | pcie_through.SWAP_BESIDE_COMPUTE
    with pytest.raises(ValueError):
        pcie_through.swap_flags(host + [Dev()], [Dev()])


def test_ops_have_no_cpu_fallback():
    import pcie_through  # noqa: F401

    with pytest.raises(NotImplementedError):
        torch.ops.pcie_through.gather(torch.zeros(4, 4), torch.zeros(2, 4), torch.zeros(2, dtype=torch.int64))
    with pytest.raises(NotImplementedError):
        torch.ops.pcie_through.multi_layer_block_transfer(torch.zeros(2, dtype=torch.int64),
                                                          torch.zeros(2, 2, 2, 2), 4)


def test_package_layout():
    import pcie_through

    pkg = os.path.dirname(pcie_through.__file__)
    assert os.path.exists(os.path.join(pkg, "lib", "libpcie_through.so"))   # pcie_through/_load.py:10
    from heterofusedkernels import memory

    for name in ("alloc_numa_pinned_tensor", "host_register", "get_device_ptr"):  # common/csrc/pybind.cpp:8-10
        assert callable(getattr(memory, name))
    assert os.path.dirname(pkg) == heterofusedkernels_amd.DROPIN_DIR


def test_pageable_memory_is_refused_and_leaves_no_record():
    """The library adopts pinned memory and allocates its own; it never pins existing pageable memory."""
    L = ctypes.CDLL(_build.MANAGED_MEMORY_SO)
    L.hfk_mm_register.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.POINTER(ctypes.c_void_p)]
    L.hfk_mm_get_device_ptr.argtypes = [ctypes.c_void_p]
    L.hfk_mm_get_device_ptr.restype = ctypes.c_void_p
    L.hfk_mm_record_count.restype = ctypes.c_size_t
    L.hfk_mm_status_string.restype = ctypes.c_char_p
    text = open(os.path.join(ROOT, "include", "hfk_managed_memory.h")).read()
    not_pinned = int(re.search(r"HFK_MM_ERR_NOT_PINNED = (-\d+)", text).group(1))
    buf = ctypes.create_string_buffer(1 << 16)             # plain malloc'd memory
    before = L.hfk_mm_record_count()
    dev = ctypes.c_void_p(0)
    assert L.hfk_mm_register(buf, len(buf), ctypes.byref(dev)) == not_pinned
    assert not dev.value
    assert L.hfk_mm_record_count() == before
    assert not L.hfk_mm_get_device_ptr(ctypes.addressof(buf))
    assert b"alloc_pinned" in L.hfk_mm_status_string(not_pinned)


# ---- registry (no HIP call is made by adopt / lookup) ------------------------
@pytest.fixture
def mm():
    L = ctypes.CDLL(_build.MANAGED_MEMORY_SO)
    L.hfk_mm_adopt.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    L.hfk_mm_unregister.argtypes = [ctypes.c_void_p]
    L.hfk_mm_get_device_ptr.argtypes = [ctypes.c_void_p]
    L.hfk_mm_get_device_ptr.restype = ctypes.c_void_p
    L.hfk_mm_record_size.argtypes = [ctypes.c_void_p]
    L.hfk_mm_record_size.restype = ctypes.c_size_t
    L.hfk_mm_record_count.restype = ctypes.c_size_t
    L.hfk_mm_status_string.restype = ctypes.c_char_p
    L.hfk_mm_unregister_all()
    yield L
    L.hfk_mm_unregister_all()


def test_registry_range_lookup_and_offsets(mm):
    # common/csrc/managed_memory/managed_mem.cpp:139-160: interior pointers resolve by offset
    assert mm.hfk_mm_adopt(0x10000, 0x900000, 0x1000, 0) == 0
    assert mm.hfk_mm_adopt(0x30000, 0xA00000, 0x2000, 0) == 0
    assert mm.hfk_mm_get_device_ptr(0x10000) == 0x900000
    assert mm.hfk_mm_get_device_ptr(0x10fff) == 0x900fff
    assert mm.hfk_mm_get_device_ptr(0x11000) is None          # one past the end
    assert mm.hfk_mm_get_device_ptr(0xffff) is None
    assert mm.hfk_mm_get_device_ptr(0x31234) == 0xA01234
    assert mm.hfk_mm_get_device_ptr(0) is None                 # :140-142
    assert mm.hfk_mm_record_size(0x30010) == 0x2000            # :163-179
    assert mm.hfk_mm_record_size(0x50000) == 0
    assert mm.hfk_mm_record_count() == 2


def test_registry_idempotent_overlap_and_unregister(mm):
    assert mm.hfk_mm_adopt(0x10000, 0x900000, 0x1000, 0) == 0
    assert mm.hfk_mm_adopt(0x10000, 0x123456, 0x1000, 0) == 0   # :49-52 same start: existing record kept
    assert mm.hfk_mm_get_device_ptr(0x10000) == 0x900000
    assert mm.hfk_mm_adopt(0x10800, 0x777000, 0x1000, 0) == -2  # overlaps a different record
    assert mm.hfk_mm_adopt(0xf800, 0x777000, 0x1000, 0) == -2
    assert mm.hfk_mm_adopt(0, 0x777000, 0x1000, 0) == -1        # :46 null / zero size rejected
    assert mm.hfk_mm_adopt(0x70000, 0x777000, 0, 0) == -1
    assert mm.hfk_mm_unregister(0x424242) == 0                  # :110-113 unknown pointer is not an error
    assert mm.hfk_mm_unregister(0x10000) == 0
    assert mm.hfk_mm_get_device_ptr(0x10000) is None
    assert mm.hfk_mm_record_count() == 0
    assert b"overlap" in mm.hfk_mm_status_string(-2)


def test_registry_adopted_record_grows_but_never_into_its_neighbour(mm):
    assert mm.hfk_mm_adopt(0x10000, 0x900000, 0x1000, 0) == 0
    assert mm.hfk_mm_adopt(0x14000, 0xA00000, 0x1000, 0) == 0
    assert mm.hfk_mm_adopt(0x10000, 0x900000, 0x3000, 0) == 0      # same start, longer: record grows
    assert mm.hfk_mm_record_size(0x10000) == 0x3000
    assert mm.hfk_mm_get_device_ptr(0x12fff) == 0x902fff
    assert mm.hfk_mm_adopt(0x10000, 0x900000, 0x5000, 0) == 0      # would run into 0x14000: size kept
    assert mm.hfk_mm_record_size(0x10000) == 0x3000
    assert mm.hfk_mm_get_device_ptr(0x14010) == 0xA00010
    assert mm.hfk_mm_adopt(0x10000, 0x900000, 0x800, 0) == 0       # shorter: unchanged
    assert mm.hfk_mm_record_size(0x10000) == 0x3000


def test_registry_is_thread_safe(mm):
    # managed_mem.h:31: writers exclude, readers share
    errors = []

    def worker(k):
        base = 0x1000000 * (k + 1)
        try:
            for i in range(300):
                host = base + i * 0x2000
                assert mm.hfk_mm_adopt(host, host + 0x5000000000, 0x1000, k) == 0
                assert mm.hfk_mm_get_device_ptr(host + 0x10) == host + 0x5000000000 + 0x10
                if i % 3 == 0:
                    assert mm.hfk_mm_unregister(host) == 0
        except AssertionError as exc:  # pragma: no cover
            errors.append(exc)

    threads = [threading.Thread(target=worker, args=(k,)) for k in range(8)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors
    assert mm.hfk_mm_record_count() == 8 * 200


def test_memory_module_cpu_behaviour():
    from heterofusedkernels import memory

    assert memory.get_device_ptr(0x1234) == 0                    # managed_mem.cpp:372-375
    with pytest.raises(RuntimeError, match="Device must be CPU and tensor must be pinned"):
        memory.host_register(torch.zeros(16))                    # managed_mem.cpp:336-340


def test_public_headers_are_strict_c99(tmp_path):
    """A foreign runtime binds the headers from C: they must compile as C99 with -pedantic -Werror,
    alone and in either order."""
    src = tmp_path / "headers.c"
    for order in (("hfk.h", "hfk_managed_memory.h"), ("hfk_managed_memory.h", "hfk.h")):
        src.write_text("".join('#include "%s"\n' % h for h in order) + "int main(void) { return HFK_OK + HFK_MM_OK; }\n")
        subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only",
                        "-I" + _build.INCLUDE, str(src)], check=True)


def test_c_client_fails_cleanly_without_a_gpu():
    """The plain-C client links against the two libraries and, with no device, stops at its first HIP call
    with a message and a non-zero status (no crash)."""
    if torch.cuda.is_available():
        pytest.skip("a GPU is present; the GPU test runs the client for real")
    proc = subprocess.run([_build.C_CLIENT], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert proc.returncode == 2, (proc.returncode, proc.stdout, proc.stderr)
    assert "hipSetDevice" in proc.stderr
