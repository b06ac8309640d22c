"""CPU checks of the drop-in boundary: the shared library loads without a GPU,
exports every symbol include/mhip.h declares, and rejects bad arguments before
anything could be launched."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    src = open(os.path.join(ROOT, "include", header)).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(m(?:hip|hlo)_[a-z0-9_]+)\s*\(", src)))


def test_library_exports_every_declared_symbol(lib):
    names = _declared("mhip.h")
    assert len(names) >= 19
    for n in names:
        assert hasattr(lib, n), f"libmetalhlo_hip.so lacks {n}"
    from metalhlo_amd import _lib
    assert sorted(_lib.SIGNATURES) == names, "ctypes table and header disagree"


def test_version_and_device_queries_without_gpu(lib):
    assert lib.mhip_version().decode().startswith("0.")
    n = lib.mhip_device_count()
    assert n >= 0
    if n == 0:
        cus = C.c_int(0)
        assert lib.mhip_device_info(0, C.byref(cus), None, None, 0) == 4      # MHIP_ERR_NO_DEVICE
        assert b"no HIP device" in lib.mhip_last_error()


def test_argument_validation_needs_no_gpu(lib):
    # negative sizes, NULL tensors and unknown enums are rejected on the host
    assert lib.mhip_softmax(None, None, None, -1, 4, 3) == 1
    assert lib.mhip_softmax(None, None, None, 4, 4, 3) == 1 and b"NULL" in lib.mhip_last_error()
    assert lib.mhip_softmax(None, None, None, 0, 4, 3) == 0                    # empty: no-op
    assert lib.mhip_layer_norm(None, None, None, None, None, 2, 2, 1e-5, 3) == 1
    assert lib.mhip_rms_norm(None, None, None, None, 2, -2, 1e-5, 3) == 1
    assert lib.mhip_bias_gelu(None, None, None, None, 2, 2, 3) == 1
    assert lib.mhip_gemm(None, None, None, None, None, 4, 4, 4, 1, 0, 0, 0, 0, 0, 0, 3) == 1
    assert lib.mhip_gemm(None, None, None, None, None, 4, 4, 4, 1, 0, 0, 0, 0, 0, 42, 3) == 1
    assert lib.mhip_gemm(None, None, None, None, None, 0, 4, 4, 1, 0, 0, 0, 0, 0, 0, 3) == 0
    assert lib.mhip_flash_attention(None, None, None, None, None, None, 1, 1, 8, 8, 64, 1.0, 0, 0, 0, 3) == 1
    assert lib.mhip_flash_attention(None, None, None, None, None, None, 1, 1, 8, 8, 0, 1.0, 0, 0, 0, 3) == 1
    buf = (C.c_char * 64)()
    p = C.addressof(buf)
    assert lib.mhip_flash_attention(None, p, p, p, None, p, 1, 1, 1, 1, 512, 1.0, 0, 0, 0, 3) == 2
    assert lib.mhip_softmax(None, p, p, 2, 2, 8) == 2 and b"dtype" in lib.mhip_last_error()
    assert lib.mhip_gather_rows(None, None, None, None, 1, 1, 1, 1, 7) == 1
    assert lib.mhip_convert(None, None, None, 4, 1, 3) == 1
    assert lib.mhip_argmax(None, None, None, None, 1, 0, 1, 7) == 1


def test_missing_library_fails_loudly(monkeypatch):
    from metalhlo_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmetalhlo_hip.so")
    with pytest.raises(ImportError, match="metalhlo_amd.build"):
        _lib.load()


def test_host_wrappers_refuse_cpu_tensors():
    import torch
    from metalhlo_amd import kernels
    with pytest.raises(RuntimeError, match="no CPU path"):
        kernels.softmax(torch.zeros(2, 2))


def _exported(libname):
    import subprocess
    path = os.path.join(ROOT, "metalhlo_amd", "lib", libname)
    out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True, check=True).stdout
    return sorted(line.split()[-1] for line in out.splitlines() if line.strip())


def test_libraries_export_their_c_abi_and_nothing_else():
    """The sealed boundary: the kernel library exports exactly the mhip_* functions of include/mhip.h,
    the C API library exactly the mhlo_* functions of include/metalhlo.h, the PJRT plugin the one
    symbol GetPjrtApi (Sources/PJRTMetalHLO/PJRTApi.swift:170-173).  The C API library and the
    plugin contain the same C++ host; with its symbols private, a process that loads both gets
    two independent copies instead of one library's calls bound to the other's definitions."""
    assert _exported("libmetalhlo_hip.so") == _declared("mhip.h")
    assert _exported("libCMetalHLO.so") == _declared("metalhlo.h")
    assert _exported("libPJRTMetalHLO.so") == ["GetPjrtApi"]


def test_reference_c_example_builds_against_this_header_and_library(tmp_path):
    """The reference's own C program (Examples/CExample/main.c, which includes "metalhlo.h" and
    calls the mhlo_* API) compiles against include/metalhlo.h and links against libCMetalHLO.so
    unchanged.  Needs the reference tree (METALHLO_REFERENCE, default /root/reference); the file
    is read where it lies, never copied.  Running it needs a GPU and is not part of this check."""
    import subprocess
    ref = os.environ.get("METALHLO_REFERENCE", "/root/reference")
    src = os.path.join(ref, "Examples", "CExample", "main.c")
    if not os.path.exists(src):
        pytest.skip("the reference tree is not present")
    exe = str(tmp_path / "cexample")
    libdir = os.path.join(ROOT, "metalhlo_amd", "lib")
    r = subprocess.run(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), src, "-o", exe,
                        "-L", libdir, "-lCMetalHLO", "-Wl,-rpath," + libdir, "-Wl,-rpath-link," + libdir,
                        "-Wl,-rpath-link,/opt/rocm/lib", "-lm"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]
    undefined = subprocess.run(["nm", "-u", exe], capture_output=True, text=True, check=True).stdout
    used = sorted(set(re.findall(r"\b(mhlo_[a-z_]+)", undefined)))
    assert len(used) >= 15 and set(used) <= set(_declared("metalhlo.h")), used
