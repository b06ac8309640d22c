"""PJRT plugin, host side: the exported table, its layout against the OpenXLA header, and
every case of the driver that needs no device (tests/pjrt/pjrt_driver.cpp restates the
reference's Tests/PJRTMetalHLOTests/PJRTPluginTests.swift)."""
import ctypes
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PLUGIN = os.path.join(ROOT, "metalhlo_amd", "lib", "libPJRTMetalHLO.so")
DRIVER = os.path.join(ROOT, "tests", "pjrt", "pjrt_driver")
# a copy of the OpenXLA PJRT C API header (v0.90), when one is around
HEADERS = [os.environ.get("PJRT_C_API_HEADER", ""), "/root/reference/Sources/CPJRTApi/include/pjrt_c_api.h"]


def _need_built():
    if not (os.path.exists(PLUGIN) and os.path.exists(DRIVER)):
        pytest.fail("libPJRTMetalHLO.so / pjrt_driver are not built: run __graft_entry__.build()")


def test_plugin_exports_getpjrtapi_and_a_1064_byte_table():
    _need_built()
    lib = ctypes.CDLL(PLUGIN)
    lib.GetPjrtApi.restype = ctypes.c_void_p
    api = lib.GetPjrtApi()
    assert api and lib.GetPjrtApi() == api
    words = (ctypes.c_uint64 * 5).from_address(api)
    assert words[0] == 1064                      # struct_size: 3 header words + version struct + 130 slots
    assert words[1] == 0                         # no extensions
    assert words[2] == 24                        # PJRT_Api_Version.struct_size
    major, minor = (ctypes.c_int32 * 2).from_address(api + 32)
    assert (major, minor) == (0, 90)
    slots = (ctypes.c_uint64 * 130).from_address(api + 40)
    assert sum(1 for s in slots if s) == 94      # functions offered; the others are NULL


def test_abi_header_matches_the_openxla_header():
    header = next((h for h in HEADERS if h and os.path.exists(h)), None)
    if header is None or shutil.which("g++") is None:
        pytest.skip("no pjrt_c_api.h to compare with (set PJRT_C_API_HEADER)")
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-I", os.path.join(ROOT, "include"),
                        f'-DPJRT_REFERENCE_HEADER="{header}"', os.path.join(ROOT, "tests", "pjrt", "layout_check.cpp")],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]


def test_abi_header_is_plain_c():
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    r = subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", "-fsyntax-only", "-x", "c", os.path.join(ROOT, "include", "pjrt_abi.h")],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-3000:]


def test_driver_host_cases():
    _need_built()
    env = dict(os.environ, METALHLO_ALLOW_NO_DEVICE="1", HIP_VISIBLE_DEVICES="")
    r = subprocess.run([DRIVER, PLUGIN, "host"], capture_output=True, text=True, env=env, timeout=120)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-3000:]
    for case in ("table", "errors", "platform", "compile", "no_device_buffers", "all"):
        assert f"ok {case}\n" in r.stdout, r.stdout
