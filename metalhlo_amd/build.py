"""Builds the gfx950 kernel library (``libmetalhlo_hip.so``) and the C++ host
libraries in-tree with hipcc / g++.  ``python -m metalhlo_amd.build`` rebuilds
everything; nothing here needs a GPU (hipcc cross-compiles)."""
from __future__ import annotations

import os
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
ROOT = os.path.dirname(HERE)

HIP_SOURCES = ["runtime.hip", "row_kernels.hip", "gemm.hip", "gemm_f32.hip", "gemm256.hip", "gemm_twoset.hip", "tuning.hip", "attention.hip", "attention_pipe.hip", "attention_f32.hip", "glue_kernels.hip", "elementwise.hip", "fused_misc.hip"]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=fast",
    # packed fp32 VALU forms are kept out of generated code on this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument", "-Wno-unknown-warning-option",
]


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + r.stdout + r.stderr)
        raise RuntimeError("build step failed: " + os.path.basename(cmd[-1]))
    noisy = [l for l in r.stderr.splitlines()
             if l.strip() and "packed-fp32-ops" not in l and "is not a recognized feature" not in l]
    if noisy:
        sys.stderr.write("\n".join(noisy) + "\n")


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.isabs(cand) and os.path.exists(cand) or not os.path.isabs(cand)):
            return cand
    return "hipcc"


def _exports(lib: str) -> str:
    """Linker option that limits a library's dynamic symbols to its C-ABI (csrc/exports/<lib>.map)."""
    return "-Wl,--version-script=" + os.path.join(CSRC, "exports", lib + ".map")


def generate_sources(verbose: bool = True) -> None:
    """Regenerates the hand-scheduled loops included by gemm256.hip, gemm_twoset.hip and attention_pipe.hip."""
    for script, args, target in (("gen_gemm256_loop.py", [], "gemm256_loop.inc"),
                                 ("gen_gemm256_loop.py", ["two_set"], "gemm_twoset_loop.inc"),
                                 ("gen_fa_loop.py", [], "fa_loop.inc")):
        r = subprocess.run([sys.executable, os.path.join(CSRC, script), *args], capture_output=True, text=True)
        if r.returncode != 0:
            sys.stderr.write(r.stderr)
            raise RuntimeError("build step failed: " + script)
        out = os.path.join(CSRC, target)
        old = open(out).read() if os.path.exists(out) else None
        if old != r.stdout:
            with open(out, "w") as f:
                f.write(r.stdout)
        if verbose:
            print("  gen   " + target, flush=True)


def build_kernels(verbose: bool = True) -> str:
    os.makedirs(LIBDIR, exist_ok=True)
    generate_sources(verbose)
    objdir = tempfile.mkdtemp(prefix="mhip_obj_")
    srcs = [s for s in HIP_SOURCES if os.path.exists(os.path.join(CSRC, s))]
    objs = [os.path.join(objdir, s.replace(".hip", ".o")) for s in srcs]

    def one(pair):
        src, obj = pair
        _run([hipcc(), *HIPCC_FLAGS, "-I", os.path.join(ROOT, "include"), "-c",
              os.path.join(CSRC, src), "-o", obj])
        if verbose:
            print("  hipcc", src, flush=True)

    with ThreadPoolExecutor(max_workers=min(8, len(srcs))) as ex:
        list(ex.map(one, zip(srcs, objs)))
    out = os.path.join(LIBDIR, "libmetalhlo_hip.so")
    # (-z defs: a kernel whose host-side launch stub was not emitted must fail here, not at load time)
    _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-Wl,-z,defs", _exports("libmetalhlo_hip"), "-o", out, *objs])
    if verbose:
        print("  link ", os.path.relpath(out, ROOT), flush=True)
    return out


def build_host(verbose: bool = True) -> list:
    """C++ host libraries above the kernel C-ABI (built when their sources exist)."""
    outs = []
    host = os.path.join(CSRC, "host")
    if not os.path.isdir(host):
        return outs
    srcs = sorted(os.path.join(host, f) for f in os.listdir(host) if f.endswith(".cpp"))
    if not srcs:
        return outs
    out = os.path.join(LIBDIR, "libCMetalHLO.so")
    _run([hipcc(), "-x", "c++", "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__", "-Wall",
          "-I", os.path.join(ROOT, "include"), "-I", "/opt/rocm/include", *srcs,
          "-shared", _exports("libCMetalHLO"), "-o", out, "-L", LIBDIR, "-lmetalhlo_hip", "-L", "/opt/rocm/lib", "-lamdhip64",
          "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"])
    if verbose:
        print("  link ", os.path.relpath(out, ROOT), flush=True)
    outs.append(out)
    # the PJRT plugin: same parser / executor, its own boundary file instead of the mhlo_* one
    pjrt = os.path.join(CSRC, "pjrt", "pjrt.cpp")
    if os.path.exists(pjrt):
        out = os.path.join(LIBDIR, "libPJRTMetalHLO.so")
        _run([hipcc(), "-x", "c++", "-O2", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__", "-Wall",
              "-I", os.path.join(ROOT, "include"), "-I", "/opt/rocm/include", pjrt,
              *[f for f in srcs if os.path.basename(f) != "capi.cpp"],
              "-shared", _exports("libPJRTMetalHLO"), "-o", out, "-L", LIBDIR, "-lmetalhlo_hip", "-L", "/opt/rocm/lib", "-lamdhip64",
              "-Wl,-rpath,$ORIGIN", "-Wl,-rpath,/opt/rocm/lib"])
        if verbose:
            print("  link ", os.path.relpath(out, ROOT), flush=True)
        outs.append(out)
        # the test program that drives the plugin through its function table (tests/test_pjrt_*.py)
        drv_src = os.path.join(ROOT, "tests", "pjrt", "pjrt_driver.cpp")
        if os.path.exists(drv_src):
            drv = os.path.join(ROOT, "tests", "pjrt", "pjrt_driver")
            _run(["g++", "-O1", "-g", "-std=c++17", "-Wall", "-pthread", "-rdynamic", "-I", os.path.join(ROOT, "include"), drv_src, "-o", drv, "-ldl"])
            if verbose:
                print("  link ", os.path.relpath(drv, ROOT), flush=True)
    return outs


def build_all(verbose: bool = True):
    """The product: the HIP kernel library and the host libraries over it."""
    build_kernels(verbose)
    build_host(verbose)


if __name__ == "__main__":
    build_all()
