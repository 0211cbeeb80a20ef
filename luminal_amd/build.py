"""Build recipe of libluminal_hip.so (hipcc, gfx950 only).

``python -m luminal_amd.build`` compiles every HIP source under ``csrc/`` into
one shared library beside this file.  The kernels are C++ templates launched by
the library's own ``extern "C"`` entry points; callers bind those entry points,
not the kernels.
"""
from __future__ import annotations

import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libluminal_hip.so")
OBJ_DIR = os.path.join(HERE, "build")  # objects, one per source (not tracked)
# Code object with the matvec kernels under C names, for hosts that launch through hipModule* themselves.
MODULE_SRC = os.path.join(CSRC, "module", "q8_gemv_module.hip")
MODULE = os.path.join(HERE, "luminal_hip_kernels.hsaco")

ARCH = "gfx950"
# Packed-FP32 instructions are switched off for all device code.  The leading scalar arguments of a kernel (up to 16
# dwords, until the first by-value struct) are preloaded into SGPRs by the command processor instead of being loaded
# by every wave's first instructions: measured 0.25 us per launch on the 4096 x 4096 matvec (5.65 -> 5.40 us), 0.06 to
# 0.1 us on the other single-weight shapes; kernels whose first argument is a struct are unaffected, and a part whose
# firmware lacks the feature runs the loads the compiler keeps in front of the kernel.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-mllvm", "-amdgpu-kernarg-preload-count=16"]
COMMON = ["-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-command-line-argument", f"--offload-arch={ARCH}"]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def sources() -> list[str]:
    return sorted(glob.glob(os.path.join(CSRC, "*.hip")))


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # The host pass does not know the device-only feature flag and says so: harmless.
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("build failed: " + " ".join(cmd) + "\n" + out)
    if out.strip():
        print(out, file=sys.stderr)


def _object_path(src: str) -> str:
    return os.path.join(OBJ_DIR, os.path.splitext(os.path.basename(src))[0] + ".o")


def _headers() -> list[str]:
    return glob.glob(os.path.join(CSRC, "*.h")) + glob.glob(os.path.join(os.path.dirname(HERE), "include", "*.h"))


def build(verbose: bool = True, incremental: bool = False, jobs: int | None = None) -> str:
    """Compile every source to an object (in parallel), then link.  ``incremental`` skips a source whose object is
    newer than it and than every header; the default recompiles everything."""
    from concurrent.futures import ThreadPoolExecutor

    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    cc = hipcc()
    os.makedirs(OBJ_DIR, exist_ok=True)
    newest_header = max((os.path.getmtime(h) for h in _headers()), default=0.0)

    def stale(src: str) -> bool:
        obj = _object_path(src)
        return not (incremental and os.path.exists(obj) and
                    os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header))

    todo = [s for s in srcs if stale(s)]
    if verbose:
        print(f"[luminal_amd.build] {cc}: {len(todo)} of {len(srcs)} sources -> {LIB}", file=sys.stderr)
    jobs = jobs or min(8, os.cpu_count() or 1, int(os.environ.get("MAX_JOBS", "8")))
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        list(pool.map(lambda s: _run([cc, *COMMON, *DEVICE_FLAGS, "-c", "-o", _object_path(s), s]), todo))
    _run([cc, *COMMON, "-shared", "-o", LIB, *[_object_path(s) for s in srcs]])
    if todo or not os.path.exists(MODULE):
        build_module(verbose)
    return LIB


def build_module(verbose: bool = True) -> str:
    """Device-only compile of the kernel module into a plain gfx950 ELF code object."""
    if verbose:
        print(f"[luminal_amd.build] {hipcc()} -> {MODULE}", file=sys.stderr)
    _run([hipcc(), "--cuda-device-only", "--no-gpu-bundle-output", "-O3", "-std=c++17", f"--offload-arch={ARCH}",
          *DEVICE_FLAGS, "-o", MODULE, MODULE_SRC])
    return MODULE


HOST_TEST_SRC = os.path.join(os.path.dirname(HERE), "tests", "cpp", "host_mirror_test.cpp")
HOST_TEST_BIN = os.path.join(os.path.dirname(HERE), "tests", "cpp", "_build", "host_mirror_test")


def build_host_test(verbose: bool = True) -> str:
    """Compile the test program of the C++ host mirror (host/luminal_hip.hpp) with the host compiler; it links
    against libluminal_hip.so only."""
    cxx = os.environ.get("CXX") or shutil.which("g++") or shutil.which("c++")
    if not cxx:
        raise RuntimeError("no host C++ compiler found (g++)")
    os.makedirs(os.path.dirname(HOST_TEST_BIN), exist_ok=True)
    if verbose:
        print(f"[luminal_amd.build] {cxx} -> {HOST_TEST_BIN}", file=sys.stderr)
    _run([cxx, "-std=c++17", "-O1", "-Wall", "-o", HOST_TEST_BIN, HOST_TEST_SRC, "-L" + HERE, "-lluminal_hip",
          "-Wl,-rpath," + HERE, "-Wl,-rpath,$ORIGIN/../../../luminal_amd"])
    return HOST_TEST_BIN


if __name__ == "__main__":
    build(incremental="--incremental" in sys.argv)
    build_host_test()
