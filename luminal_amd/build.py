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
# Code object with the matvec kernels under C names, for hosts that launch through hipModule* themselves.
MODULE_SRC = os.path.join(CSRC, "module", "q8_gemv_module.hip")
MODULE = os.path.join(HERE, "luminal_hip_kernels.hsaco")

ARCH = "gfx950"
# Packed-FP32 instructions are switched off for all device code.
DEVICE_FLAGS = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
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


def build(verbose: bool = True) -> str:
    srcs = sources()
    if not srcs:
        raise RuntimeError(f"no HIP sources under {CSRC}")
    cc = hipcc()
    if verbose:
        print(f"[luminal_amd.build] {cc} -> {LIB}", file=sys.stderr)
    _run([cc, *COMMON, *DEVICE_FLAGS, "-shared", "-o", LIB, *srcs])
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
    build()
    build_host_test()
