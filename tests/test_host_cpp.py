"""The C++ host mirror (luminal_amd/host/*.hpp) through its own test program, tests/cpp/host_mirror_test.cpp:
the compiler passes, the GGUF header reader and the operators' panics without a device, then the reference-style
matvec / gather / matmul checks, a GGUF file through loader and pass, and the fused decoder layer on the GPU."""
import os
import subprocess

import pytest

from luminal_amd import build as lib_build
from luminal_amd import capi


def _binary():
    if not os.path.exists(capi.LIB_PATH):
        pytest.skip("libluminal_hip.so has not been built")
    host_dir = os.path.join(os.path.dirname(capi.LIB_PATH), "host")
    src_time = max([os.path.getmtime(lib_build.HOST_TEST_SRC)] +
                   [os.path.getmtime(os.path.join(host_dir, f)) for f in os.listdir(host_dir) if f.endswith(".hpp")])
    if not os.path.exists(lib_build.HOST_TEST_BIN) or os.path.getmtime(lib_build.HOST_TEST_BIN) < src_time:
        lib_build.build_host_test(verbose=False)
    return lib_build.HOST_TEST_BIN


def _run(mode):
    proc = subprocess.run([_binary(), mode], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0 and "0 failures" in proc.stdout, proc.stdout


def test_compiler_pass_and_panics_without_a_device():
    _run("cpu")


@pytest.mark.gpu
def test_reference_style_checks_on_the_gpu():
    _run("gpu")
