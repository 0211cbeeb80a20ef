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


@pytest.mark.parametrize("version", [1, 2, 3])
@pytest.mark.parametrize("alignment", [None, 64, 8])
def test_cpp_gguf_reader_agrees_with_the_python_one(tmp_path, version, alignment):
    """Files made by the Python writer (every header version, alignment keys, string / array / bool / float metadata)
    read by the C++ reader: version, alignment, data offset and every tensor's element count, offset and dtype code."""
    import numpy as np

    from luminal_amd import gguf, synth

    qs, d = synth.q8_0_random(4, 64, seed=1)
    tensors = {"a.weight": ("F32", (5,), np.arange(5, dtype="<f4").tobytes()),
               "blk.0.attn_q.weight": ("Q8_0", (64, 4), synth.q8_0_raw_blocks(qs, d).tobytes()),
               "output_norm.weight": ("F32", (64,), np.ones(64, dtype="<f4").tobytes())}
    md = {"general.architecture": "llama", "llama.block_count": 1, "flag": True, "eps": 1e-5, "neg": -3,
          "tokens": ["a", "bc"], "ids": [1, 2, 3]}
    path = tmp_path / "t.gguf"
    gguf.write_gguf(path, md, tensors, version=version, alignment=alignment)
    proc = subprocess.run([_binary(), "gguf-header", str(path)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=60)
    assert proc.returncode == 0, proc.stdout
    facts = [line.split() for line in proc.stdout.splitlines()]
    with open(path, "rb") as f:
        c = gguf.Content.read(f)
    assert ["version", str(version)] in facts and ["alignment", str(alignment or 32)] in facts
    assert ["data_offset", str(c.tensor_data_offset)] in facts
    codes = {"F32": 0, "Q8_0": 8}
    seen = {f[1]: (int(f[2]), int(f[3]), int(f[4])) for f in facts if f[0] == "tensor"}
    assert seen == {name: (info.n_elements, info.offset, codes[info.dtype]) for name, info in c.tensor_infos.items()}


def test_cpp_gguf_reader_reports_a_bad_file(tmp_path):
    path = tmp_path / "bad.gguf"
    path.write_bytes(b"GGUF" + (9).to_bytes(4, "little"))
    proc = subprocess.run([_binary(), "gguf-header", str(path)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                          timeout=60)
    assert proc.returncode == 3 and "unsupported version 9" in proc.stdout


@pytest.mark.gpu
def test_reference_style_checks_on_the_gpu():
    _run("gpu")
