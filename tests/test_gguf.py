"""GGUF reader against files made by the writer (the reference ships no GGUF fixtures: *.gguf is git-ignored
there), for every header version, alignment handling and the error cases the reference panics on."""
import io
import struct

import numpy as np
import pytest

from luminal_amd import gguf, synth


def sample_tensors():
    qs, d = synth.q8_0_random(4, 64, seed=1)
    return {"a.weight": ("F32", (5,), np.arange(5, dtype="<f4").tobytes()),
            "blk.0.attn_q.weight": ("Q8_0", (64, 4), synth.q8_0_raw_blocks(qs, d).tobytes())}, qs, d


@pytest.mark.parametrize("version", [1, 2, 3])
@pytest.mark.parametrize("alignment", [None, 64, 8])
def test_round_trip_all_versions(tmp_path, version, alignment):
    tensors, qs, d = sample_tensors()
    md = {"general.architecture": "llama", "llama.block_count": 1, "flag": True, "eps": 1e-5, "neg": -3,
          "tokens": ["a", "bc"], "ids": [1, 2, 3]}
    p = tmp_path / "t.gguf"
    gguf.write_gguf(p, md, tensors, version=version, alignment=alignment)
    with open(p, "rb") as f:
        c = gguf.Content.read(f)
        assert c.version == version
        assert c.metadata["general.architecture"] == "llama" and c.metadata["llama.block_count"] == 1
        assert c.metadata["flag"] is True and c.metadata["neg"] == -3 and c.metadata["tokens"] == ["a", "bc"]
        assert c.metadata["ids"] == [1, 2, 3] and abs(c.metadata["eps"] - 1e-5) < 1e-12
        a = alignment or 32
        assert c.tensor_data_offset % a == 0
        info = c.tensor_infos["blk.0.attn_q.weight"]
        assert (info.n_elements, info.dtype, info.dims) == (256, "Q8_0", (64, 4))
        assert gguf.tensor_nbytes(info) == 256 + 16  # n + n/16
        assert np.array_equal(gguf.read_tensor(f, c, "a.weight"), np.arange(5, dtype=np.float32))
        assert np.array_equal(gguf.read_tensor(f, c, "blk.0.attn_q.weight"), synth.q8_0_raw_blocks(qs, d))


def test_errors_the_reference_panics_on(tmp_path):
    with pytest.raises(gguf.GgufError, match="unknown magic"):
        gguf.Content.read(io.BytesIO(struct.pack("<II", 0x12345678, 3)))
    with pytest.raises(gguf.GgufError, match="unsupported version"):
        gguf.Content.read(io.BytesIO(struct.pack("<II", gguf.MAGIC, 4)))
    with pytest.raises(gguf.GgufError, match="end of file"):
        gguf.Content.read(io.BytesIO(struct.pack("<IIQ", gguf.MAGIC, 3, 1)))
    # byte-swapped magic is accepted like in the reference (0x47475546)
    gguf.Content.read(io.BytesIO(struct.pack("<IIQQ", 0x47475546, 3, 0, 0)))
    # unknown ggml dtype code
    bad = struct.pack("<IIQQ", gguf.MAGIC, 3, 1, 0) + struct.pack("<Q", 1) + b"x" + struct.pack("<IQIQ", 1, 4, 99, 0)
    with pytest.raises(gguf.GgufError, match="unknown dtype"):
        gguf.Content.read(io.BytesIO(bad))
    # a dtype the loader does not support (only F32 and Q8_0, loader.rs:124-131)
    with pytest.raises(gguf.GgufError, match="Unsupported dtype"):
        gguf.tensor_nbytes(gguf.TensorInfo(32, 0, "Q4_0", (32,)))


def test_llama_tensor_names_follow_the_reference_paths():
    names = gguf.llama_tensor_names(2)
    assert names[:3] == ["token_embd.weight", "output_norm.weight", "output.weight"]
    assert "blk.1.attn_output.weight" in names and "blk.0.ffn_gate.weight" in names and len(names) == 3 + 2 * 9
