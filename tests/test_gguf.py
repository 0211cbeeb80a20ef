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


def literal_bytes():
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "gguf_v3_literal.hex")
    with open(path) as f:
        return b"".join(bytes.fromhex(line.split("#")[0]) for line in f)


def test_hand_assembled_v3_file(oracle):
    """A file written out byte by byte from examples/llama/src/gguf.rs:190-263 (not by write_gguf): one key of every
    value type, nested arrays, a string with a trailing NUL, alignment 64, one F32 and one Q8_0 tensor."""
    b = literal_bytes()
    assert len(b) == 644
    f = io.BytesIO(b)
    c = gguf.Content.read(f)
    assert c.version == 3 and len(c.metadata) == 15
    md = c.metadata
    assert (md["u8"], md["i8"], md["u16"], md["i16"], md["u32"], md["i32"]) == (254, -128, 65534, -2, 4000000000, -5)
    assert md["f32"] == 1.5 and md["bool"] is True and md["str"] == "ab" and md["arr"] == ["x", "yz"]
    assert md["u64"] == 2 ** 40 + 1 and md["i64"] == -1 and md["f64"] == 0.25 and md["nest"] == [[7, 8]]
    assert md["general.alignment"] == 64 and c.tensor_data_offset == 512  # 477 header bytes rounded up to 64
    a, q = c.tensor_infos["a.weight"], c.tensor_infos["blk.0.attn_q.weight"]
    assert (a.n_elements, a.offset, a.dtype) == (3, 0, "F32")
    assert (q.n_elements, q.offset, q.dtype, q.dims) == (64, 64, "Q8_0", (32, 2))
    assert np.array_equal(gguf.read_tensor(f, c, "a.weight"), np.array([1.0, -2.0, 0.5], np.float32))
    raw = gguf.read_tensor(f, c, "blk.0.attn_q.weight")
    assert raw.size == 68
    w = oracle.q8_0_dequant(raw, 64).reshape(2, 32)
    assert np.array_equal(w[0], 0.5 * np.arange(32, dtype=np.float32))
    assert np.array_equal(w[1], -2.0 * np.arange(-16, 16, dtype=np.float32))


def test_alignment_key_types(tmp_path):
    # only 8/16/32-bit integer types set the alignment (gguf.rs:246-255): a u64 value is ignored
    b = bytearray(literal_bytes())
    at = bytes(b).index(b"general.alignment") + 17
    assert bytes(b[at:at + 8]) == struct.pack("<II", 4, 64)
    head = bytes(b[:at]) + struct.pack("<IQ", 10, 64) + bytes(b[at + 8:477])
    c = gguf.Content.read(io.BytesIO(head))
    assert c.metadata["general.alignment"] == 64 and c.tensor_data_offset == -(-len(head) // 32) * 32
    head = bytes(b[:at]) + struct.pack("<Ii", 5, -64) + bytes(b[at + 8:477])  # negative i32: default
    assert gguf.Content.read(io.BytesIO(head)).tensor_data_offset == -(-len(head) // 32) * 32
    head = bytes(b[:at]) + struct.pack("<IB", 0, 16) + bytes(b[at + 8:477])   # u8 16
    assert gguf.Content.read(io.BytesIO(head)).tensor_data_offset == -(-len(head) // 16) * 16
