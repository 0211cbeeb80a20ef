"""GGUF container: reader, a writer for synthetic test files, and the Llama Q8_0 loader.

Reader = examples/llama/src/gguf.rs:190-263 (Content::read): magic 'GGUF', versions 1-3 (v1 has 32-bit counts
and lengths, v2/v3 64-bit), metadata key/values (value types :207-225), tensor infos (name, dims, ggml dtype,
offset), data section aligned to `general.alignment` (default 32, :9,246-255).  Like the reference it keeps
(n_elements, offset, dtype) per tensor; the dimensions are kept too.  Loader = the `q8_load` of
examples/llama/src/loader.rs:99-165: F32 tensors are read as floats, Q8_0 tensors as n + n/16 raw block bytes
that go to the device untouched (and are re-arranged there by lhip_q8_0_repack); other dtypes are refused.
"""
from __future__ import annotations

import struct
from dataclasses import dataclass

import numpy as np

DEFAULT_ALIGNMENT = 32
MAGIC = 0x46554747  # 'GGUF' little-endian; the byte-swapped form is accepted too, as in the reference

# ggml dtype codes (gguf.rs:283-303)
GGML_DTYPES = {0: "F32", 1: "F16", 2: "Q4_0", 3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 8: "Q8_0", 9: "Q8_1", 10: "Q2K",
               11: "Q3K", 12: "Q4K", 13: "Q5K", 14: "Q6K", 15: "Q8K"}
GGML_CODES = {v: k for k, v in GGML_DTYPES.items()}

# metadata value types (gguf.rs:207-225)
_SCALARS = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 10: "<Q", 11: "<q", 12: "<d"}
_T_BOOL, _T_STRING, _T_ARRAY = 7, 8, 9


class GgufError(ValueError):
    pass


@dataclass
class TensorInfo:
    n_elements: int
    offset: int
    dtype: str
    dims: tuple


class Content:
    def __init__(self, version, metadata, tensor_infos, tensor_data_offset):
        self.version, self.metadata, self.tensor_infos = version, metadata, tensor_infos
        self.tensor_data_offset = tensor_data_offset

    @staticmethod
    def read(f) -> "Content":
        def rd(fmt):
            n = struct.calcsize(fmt)
            b = f.read(n)
            if len(b) != n:
                raise GgufError("unexpected end of file")
            return struct.unpack(fmt, b)[0]

        magic = rd("<I")
        if magic not in (0x46554747, 0x47475546):
            raise GgufError(f"unknown magic 0x{magic:08x}")
        version = rd("<I")
        if version not in (1, 2, 3):
            raise GgufError(f"gguf: unsupported version {version}")
        size = "<I" if version == 1 else "<Q"

        def rd_string():
            n = rd(size)
            b = f.read(n)
            if len(b) != n:
                raise GgufError("unexpected end of file")
            while b.endswith(b"\0"):  # v1 files may carry a terminator
                b = b[:-1]
            return b.decode("utf-8", errors="replace")

        def rd_value(t):
            if t in _SCALARS:
                return rd(_SCALARS[t])
            if t == _T_BOOL:
                b = rd("<B")
                if b not in (0, 1):
                    raise GgufError(f"unexpected bool value {b}")
                return bool(b)
            if t == _T_STRING:
                return rd_string()
            if t == _T_ARRAY:
                et = rd("<I")
                n = rd(size)
                return [rd_value(et) for _ in range(n)]
            raise GgufError(f"unrecognized value-type {t:#08x}")

        tensor_count = rd(size)
        kv_count = rd(size)
        metadata, value_types = {}, {}
        for _ in range(kv_count):
            key = rd_string()
            value_types[key] = rd("<I")
            metadata[key] = rd_value(value_types[key])
        infos = {}
        for _ in range(tensor_count):
            name = rd_string()
            nd = rd("<I")
            dims = tuple(rd("<I" if version == 1 else "<Q") for _ in range(nd))
            code = rd("<I")
            if code not in GGML_DTYPES:
                raise GgufError(f"unknown dtype for tensor {code}")
            offset = rd("<Q")
            infos[name] = TensorInfo(int(np.prod(dims, dtype=np.int64)) if dims else 1, offset, GGML_DTYPES[code], dims)
        pos = f.tell()
        # the reference takes general.alignment from the 8/16/32-bit integer types only, signed ones when they are not
        # negative (gguf.rs:246-255); anything else means the default.  (Zero would divide by zero there: default here.)
        a = metadata.get("general.alignment")
        alignment = a if value_types.get("general.alignment") in (0, 1, 2, 3, 4, 5) and a > 0 else DEFAULT_ALIGNMENT
        return Content(version, metadata, infos, -(-pos // alignment) * alignment)


def tensor_nbytes(info: TensorInfo) -> int:
    """F32: 4 bytes per element; Q8_0: n + n/16 (loader.rs:124-130); anything else is refused."""
    if info.dtype == "F32":
        return info.n_elements * 4
    if info.dtype == "Q8_0":
        return info.n_elements + info.n_elements // 16
    raise GgufError(f"Unsupported dtype: {info.dtype}")


def read_tensor(f, content: Content, name: str) -> np.ndarray:
    """Raw bytes of a tensor: float32 array for F32, uint8 block bytes for Q8_0."""
    info = content.tensor_infos[name]
    n = tensor_nbytes(info)
    f.seek(info.offset + content.tensor_data_offset)
    b = f.read(n)
    if len(b) != n:
        raise GgufError(f"tensor {name}: file too short")
    return np.frombuffer(b, dtype="<f4").copy() if info.dtype == "F32" else np.frombuffer(b, dtype=np.uint8).copy()


# ---------------------------------------------------------------------------- writer (tests)

def write_gguf(path, metadata: dict, tensors: dict, version: int = 3, alignment: int | None = None):
    """tensors: name -> (dtype_name, dims (ggml order: innermost first), bytes-like data)."""
    size = "<I" if version == 1 else "<Q"

    def s(x: str) -> bytes:
        b = x.encode()
        return struct.pack(size, len(b)) + b

    def value(v) -> bytes:
        if isinstance(v, bool):
            return struct.pack("<IB", _T_BOOL, int(v))
        if isinstance(v, int):
            return struct.pack("<II", 4, v) if 0 <= v < 2 ** 32 else struct.pack("<Iq", 11, v)
        if isinstance(v, float):
            return struct.pack("<If", 6, v)
        if isinstance(v, str):
            return struct.pack("<I", _T_STRING) + s(v)
        if isinstance(v, (list, tuple)):  # arrays of strings or u32
            if all(isinstance(e, str) for e in v):
                return struct.pack("<II", _T_ARRAY, _T_STRING) + struct.pack(size, len(v)) + b"".join(s(e) for e in v)
            return struct.pack("<II", _T_ARRAY, 4) + struct.pack(size, len(v)) + b"".join(struct.pack("<I", e) for e in v)
        raise TypeError(type(v))

    md = dict(metadata)
    if alignment is not None:
        md["general.alignment"] = alignment
    align = alignment or DEFAULT_ALIGNMENT
    head = struct.pack("<II", MAGIC, version) + struct.pack(size, len(tensors)) + struct.pack(size, len(md))
    for k, v in md.items():
        head += s(k) + value(v)
    offsets, off = {}, 0
    for name, (dt, dims, data) in tensors.items():
        offsets[name] = off
        off += -(-len(bytes(data)) // align) * align
    for name, (dt, dims, data) in tensors.items():
        head += s(name) + struct.pack("<I", len(dims))
        head += b"".join(struct.pack("<I" if version == 1 else "<Q", d) for d in dims)
        head += struct.pack("<IQ", GGML_CODES[dt], offsets[name])
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (-(-len(head) // align) * align - len(head)))
        for name, (dt, dims, data) in tensors.items():
            b = bytes(data)
            f.write(b)
            f.write(b"\0" * (-(-len(b) // align) * align - len(b)))


# ---------------------------------------------------------------------------- Llama loader

def llama_tensor_names(layers: int):
    """Names the reference's SerializeModule paths give with '/' -> '.' (model.rs:44-50,155-162,201-208,250-258)."""
    names = ["token_embd.weight", "output_norm.weight", "output.weight"]
    for i in range(layers):
        names += [f"blk.{i}.attn_norm.weight", f"blk.{i}.ffn_norm.weight"]
        names += [f"blk.{i}.{p}.weight" for p in ("attn_q", "attn_k", "attn_v", "attn_output", "ffn_gate", "ffn_up",
                                                  "ffn_down")]
    return names


def q8_load(path, cfg, device="cuda:0") -> dict:
    """Reads a Llama GGUF (linears Q8_0, norms F32, embedding F32 or Q8_0) into the weight dict of luminal_amd.llama.LlamaQ8.
    Q8_0 bytes are uploaded raw and re-arranged on the device; q|k|v are row-concatenated, gate and up rows interleaved."""
    import torch

    from .llama import fuse_rows, interleave_rows
    from .quantized import Q8Weight

    hd = cfg.head_dim
    with open(path, "rb") as f:
        c = Content.read(f)
        missing = [n for n in llama_tensor_names(cfg.layers) if n not in c.tensor_infos]
        if missing:
            raise GgufError(f"missing tensors: {missing[:4]}")

        def f32(name, n):
            info = c.tensor_infos[name]
            if info.dtype != "F32" or info.n_elements != n:
                raise GgufError(f"{name}: expected {n} F32 elements, found {info.n_elements} {info.dtype}")
            return torch.from_numpy(read_tensor(f, c, name)).to(device)

        def raw(name, n, k):
            info = c.tensor_infos[name]
            if info.dtype != "Q8_0" or info.n_elements != n * k:
                raise GgufError(f"{name}: expected {n}x{k} Q8_0, found {info.n_elements} {info.dtype}")
            return read_tensor(f, c, name)

        # the embedding table in whatever dtype the file holds it, as the reference's loader takes each tensor
        # (loader.rs:124-131): f32 rows, or Q8_0 blocks gathered by lhip_q8_0_gather_f32 (QuantizedGather)
        if c.tensor_infos["token_embd.weight"].dtype == "Q8_0":
            embed = Q8Weight.from_raw(raw("token_embd.weight", cfg.vocab, cfg.dim), cfg.vocab, cfg.dim, device)
        else:
            embed = f32("token_embd.weight", cfg.vocab * cfg.dim).reshape(cfg.vocab, cfg.dim)
        w = {"embed": embed,
             "out_norm": f32("output_norm.weight", cfg.dim),
             "lm_head": Q8Weight.from_raw(raw("output.weight", cfg.vocab, cfg.dim), cfg.vocab, cfg.dim, device)}
        for i in range(cfg.layers):
            b = f"blk.{i}."
            w[f"{i}.attn_norm"] = f32(b + "attn_norm.weight", cfg.dim)
            w[f"{i}.ffn_norm"] = f32(b + "ffn_norm.weight", cfg.dim)
            qkv = fuse_rows(raw(b + "attn_q.weight", cfg.dim, cfg.dim), raw(b + "attn_k.weight", cfg.kv_heads * hd, cfg.dim),
                            raw(b + "attn_v.weight", cfg.kv_heads * hd, cfg.dim))
            w[f"{i}.qkv"] = Q8Weight.from_raw(qkv, cfg.qkv_rows, cfg.dim, device)
            w[f"{i}.o"] = Q8Weight.from_raw(raw(b + "attn_output.weight", cfg.dim, cfg.dim), cfg.dim, cfg.dim, device)
            gu = interleave_rows(raw(b + "ffn_gate.weight", cfg.ffn, cfg.dim), raw(b + "ffn_up.weight", cfg.ffn, cfg.dim), cfg.dim)
            w[f"{i}.gate_up"] = Q8Weight.from_raw(gu, 2 * cfg.ffn, cfg.dim, device)
            w[f"{i}.down"] = Q8Weight.from_raw(raw(b + "ffn_down.weight", cfg.dim, cfg.ffn), cfg.dim, cfg.ffn, device)
    return w
