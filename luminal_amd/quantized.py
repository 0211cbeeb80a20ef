"""Host-side mirror of the reference's quantized operators over the C ABI.

Names and argument meaning follow crates/luminal_cuda/src/quantized.rs:
``QuantizedMatmul.process`` takes the activations first and the weight second
and returns a freshly allocated output; ``QuantizedGather`` carries
``embed_dim``.  torch is used for device memory and the current stream only:
all arithmetic happens in libluminal_hip.so, and there is no fallback.
"""
from __future__ import annotations

import numpy as np
import torch

from . import capi


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: torch.Tensor) -> int:
    return t.data_ptr()


class Q8Weight:
    """A (N, K) Q8_0 weight resident on the device in planar form
    (the role of ``CudaData<u8>`` in examples/llama/src/loader.rs:156-158)."""

    def __init__(self, planar: torch.Tensor, n: int, k: int):
        self.planar, self.n, self.k = planar, n, k

    @staticmethod
    def planar_nbytes(n: int, k: int) -> int:
        nb = capi.load_library().lhip_q8_0_planar_nbytes(n, k)
        if nb == 0:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "Q8Weight", f"invalid Q8_0 shape ({n}, {k})")
        return nb

    @classmethod
    def from_raw(cls, raw, n: int, k: int, device="cuda:0") -> "Q8Weight":
        """raw: GGUF Q8_0 block bytes (numpy uint8, or a uint8 torch tensor on host or device)."""
        lib = capi.load_library()
        if isinstance(raw, np.ndarray):
            raw = torch.from_numpy(np.ascontiguousarray(raw, dtype=np.uint8))
        raw = raw.reshape(-1)
        expect = lib.lhip_q8_0_raw_nbytes(n, k)
        if expect == 0 or raw.numel() != expect:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "Q8Weight.from_raw",
                                 f"expected {expect} bytes for ({n}, {k}), got {raw.numel()}")
        raw_dev = raw.to(device)
        planar = torch.empty(cls.planar_nbytes(n, k), dtype=torch.uint8, device=device)
        with torch.cuda.device(planar.device):
            capi.check(lib.lhip_q8_0_repack(_ptr(raw_dev), _ptr(planar), n, k, _stream()), "lhip_q8_0_repack")
            torch.cuda.current_stream().synchronize()  # raw_dev is released on return
        return cls(planar, n, k)

    @classmethod
    def interleave_rows(cls, a: "Q8Weight", b: "Q8Weight") -> "Q8Weight":
        """(2n, k) weight whose rows alternate between a's and b's: the (gate, up) order the SwiGLU epilogues read
        (gate and up are separate tensors in examples/llama/src/model.rs:17-32)."""
        if (a.n, a.k) != (b.n, b.k):
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "Q8Weight.interleave_rows",
                                 f"shapes differ: ({a.n}, {a.k}) and ({b.n}, {b.k})")
        lib = capi.load_library()
        out = torch.empty(cls.planar_nbytes(2 * a.n, a.k), dtype=torch.uint8, device=a.planar.device)
        with torch.cuda.device(out.device):
            capi.check(lib.lhip_q8_0_interleave_rows(_ptr(a.planar), _ptr(b.planar), _ptr(out), a.n, a.k, _stream()),
                       "lhip_q8_0_interleave_rows")
        return cls(out, 2 * a.n, a.k)

    def to_raw(self) -> torch.Tensor:
        lib = capi.load_library()
        raw = torch.empty(lib.lhip_q8_0_raw_nbytes(self.n, self.k), dtype=torch.uint8, device=self.planar.device)
        with torch.cuda.device(raw.device):
            capi.check(lib.lhip_q8_0_unpack(_ptr(self.planar), _ptr(raw), self.n, self.k, _stream()),
                       "lhip_q8_0_unpack")
        return raw

    def dequantize(self) -> torch.Tensor:
        lib = capi.load_library()
        out = torch.empty((self.n, self.k), dtype=torch.float32, device=self.planar.device)
        with torch.cuda.device(out.device):
            capi.check(lib.lhip_q8_0_dequant_f32(_ptr(self.planar), _ptr(out), self.n, self.k, _stream()),
                       "lhip_q8_0_dequant_f32")
        return out


class QuantizedMatmul:
    """(.., M, K) x Q8_0 (N, K) -> (.., M, N) in the activation type T = f32 or f16, f32 accumulation either way
    (QuantizedMatmul<T>::process, crates/luminal_cuda/src/quantized.rs:116-168).  The library runs one matvec per
    group of activation rows, as the reference does per row, or from two to six rows on, by matrix size (where the shape allows it), the
    matrix-core form with exact products (x as three bf16 limbs, an f16 x as two), which streams the weights once per 64 rows.  A launch shape
    can be chosen for f32 only and always means the matvec form."""

    def __init__(self, rows_per_wave: int | None = None, k_unroll: int | None = None, blocks_per_cu: int = 0,
                 waves_per_block: int = 4):
        self.cfg = (rows_per_wave, k_unroll, blocks_per_cu, waves_per_block) if rows_per_wave else None

    def process(self, x: torch.Tensor, w: Q8Weight) -> torch.Tensor:
        lib = capi.load_library()
        if x.dtype not in (torch.float32, torch.float16) or not x.is_cuda:
            raise TypeError("QuantizedMatmul expects f32 or f16 activations on the GPU")
        if x.shape[-1] != w.k:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "QuantizedMatmul",
                                 f"activation K {x.shape[-1]} != weight K {w.k}")
        x = x.contiguous()
        m = x.numel() // w.k
        out = torch.empty(x.shape[:-1] + (w.n,), dtype=x.dtype, device=x.device)
        with torch.cuda.device(x.device):
            if x.dtype == torch.float16:
                if self.cfg:
                    raise TypeError("QuantizedMatmul: a launch shape can be chosen for f32 activations only")
                st = lib.lhip_q8_0_matmul_f16(_ptr(w.planar), _ptr(x), _ptr(out), m, w.n, w.k, _stream())
                capi.check(st, "lhip_q8_0_matmul_f16")
                return out
            if self.cfg:
                st = lib.lhip_q8_0_matmul_f32_cfg(_ptr(w.planar), _ptr(x), _ptr(out), m, w.n, w.k, self.cfg[0],
                                                  self.cfg[1], self.cfg[2], self.cfg[3], _stream())
            else:
                st = lib.lhip_q8_0_matmul_f32(_ptr(w.planar), _ptr(x), _ptr(out), m, w.n, w.k, _stream())
        capi.check(st, "lhip_q8_0_matmul_f32")
        return out


class QuantizedMatmulBf16:
    """(.., M, K) bf16 x Q8_0 (N, K) -> (.., M, N) bf16 with f32 accumulation on
    the matrix cores (the prefill path; dispatch by dtype, where the Metal
    backend dispatches matvec vs matmul by M,
    crates/luminal_metal/src/quantized.rs:339-376)."""

    def __init__(self, tile: int | None = None):
        self.tile = tile

    def process(self, x: torch.Tensor, w: Q8Weight) -> torch.Tensor:
        lib = capi.load_library()
        if x.dtype != torch.bfloat16 or not x.is_cuda:
            raise TypeError("QuantizedMatmulBf16 expects bf16 activations on the GPU")
        if x.shape[-1] != w.k:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "QuantizedMatmulBf16",
                                 f"activation K {x.shape[-1]} != weight K {w.k}")
        x = x.contiguous()
        m = x.numel() // w.k
        out = torch.empty(x.shape[:-1] + (w.n,), dtype=torch.bfloat16, device=x.device)
        with torch.cuda.device(x.device):
            if self.tile is None:
                st = lib.lhip_q8_0_matmul_bf16(_ptr(w.planar), _ptr(x), _ptr(out), m, w.n, w.k, _stream())
            else:
                st = lib.lhip_q8_0_matmul_bf16_cfg(_ptr(w.planar), _ptr(x), _ptr(out), m, w.n, w.k, self.tile,
                                                   _stream())
        capi.check(st, "lhip_q8_0_matmul_bf16")
        return out


class QuantizedGather:
    """Row gather from a Q8_0 table into T = f32 (default) or f16; indices are f32 as in the reference
    (QuantizedGather<T>::process, crates/luminal_cuda/src/quantized.rs:202-233)."""

    def __init__(self, embed_dim: int, dtype: torch.dtype = torch.float32):
        if dtype not in (torch.float32, torch.float16):
            raise TypeError("QuantizedGather gathers into f32 or f16")
        self.embed_dim = embed_dim
        self.dtype = dtype

    def process(self, indexes: torch.Tensor, w: Q8Weight) -> torch.Tensor:
        lib = capi.load_library()
        if w.k != self.embed_dim:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "QuantizedGather",
                                 f"embed_dim {self.embed_dim} != weight K {w.k}")
        idx = indexes.to(device=w.planar.device, dtype=torch.float32).contiguous().reshape(-1)
        out = torch.empty((idx.numel(), w.k), dtype=self.dtype, device=idx.device)
        gather = lib.lhip_q8_0_gather_f32 if self.dtype == torch.float32 else lib.lhip_q8_0_gather_f16
        with torch.cuda.device(idx.device):
            st = gather(_ptr(w.planar), _ptr(idx), _ptr(out), idx.numel(), w.n, w.k, _stream())
        capi.check(st, "lhip_q8_0_gather")
        return out


class FusedMatvec:
    """Batch-1 decode: up to four Q8_0 weights that read the same (K,) f32 activation in one launch, with an optional
    RMS-norm prologue (norm_weight, eps) and epilogue (EPI_ADD: y = residual + W x; EPI_SWIGLU: rows are (gate, up)
    pairs and y[j] = up_j * swish(gate_j)).  A plan object: the operand addresses are fixed at construction, `run`
    only launches (lhip_q8_0_matvec_fused_f32)."""

    EPI_NONE, EPI_ADD, EPI_SWIGLU = 0, 1, 2

    def __init__(self, weights, outs, norm_weight: torch.Tensor | None = None, eps: float = 0.0,
                 residual: torch.Tensor | None = None, epilogue: int = 0, cfg: tuple | None = None):
        import ctypes as C

        if len(weights) != len(outs) or not 1 <= len(weights) <= 4:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "FusedMatvec", "1..4 weights, one output each")
        k = weights[0].k
        for w, y in zip(weights, outs):
            want = w.n // 2 if epilogue == self.EPI_SWIGLU else w.n
            if w.k != k or y.dtype != torch.float32 or y.numel() != want or not y.is_contiguous():
                raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "FusedMatvec", "weights share K; outputs f32 (n,)")
        if norm_weight is not None and (norm_weight.dtype != torch.float32 or norm_weight.numel() != k):
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "FusedMatvec", "norm weight is f32 (K,)")
        if residual is not None and (residual.dtype != torch.float32 or residual.numel() != weights[0].n):
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "FusedMatvec", "residual is f32 (n,)")
        self.k, self.count = k, len(weights)
        self._keep = (list(weights), list(outs), norm_weight, residual)
        self._w = (C.c_void_p * self.count)(*[w.planar.data_ptr() for w in weights])
        self._y = (C.c_void_p * self.count)(*[y.data_ptr() for y in outs])
        self._n = (C.c_int64 * self.count)(*[w.n for w in weights])
        self._norm = norm_weight.data_ptr() if norm_weight is not None else None
        self._res = residual.data_ptr() if residual is not None else None
        self.eps, self.epilogue, self.cfg = float(eps), int(epilogue), cfg
        self.lib = capi.load_library()

    def run(self, x: torch.Tensor) -> None:
        if x.dtype != torch.float32 or not x.is_cuda or x.numel() != self.k:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "FusedMatvec", f"activation must be f32 ({self.k},)")
        if self.cfg:
            st = self.lib.lhip_q8_0_matvec_fused_f32_cfg(self._w, self._y, self._n, self.count, _ptr(x), self.k,
                                                         self._norm, self.eps, self._res, self.epilogue, *self.cfg,
                                                         _stream())
        else:
            st = self.lib.lhip_q8_0_matvec_fused_f32(self._w, self._y, self._n, self.count, _ptr(x), self.k,
                                                     self._norm, self.eps, self._res, self.epilogue, _stream())
        capi.check(st, "lhip_q8_0_matvec_fused_f32")


class DecodeProgram:
    """A batch-1 decode step as one persistent launch (lhip_decode_program_*): a list of fused matvecs and attention
    operations that a resident grid walks in order.  Operand addresses are fixed at construction; `run` queues the
    launch on the current stream, `timed_out` asks (after a device sync) whether a grid-wide wait ever gave up."""

    def __init__(self, q_heads: int = 0, kv_heads: int = 0, head_dim: int = 0, max_seq: int = 0, theta: float = 0.0,
                 pos: torch.Tensor | None = None):
        self._geom = (q_heads, kv_heads, head_dim, max_seq, float(theta))
        self._pos = pos
        self._ops, self._keep, self._handle = [], [], None
        self.lib = capi.load_library()

    def matvec(self, w: Q8Weight, x: torch.Tensor, y: torch.Tensor, norm_weight: torch.Tensor | None = None,
               eps: float = 0.0, residual: torch.Tensor | None = None, epilogue: int = 0):
        want = w.n // 2 if epilogue == FusedMatvec.EPI_SWIGLU else w.n
        for t, size, what in ((x, w.k, "activation"), (y, want, "output")):
            if t.dtype != torch.float32 or not t.is_cuda or t.numel() != size or not t.is_contiguous():
                raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "DecodeProgram", f"{what} must be f32 ({size},)")
        if norm_weight is not None and (norm_weight.dtype != torch.float32 or norm_weight.numel() != w.k):
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "DecodeProgram", "norm weight is f32 (K,)")
        if residual is not None and (residual.dtype != torch.float32 or residual.numel() != w.n):
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "DecodeProgram", "residual is f32 (n,)")
        self._keep += [w, x, y, norm_weight, residual]
        self._ops.append(capi.DecodeOp(capi.LHIP_DECODE_MATVEC, int(epilogue), w.planar.data_ptr(), w.n, w.k,
                                       x.data_ptr(), y.data_ptr(),
                                       norm_weight.data_ptr() if norm_weight is not None else None, float(eps),
                                       residual.data_ptr() if residual is not None else None, None, None))
        return self

    def attention(self, qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor):
        q_heads, kv_heads, head_dim, max_seq, _ = self._geom
        sizes = ((qkv, (q_heads + 2 * kv_heads) * head_dim), (out, q_heads * head_dim),
                 (k_cache, kv_heads * max_seq * head_dim), (v_cache, kv_heads * max_seq * head_dim))
        for t, size in sizes:
            if t.dtype != torch.float32 or not t.is_cuda or t.numel() != size or not t.is_contiguous():
                raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "DecodeProgram", "attention operand shapes")
        self._keep += [qkv, k_cache, v_cache, out]
        self._ops.append(capi.DecodeOp(capi.LHIP_DECODE_ATTENTION, 0, None, 0, 0, qkv.data_ptr(), out.data_ptr(), None,
                                       0.0, None, k_cache.data_ptr(), v_cache.data_ptr()))
        return self

    def build(self):
        import ctypes as C

        if self._handle is not None:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "DecodeProgram", "already built")
        if self._pos is None or self._pos.dtype != torch.int32 or not self._pos.is_cuda:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "DecodeProgram", "pos must be an int32 device tensor")
        arr = (capi.DecodeOp * len(self._ops))(*self._ops)
        handle = C.c_void_p()
        capi.check(self.lib.lhip_decode_program_create(arr, len(self._ops), *self._geom, self._pos.data_ptr(),
                                                       C.byref(handle)), "lhip_decode_program_create")
        self._handle = handle
        return self

    def run(self):
        capi.check(self.lib.lhip_decode_program_run(self._handle, _stream()), "lhip_decode_program_run")

    def trace(self, on: bool = True):
        """Switches the per-phase clock on (returns the int64 device tensor later runs fill: enter / done ticks of
        workgroup 0 per phase, 100 MHz) or off."""
        import ctypes as C

        n = C.c_int32()
        if not on:
            capi.check(self.lib.lhip_decode_program_trace(self._handle, None, C.byref(n)), "lhip_decode_program_trace")
            self._ticks = None
            return None
        capi.check(self.lib.lhip_decode_program_trace(self._handle, None, C.byref(n)), "lhip_decode_program_trace")
        self._ticks = torch.zeros(2 * n.value, dtype=torch.int64, device=self._pos.device)
        capi.check(self.lib.lhip_decode_program_trace(self._handle, self._ticks.data_ptr(), None), "lhip_decode_program_trace")
        return self._ticks

    def timed_out(self) -> bool:
        import ctypes as C

        flag = C.c_int32()
        capi.check(self.lib.lhip_decode_program_status(self._handle, C.byref(flag)), "lhip_decode_program_status")
        return bool(flag.value)

    def __del__(self):
        if getattr(self, "_handle", None) is not None:
            self.lib.lhip_decode_program_destroy(self._handle)
            self._handle = None
