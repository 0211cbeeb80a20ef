"""ctypes front-end of the CPU oracle (``luminal_cpu_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by
the benchmark's ``cpu_baseline`` leg, never by the shipped package.

Every wrapper takes and returns numpy arrays; see the C file for the
reference file:line each function restates.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libluminal_cpu_oracle.so")


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside this file."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _SO


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _lib.lo_f16_to_f32.restype = C.c_float
        _lib.lo_f16_to_f32.argtypes = [C.c_uint16]
        _lib.lo_f32_to_f16.restype = C.c_uint16
        _lib.lo_f32_to_f16.argtypes = [C.c_float]
        _lib.lo_f32_to_bf16.restype = C.c_uint16
        _lib.lo_f32_to_bf16.argtypes = [C.c_float]
        _lib.lo_bf16_to_f32.restype = C.c_float
        _lib.lo_bf16_to_f32.argtypes = [C.c_uint16]
        _lib.lo_e8m0_to_f32.restype = C.c_float
        _lib.lo_e8m0_to_f32.argtypes = [C.c_uint8]
        _lib.lo_q8_0_nbytes.restype = C.c_size_t
        _lib.lo_q8_0_nbytes.argtypes = [C.c_size_t]
    return _lib


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def f16_to_f32(code: int) -> float:
    return float(lib().lo_f16_to_f32(int(code)))


def f32_to_f16(x: float) -> int:
    return int(lib().lo_f32_to_f16(float(x)))


def q8_0_nbytes(n_elements: int) -> int:
    return int(lib().lo_q8_0_nbytes(n_elements))


def q8_0_pack(qs: np.ndarray, d_codes: np.ndarray) -> np.ndarray:
    """int8 quants (any shape, size % 32 == 0) + uint16 f16 codes -> raw blocks."""
    qs = _c(qs, np.int8).reshape(-1)
    d = _c(d_codes, np.uint16).reshape(-1)
    assert qs.size % 32 == 0 and d.size == qs.size // 32
    out = np.empty(q8_0_nbytes(qs.size), np.uint8)
    lib().lo_q8_0_pack(_p(qs), _p(d), C.c_size_t(qs.size), _p(out))
    return out


def q8_0_dequant(blocks: np.ndarray, n_elements: int) -> np.ndarray:
    blocks = _c(blocks, np.uint8).reshape(-1)
    assert blocks.size == q8_0_nbytes(n_elements)
    out = np.empty(n_elements, np.float32)
    lib().lo_q8_0_dequant(_p(blocks), C.c_size_t(n_elements), _p(out))
    return out


def q8_0_gather(blocks: np.ndarray, idx_f32: np.ndarray, dim: int) -> np.ndarray:
    blocks = _c(blocks, np.uint8).reshape(-1)
    idx = _c(idx_f32, np.float32).reshape(-1)
    out = np.empty((idx.size, dim), np.float32)
    lib().lo_q8_0_gather(_p(blocks), _p(idx), C.c_size_t(idx.size), C.c_size_t(dim), _p(out))
    return out


def matmul_seq_f32(a: np.ndarray, w: np.ndarray) -> np.ndarray:
    """a (M,K) f32, w (N,K) f32 -> (M,N) f32, product-then-in-order-sum in f32."""
    a = _c(a, np.float32)
    w = _c(w, np.float32)
    a2 = a.reshape(-1, a.shape[-1])
    M, K = a2.shape
    N = w.shape[0]
    assert w.shape == (N, K)
    c = np.empty((M, N), np.float32)
    lib().lo_matmul_seq_f32(_p(a2), _p(w), _p(c), C.c_size_t(M), C.c_size_t(N), C.c_size_t(K))
    return c


def matmul_f64(a: np.ndarray, w: np.ndarray) -> np.ndarray:
    a = _c(a, np.float32)
    w = _c(w, np.float32)
    a2 = a.reshape(-1, a.shape[-1])
    M, K = a2.shape
    N = w.shape[0]
    c = np.empty((M, N), np.float64)
    lib().lo_matmul_f64(_p(a2), _p(w), _p(c), C.c_size_t(M), C.c_size_t(N), C.c_size_t(K))
    return c


def matmul_fast_f32(a: np.ndarray, w: np.ndarray, threads: int = 1, out: np.ndarray | None = None) -> np.ndarray:
    a = _c(a, np.float32)
    w = _c(w, np.float32)
    a2 = a.reshape(-1, a.shape[-1])
    M, K = a2.shape
    N = w.shape[0]
    c = out if out is not None else np.empty((M, N), np.float32)
    lib().lo_matmul_fast_f32(_p(a2), _p(w), _p(c), C.c_size_t(M), C.c_size_t(N), C.c_size_t(K), C.c_int(threads))
    return c


def mxfp4_dequant(blocks: np.ndarray, n_elements: int) -> np.ndarray:
    blocks = _c(blocks, np.uint8).reshape(-1)
    assert blocks.size == n_elements // 32 * 17
    out = np.empty(n_elements, np.float32)
    lib().lo_mxfp4_dequant(_p(blocks), C.c_size_t(n_elements), _p(out))
    return out


def moe_route(logits: np.ndarray, topk: int):
    logits = _c(logits, np.float32)
    T, E = logits.shape
    sel = np.empty((T, topk), np.int32)
    wts = np.empty((T, topk), np.float32)
    lib().lo_moe_route(_p(logits), C.c_size_t(T), C.c_size_t(E), C.c_size_t(topk), _p(sel), _p(wts))
    return sel, wts


def moe_forward(x, w_gu, w_down, sel, wts, act_bf16: bool) -> np.ndarray:
    x = _c(x, np.float32)
    w_gu = _c(w_gu, np.float32)
    w_down = _c(w_down, np.float32)
    sel = _c(sel, np.int32)
    wts = _c(wts, np.float32)
    T, H = x.shape
    E, I2, H2 = w_gu.shape
    I = I2 // 2
    assert H2 == H and w_down.shape == (E, H, I)
    topk = sel.shape[1]
    out = np.empty((T, H), np.float32)
    lib().lo_moe_forward(_p(x), _p(w_gu), _p(w_down), _p(sel), _p(wts), C.c_size_t(T), C.c_size_t(H),
                         C.c_size_t(I), C.c_size_t(topk), C.c_int(int(act_bf16)), _p(out))
    return out


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even f32 -> bf16 codes (numpy, vectorised; checked against the C routine in tests)."""
    u = _c(x, np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (_c(b, np.uint16).astype(np.uint32) << 16).view(np.float32)
