"""Seeded synthetic inputs of the benchmark configurations (numpy only).

Q8_0 weights: quants uniform in [-127, 127], one f16 scale per 32-value block
drawn from |N(0, 0.02)| / 127; activations N(0, 1).
"""
from __future__ import annotations

import numpy as np


def q8_0_random(n: int, k: int, seed: int, scale_sigma: float = 0.02):
    """Returns (qs int8 (n,k), d f16 (n,k//32))."""
    assert k % 32 == 0
    rng = np.random.default_rng(seed)
    qs = rng.integers(-127, 128, size=(n, k), dtype=np.int8)
    d = (np.abs(rng.standard_normal((n, k // 32), dtype=np.float32)) * (scale_sigma / 127.0)).astype(np.float16)
    return qs, d


def q8_0_raw_blocks(qs: np.ndarray, d: np.ndarray) -> np.ndarray:
    """Pack quants + f16 scales into raw GGUF Q8_0 blocks (34 B each, little-endian scale first)."""
    n_blocks = qs.size // 32
    raw = np.empty((n_blocks, 34), np.uint8)
    raw[:, :2] = np.ascontiguousarray(d, dtype="<f2").reshape(-1).view(np.uint8).reshape(n_blocks, 2)
    raw[:, 2:] = np.ascontiguousarray(qs).reshape(n_blocks, 32).view(np.uint8)
    return raw.reshape(-1)


def activations(m: int, k: int, seed: int) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return rng.standard_normal((m, k), dtype=np.float32)


# Llama-3-8B projection shapes (N = out features, K = in features).
LLAMA3_8B_PROJ = {
    "q": (4096, 4096),
    "k": (1024, 4096),
    "v": (1024, 4096),
    "o": (4096, 4096),
    "gate": (14336, 4096),
    "up": (14336, 4096),
    "down": (4096, 14336),
    "lm_head": (128256, 4096),
}
LLAMA3_8B_LAYERS = 32


def q8_0_gemv_bytes(n: int, k: int) -> int:
    """Algorithmic bytes of one batch-1 Q8_0 matvec: weights once, x and y in f32."""
    return n * k * 34 // 32 + 4 * k + 4 * n


def mxfp4_random(n: int, k: int, seed: int, exp_lo: int = -8, exp_hi: int = 0):
    """Random MXFP4 weight: e2m1 codes uniform over the 16 values, one e8m0 scale
    per 32-value block with exponent uniform in [exp_lo, exp_hi].
    Returns (codes uint8 (n,k) in 0..15, scales uint8 (n,k//32))."""
    assert k % 32 == 0
    rng = np.random.default_rng(seed)
    codes = rng.integers(0, 16, size=(n, k), dtype=np.uint8)
    scales = (127 + rng.integers(exp_lo, exp_hi + 1, size=(n, k // 32))).astype(np.uint8)
    return codes, scales


def mxfp4_raw_blocks(codes: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """Pack e2m1 codes + e8m0 scales into raw 17-byte blocks (even element in the low nibble)."""
    n_blocks = codes.size // 32
    c = np.ascontiguousarray(codes, dtype=np.uint8).reshape(n_blocks, 16, 2)
    raw = np.empty((n_blocks, 17), np.uint8)
    raw[:, :16] = c[:, :, 0] | (c[:, :, 1] << 4)
    raw[:, 16] = np.ascontiguousarray(scales, dtype=np.uint8).reshape(-1)
    return raw.reshape(-1)


# gpt-oss-style expert layer of the benchmark configuration
MOE_HIDDEN, MOE_INTER, MOE_EXPERTS, MOE_TOPK = 2880, 2880, 32, 4
