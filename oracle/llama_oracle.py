"""CPU restatement (numpy, float64 accumulation) of the reference's Llama-3
forward pass — TEST INFRASTRUCTURE ONLY, small configurations.

Follows examples/llama/src/model.rs: embedding gather (crates/luminal_nn/src/embedding.rs:40-58);
RMS norm = LayerNorm(mean_norm=false): x * 1/sqrt(mean(x^2)+eps) * w (crates/luminal_nn/src/norm.rs:56-71,
src/hl_ops/unary.rs:93-104); q/k/v projections x . W^T (model.rs:89-102); rotary embedding on adjacent pairs
with inv_freq_j = 1/500000^(2j/head_dim) at positions prev_seq + t (model.rs:52-72); KV cache concat
(:108-110); grouped-query attention, scores / sqrt(head_dim), f16::MIN added above the diagonal, softmax,
times V, merge heads, output projection (:112-139); residuals and SwiGLU MLP down(up(x) * swish(gate(x)))
(:24-32, :173-187); final norm and lm_head (:232-244).

Pinned by: the closed forms above checked piecewise in tests/test_llama_oracle.py (norm and softmax against
direct formulas, rotary embedding against complex multiplication, prefill-vs-incremental consistency of the
KV cache).  The reference holds no stored vectors for this path.
"""
from __future__ import annotations

import numpy as np

F16_MIN = -65504.0


def rms_norm(x, w, eps, dtype=np.float64):
    x = x.astype(dtype)
    return x * (1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + dtype(eps))) * w.astype(dtype)


def rope(x, pos0, theta, dtype=np.float64):
    """x: (seq, heads, head_dim); adjacent pairs rotated by pos * inv_freq."""
    s, h, hd = x.shape
    j = np.arange(hd // 2, dtype=np.float64)
    inv = 1.0 / theta ** (2.0 * j / hd)
    ang = (pos0 + np.arange(s, dtype=np.float64))[:, None] * inv[None, :]
    cs, sn = np.cos(ang)[:, None, :].astype(dtype), np.sin(ang)[:, None, :].astype(dtype)
    x0, x1 = x[..., 0::2], x[..., 1::2]
    out = np.empty_like(x, dtype=dtype)
    out[..., 0::2] = x0 * cs - x1 * sn
    out[..., 1::2] = x0 * sn + x1 * cs
    return out


def swish(t):
    one = t.dtype.type(1.0)
    return t * (one / (one + np.exp(-t)))


def layer_forward(cfg, wl, x, k_prev, v_prev, pos0, dtype=np.float64):
    """One decoder layer (model.rs:81-142 attention, :24-32 MLP, :173-187 residuals).  wl: float32 arrays
    'attn_norm', 'ffn_norm', 'q', 'k', 'v', 'o', 'gate', 'up', 'down'; x: (seq, dim); k_prev / v_prev:
    (kv_heads, prev, hd).  Returns (x, k_all, v_all).  Kept separate so a caller can stream a large model through it
    one layer's weights at a time.  dtype float64 is the truth the tolerances are measured against; float32 runs the
    same operations in the reference's own arithmetic (its CPU path is f32 throughout) and shows how far that
    arithmetic alone lies from the truth."""
    hd, hq, hkv = cfg.head_dim, cfg.q_heads, cfg.kv_heads
    grp = hq // hkv
    s = x.shape[0]
    x = x.astype(dtype)
    k_prev, v_prev = k_prev.astype(dtype), v_prev.astype(dtype)
    n = rms_norm(x, wl["attn_norm"], cfg.eps, dtype)
    q = (n @ wl["q"].astype(dtype).T).reshape(s, hq, hd)
    k = (n @ wl["k"].astype(dtype).T).reshape(s, hkv, hd)
    v = (n @ wl["v"].astype(dtype).T).reshape(s, hkv, hd)
    q, k = rope(q, pos0, cfg.theta, dtype), rope(k, pos0, cfg.theta, dtype)
    k_all = np.concatenate([k_prev, k.transpose(1, 0, 2)], axis=1)   # (hkv, prev+s, hd)
    v_all = np.concatenate([v_prev, v.transpose(1, 0, 2)], axis=1)
    prev = k_all.shape[1] - s
    mask = np.triu(np.ones((s, s), dtype=dtype), 1) * dtype(F16_MIN)
    mask = np.concatenate([np.zeros((s, prev), dtype=dtype), mask], axis=1)        # (s, prev+s)
    out = np.empty((s, hq, hd), dtype=dtype)
    for h in range(hq):
        sc = q[:, h, :] @ k_all[h // grp].T / dtype(np.sqrt(hd)) + mask
        e = np.exp(sc - sc.max(axis=1, keepdims=True))
        p = e * (dtype(1.0) / e.sum(axis=1, keepdims=True))
        out[:, h, :] = p @ v_all[h // grp]
    x = x + out.reshape(s, hq * hd) @ wl["o"].astype(dtype).T
    n = rms_norm(x, wl["ffn_norm"], cfg.eps, dtype)
    gate = swish(n @ wl["gate"].astype(dtype).T)
    up = (n @ wl["up"].astype(dtype).T) * gate
    x = x + up @ wl["down"].astype(dtype).T
    return x, k_all, v_all


LAYER_KEYS = ("attn_norm", "ffn_norm", "q", "k", "v", "o", "gate", "up", "down")


def forward(cfg, w, tokens, k_cache, v_cache, pos0):
    """w: dict of float32 arrays: 'embed', 'out_norm', 'lm_head' (vocab, dim), '{i}.attn_norm', '{i}.ffn_norm',
    '{i}.q' (dim, dim), '{i}.k', '{i}.v' (kv_heads*hd, dim), '{i}.o', '{i}.gate', '{i}.up' (ffn, dim),
    '{i}.down' (dim, ffn).  k_cache/v_cache: lists of (kv_heads, prev, hd) arrays, replaced by the grown ones.
    Returns logits (seq, vocab) in float64."""
    x = w["embed"][np.asarray(tokens, dtype=np.int64)].astype(np.float64)
    for i in range(cfg.layers):
        wl = {key: w[f"{i}.{key}"] for key in LAYER_KEYS}
        x, k_cache[i], v_cache[i] = layer_forward(cfg, wl, x, k_cache[i], v_cache[i], pos0)
    n = rms_norm(x, w["out_norm"], cfg.eps)
    return n @ w["lm_head"].astype(np.float64).T


def argmax_last(v):
    """Index of the maximum; the last one on exact ties (itertools position_max_by, examples/llama/src/main.rs:194-198)."""
    v = np.asarray(v)
    return int(len(v) - 1 - np.argmax(v[::-1]))
