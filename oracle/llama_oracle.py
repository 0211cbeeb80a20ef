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


def rms_norm(x, w, eps):
    x = x.astype(np.float64)
    return x * (1.0 / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)) * w.astype(np.float64)


def rope(x, pos0, theta):
    """x: (seq, heads, head_dim); adjacent pairs rotated by pos * inv_freq."""
    s, h, hd = x.shape
    j = np.arange(hd // 2, dtype=np.float64)
    inv = 1.0 / theta ** (2.0 * j / hd)
    ang = (pos0 + np.arange(s, dtype=np.float64))[:, None] * inv[None, :]
    cs, sn = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    x0, x1 = x[..., 0::2], x[..., 1::2]
    out = np.empty_like(x, dtype=np.float64)
    out[..., 0::2] = x0 * cs - x1 * sn
    out[..., 1::2] = x0 * sn + x1 * cs
    return out


def swish(t):
    return t * (1.0 / (1.0 + np.exp(-t)))


def forward(cfg, w, tokens, k_cache, v_cache, pos0):
    """w: dict of float32 arrays: 'embed', 'out_norm', 'lm_head' (vocab, dim), '{i}.attn_norm', '{i}.ffn_norm',
    '{i}.q' (dim, dim), '{i}.k', '{i}.v' (kv_heads*hd, dim), '{i}.o', '{i}.gate', '{i}.up' (ffn, dim),
    '{i}.down' (dim, ffn).  k_cache/v_cache: lists of (kv_heads, prev, hd) arrays, replaced by the grown ones.
    Returns logits (seq, vocab) in float64."""
    hd, hq, hkv = cfg.head_dim, cfg.q_heads, cfg.kv_heads
    grp = hq // hkv
    s = len(tokens)
    x = w["embed"][np.asarray(tokens, dtype=np.int64)].astype(np.float64)
    for i in range(cfg.layers):
        n = rms_norm(x, w[f"{i}.attn_norm"], cfg.eps)
        q = (n @ w[f"{i}.q"].astype(np.float64).T).reshape(s, hq, hd)
        k = (n @ w[f"{i}.k"].astype(np.float64).T).reshape(s, hkv, hd)
        v = (n @ w[f"{i}.v"].astype(np.float64).T).reshape(s, hkv, hd)
        q, k = rope(q, pos0, cfg.theta), rope(k, pos0, cfg.theta)
        k_all = np.concatenate([k_cache[i], k.transpose(1, 0, 2)], axis=1)   # (hkv, prev+s, hd)
        v_all = np.concatenate([v_cache[i], v.transpose(1, 0, 2)], axis=1)
        k_cache[i], v_cache[i] = k_all, v_all
        prev = k_all.shape[1] - s
        mask = np.triu(np.ones((s, s)), 1) * F16_MIN
        mask = np.concatenate([np.zeros((s, prev)), mask], axis=1)            # (s, prev+s)
        out = np.empty((s, hq, hd))
        for h in range(hq):
            sc = q[:, h, :] @ k_all[h // grp].T / np.sqrt(hd) + mask
            e = np.exp(sc - sc.max(axis=1, keepdims=True))
            p = e * (1.0 / e.sum(axis=1, keepdims=True))
            out[:, h, :] = p @ v_all[h // grp]
        x = x + out.reshape(s, hq * hd) @ w[f"{i}.o"].astype(np.float64).T
        n = rms_norm(x, w[f"{i}.ffn_norm"], cfg.eps)
        gate = swish(n @ w[f"{i}.gate"].astype(np.float64).T)
        up = (n @ w[f"{i}.up"].astype(np.float64).T) * gate
        x = x + up @ w[f"{i}.down"].astype(np.float64).T
    n = rms_norm(x, w["out_norm"], cfg.eps)
    return n @ w["lm_head"].astype(np.float64).T


def argmax_last(v):
    """Index of the maximum; the last one on exact ties (itertools position_max_by, examples/llama/src/main.rs:194-198)."""
    v = np.asarray(v)
    return int(len(v) - 1 - np.argmax(v[::-1]))
