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

forward_prompt_bf16 is the same pass with round-to-nearest-even roundings to bfloat16 placed where a prompt pass on
bf16 matrix-core operands places them (the operands of every linear layer and of the attention products); it has no
counterpart in the reference, whose graph runs in one dtype throughout, and exists so that such a pass can be held
to a tight bar against a restatement with its own roundings and, separately, to the distance of that restatement
from the unrounded truth.
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


def bf16_round(x):
    """Round to bfloat16, ties to even, returned as float64 (finite inputs)."""
    a = np.ascontiguousarray(x, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).astype(np.float64).reshape(a.shape)


def attention_bf16_operands(q, k_all, v_all, pos0, tile=32):
    """Causal grouped-query attention with bf16 operands for both products: q / sqrt(head_dim), K and V rounded once;
    per tile of `tile` keys the weights exp(s - running max) rounded and the running sum taken over the rounded
    weights (so a result is a convex combination of V rows); the quotient rounded.  q: (s, hq, hd) after the rotary
    embedding, k_all / v_all: (hkv, n_keys, hd).  Returns (s, hq * hd) in float64."""
    s, hq, hd = q.shape
    grp = hq // k_all.shape[0]
    n_keys = k_all.shape[1]
    qb = bf16_round(q.astype(np.float32) * (np.float32(1.0) / np.sqrt(np.float32(hd))))
    kb, vb = bf16_round(k_all), bf16_round(v_all)
    visible = np.arange(n_keys)[None, :] <= (pos0 + np.arange(s))[:, None]
    out = np.empty((s, hq, hd))
    for h in range(hq):
        sc = np.where(visible, qb[:, h] @ kb[h // grp].T, -np.inf)
        m = np.full(s, -np.inf)
        l, acc = np.zeros(s), np.zeros((s, hd))
        for k0 in range(0, n_keys, tile):  # key 0 is visible to every row, so every running maximum is finite
            t = sc[:, k0:k0 + tile]
            m_new = np.maximum(m, t.max(axis=1))
            corr = np.exp(m - m_new)
            wgt = bf16_round(np.exp(t - m_new[:, None]))
            l = l * corr + wgt.sum(axis=1)
            acc = acc * corr[:, None] + wgt @ vb[h // grp, k0:k0 + tile]
            m = m_new
        out[:, h] = bf16_round(acc / l[:, None])
    return out.reshape(s, hq * hd)


def layer_forward_bf16(cfg, wl, x, bf16_attention=True):
    """One decoder layer of the prompt pass with bf16 operands (see forward_prompt_bf16), positions 0 .. s - 1 on empty
    caches.  wl as in layer_forward.  Returns (x, k_all, v_all), the caches as the f32 rows a device would hold."""
    hd, hq, hkv = cfg.head_dim, cfg.q_heads, cfg.kv_heads
    s = x.shape[0]
    f = lambda key: wl[key].astype(np.float64)
    n = bf16_round(rms_norm(x, wl["attn_norm"], cfg.eps))
    q = rope((n @ f("q").T).reshape(s, hq, hd), 0, cfg.theta)
    k = rope((n @ f("k").T).reshape(s, hkv, hd), 0, cfg.theta)
    v = (n @ f("v").T).reshape(s, hkv, hd)
    k_all = k.transpose(1, 0, 2).astype(np.float32).astype(np.float64)
    v_all = v.transpose(1, 0, 2).astype(np.float32).astype(np.float64)
    if bf16_attention:
        att = attention_bf16_operands(q.astype(np.float32).astype(np.float64), k_all, v_all, 0)
    else:
        grp = hq // hkv
        att = np.empty((s, hq, hd))
        mask = np.triu(np.ones((s, s)), 1) * F16_MIN
        for h in range(hq):
            sc = q[:, h, :] @ k_all[h // grp].T / np.sqrt(hd) + mask
            e = np.exp(sc - sc.max(axis=1, keepdims=True))
            att[:, h, :] = (e / e.sum(axis=1, keepdims=True)) @ v_all[h // grp]
        att = bf16_round(att.reshape(s, hq * hd))
    x = x + att @ f("o").T
    n = bf16_round(rms_norm(x, wl["ffn_norm"], cfg.eps))
    act = bf16_round((n @ f("up").T) * swish(n @ f("gate").T))
    return x + act @ f("down").T, k_all, v_all


def forward_prompt_bf16(cfg, w, tokens, bf16_attention=True, all_logits=True):
    """The prompt pass (positions 0 .. len(tokens) - 1, empty caches) with the roundings of a pass whose linear layers
    and attention products take bf16 operands and accumulate in f32: the RMS norms in front of q/k/v, gate/up and (for
    all_logits) the lm_head write bf16; q/k/v come back unrounded (they feed the rotary embedding and the f32
    caches); attention as attention_bf16_operands, or, with bf16_attention False, in full precision with only its
    result rounded; up * swish(gate) is rounded where it is formed; the o and down products join the residual
    stream unrounded.  With all_logits False the last norm and the lm_head stay unrounded and only the last position
    is returned, as the generation loop needs it.  Arithmetic between the roundings is float64.  w as in forward().
    Returns (logits, k_cache, v_cache) with the caches as lists of (kv_heads, s, hd) arrays."""
    x = w["embed"][np.asarray(tokens, dtype=np.int64)].astype(np.float64)
    kcs, vcs = [], []
    for i in range(cfg.layers):
        wl = {key: w[f"{i}.{key}"] for key in LAYER_KEYS}
        x, k_all, v_all = layer_forward_bf16(cfg, wl, x, bf16_attention)
        kcs.append(k_all)
        vcs.append(v_all)
    if all_logits:
        n = bf16_round(rms_norm(x, w["out_norm"], cfg.eps))
        return n @ w["lm_head"].astype(np.float64).T, kcs, vcs
    n = rms_norm(x[-1:], w["out_norm"], cfg.eps)
    return (n @ w["lm_head"].astype(np.float64).T)[0], kcs, vcs


def argmax_last(v):
    """Index of the maximum; the last one on exact ties (itertools position_max_by, examples/llama/src/main.rs:194-198)."""
    v = np.asarray(v)
    return int(len(v) - 1 - np.argmax(v[::-1]))
