"""Pins the numpy Llama oracle piece by piece against closed forms (no GPU)."""
import numpy as np

from luminal_amd.llama import LlamaConfig
from oracle import llama_oracle as lo


def small_cfg():
    return LlamaConfig(vocab=97, dim=64, layers=2, q_heads=4, kv_heads=2, ffn=96)


def random_f32_weights(cfg, seed):
    rng = np.random.default_rng(seed)
    hd = cfg.head_dim

    def lin(n, k):
        return (rng.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)

    w = {"embed": rng.standard_normal((cfg.vocab, cfg.dim)).astype(np.float32),
         "out_norm": (1 + 0.1 * rng.standard_normal(cfg.dim)).astype(np.float32), "lm_head": lin(cfg.vocab, cfg.dim)}
    for i in range(cfg.layers):
        w[f"{i}.attn_norm"] = (1 + 0.1 * rng.standard_normal(cfg.dim)).astype(np.float32)
        w[f"{i}.ffn_norm"] = (1 + 0.1 * rng.standard_normal(cfg.dim)).astype(np.float32)
        w[f"{i}.q"], w[f"{i}.o"] = lin(cfg.dim, cfg.dim), lin(cfg.dim, cfg.dim)
        w[f"{i}.k"], w[f"{i}.v"] = lin(cfg.kv_heads * hd, cfg.dim), lin(cfg.kv_heads * hd, cfg.dim)
        w[f"{i}.gate"], w[f"{i}.up"], w[f"{i}.down"] = lin(cfg.ffn, cfg.dim), lin(cfg.ffn, cfg.dim), lin(cfg.dim, cfg.ffn)
    return w


def empty_cache(cfg):
    return [np.zeros((cfg.kv_heads, 0, cfg.head_dim)) for _ in range(cfg.layers)]


def test_rms_norm_formula():
    x = np.array([[3.0, 4.0, 0.0, 0.0]], np.float32)
    w = np.array([1.0, 2.0, 3.0, 4.0], np.float32)
    # mean(x^2) = 6.25 -> 1/sqrt(6.25 + eps)
    assert np.allclose(lo.rms_norm(x, w, 0.0), [[1.2, 3.2, 0.0, 0.0]])
    assert np.allclose(lo.rms_norm(x, w, 2.75), [[1.0, 8.0 / 3.0, 0.0, 0.0]])


def test_rope_is_complex_rotation_of_adjacent_pairs():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 3, 8))
    y = lo.rope(x, pos0=7, theta=500000.0)
    z = x[..., 0::2] + 1j * x[..., 1::2]
    inv = 1.0 / 500000.0 ** (2.0 * np.arange(4) / 8)
    rot = np.exp(1j * (7 + np.arange(5))[:, None, None] * inv[None, None, :])
    want = z * rot
    assert np.allclose(y[..., 0::2], want.real) and np.allclose(y[..., 1::2], want.imag)
    assert np.allclose(lo.rope(x, 0, 500000.0)[0], x[0])  # position 0 is the identity


def test_prefill_equals_incremental_decode():
    cfg = small_cfg()
    w = random_f32_weights(cfg, 1)
    toks = [5, 17, 3, 96, 0, 42, 8]
    kc, vc = empty_cache(cfg), empty_cache(cfg)
    full = lo.forward(cfg, w, toks, kc, vc, 0)
    kc2, vc2 = empty_cache(cfg), empty_cache(cfg)
    rows = [lo.forward(cfg, w, [t], kc2, vc2, p)[0] for p, t in enumerate(toks)]
    assert np.allclose(full, np.stack(rows), rtol=1e-9, atol=1e-9)
    assert all(np.allclose(a, b) for a, b in zip(kc, kc2))


def test_causality_and_softmax_rows():
    cfg = small_cfg()
    w = random_f32_weights(cfg, 2)
    a = lo.forward(cfg, w, [1, 2, 3, 4], empty_cache(cfg), empty_cache(cfg), 0)
    b = lo.forward(cfg, w, [1, 2, 3, 90], empty_cache(cfg), empty_cache(cfg), 0)
    assert np.allclose(a[:3], b[:3]) and not np.allclose(a[3], b[3])  # a later token never changes earlier logits


def test_argmax_last_tie_rule():
    assert lo.argmax_last([1.0, 5.0, 5.0, 2.0]) == 2
    assert lo.argmax_last([7.0]) == 0
