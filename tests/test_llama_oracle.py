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


def test_bf16_round_is_round_to_nearest_even():
    """Against torch.bfloat16 on random values over 40 binades, the ties on both sides of an even and an odd
    neighbour, a subnormal and a large value."""
    torch = __import__("pytest").importorskip("torch")
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(50000) * 10.0 ** rng.integers(-20, 20, 50000)).astype(np.float32)
    ties = np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, -1 - 2.0 ** -8, -1 - 3 * 2.0 ** -8, 2.0 ** -130, 3.0e38, 0.0], np.float32)
    for v in (x, ties):
        assert np.array_equal(lo.bf16_round(v), torch.from_numpy(v).bfloat16().double().numpy())
    assert lo.bf16_round(np.float32(1 + 2.0 ** -8)) == 1.0 and lo.bf16_round(np.float32(1 + 3 * 2.0 ** -8)) == 1 + 2.0 ** -6


def test_bf16_prompt_pass_stays_within_the_rounding_budget_of_the_exact_pass():
    """forward_prompt_bf16 is forward() plus roundings of relative size 2^-9: its logits lie close to the exact ones
    (each rounded operand vector moves a product by about 2^-9 / sqrt(3) of its rms, and a two-layer pass rounds a
    dozen of them), its caches are the exact pass's caches computed from rounded norms, and without any rounding left
    to do (weights and inputs that bf16 holds exactly cannot be arranged for a whole pass) the two attention forms
    agree with each other within the bound 2e-2 * sum_j p_j |v_j| that three roundings of V, the weights and the
    result allow."""
    cfg = small_cfg()
    w = random_f32_weights(cfg, 7)
    tokens = [5, 17, 3, 96, 42, 8, 61]
    kc, vc = empty_cache(cfg), empty_cache(cfg)
    exact = lo.forward(cfg, w, tokens, kc, vc, 0)
    rms = np.sqrt(np.mean(exact * exact))
    for bf16_attention in (True, False):
        got, kcb, vcb = lo.forward_prompt_bf16(cfg, w, tokens, bf16_attention=bf16_attention)
        assert got.shape == exact.shape
        err = np.max(np.abs(got - exact)) / rms
        assert 1e-5 < err < 3e-2, err  # rounded somewhere, and nowhere grossly
        for i in range(cfg.layers):
            assert kcb[i].shape == kc[i].shape and np.max(np.abs(kcb[i] - kc[i])) < 3e-2 * np.sqrt(np.mean(kc[i] ** 2))
        last, _, _ = lo.forward_prompt_bf16(cfg, w, tokens, bf16_attention=bf16_attention, all_logits=False)
        assert last.shape == (cfg.vocab,) and np.max(np.abs(last - exact[-1])) / rms < 3e-2
    # the attention with bf16 operands against the exact one on the same q, K, V
    rng = np.random.default_rng(3)
    s, hq, hkv, hd = 40, 4, 2, 64
    q = rng.standard_normal((s, hq, hd)); k = rng.standard_normal((hkv, s, hd)); v = rng.standard_normal((hkv, s, hd))
    got = lo.attention_bf16_operands(q, k, v, 0).reshape(s, hq, hd)
    for h in range(hq):
        sc = q[:, h] @ k[h // 2].T / np.sqrt(hd) + np.triu(np.ones((s, s)), 1) * lo.F16_MIN
        p = np.exp(sc - sc.max(axis=1, keepdims=True)); p /= p.sum(axis=1, keepdims=True)
        assert np.all(np.abs(got[:, h] - p @ v[h // 2]) <= 2e-2 * (p @ np.abs(v[h // 2])) + 1e-12)
