"""Pins three oracle branches against torch's own implementations (CPU only):
the bf16 round-to-nearest-even conversion, the bf16-activation branch of the MoE
forward, and the whole Llama forward pass (grouped-query attention, 1/sqrt(head_dim),
swish on the gate, residual placement) against a torch forward built from
scaled_dot_product_attention, repeat_interleave and silu.

The expressions the Llama forward must agree with: examples/llama/src/model.rs:24-32 (SwiGLU),
:52-72 (rotary embedding of adjacent pairs), :81-142 (attention), :163-187 (residuals);
the tolerance convention is that of src/tests/mod.rs:67-87.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")
import torch.nn.functional as F  # noqa: E402

from luminal_amd.llama import LlamaConfig  # noqa: E402
from oracle import llama_oracle as lo  # noqa: E402


def torch_bf16_bits(x: np.ndarray) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def test_f32_to_bf16_is_torch_round_to_nearest_even(oracle):
    rng = np.random.default_rng(11)
    # every bf16 value of a few binades and the exact midpoint to its upper neighbour (ties), both signs
    codes = np.concatenate([np.arange(0x3f00, 0x4100), np.arange(0x0001, 0x0100), np.arange(0x7e00, 0x7f7f)]).astype(np.uint32)
    lo_v = (codes << 16).view(np.float32).astype(np.float64)
    hi_v = ((codes + 1) << 16).view(np.float32).astype(np.float64)
    mid = ((lo_v + hi_v) / 2).astype(np.float32)  # exact: one more significant bit than bf16
    assert np.array_equal(mid.astype(np.float64), (lo_v + hi_v) / 2)
    just_below = np.nextafter(mid, np.float32(0))
    just_above = np.nextafter(mid, np.float32(np.inf))
    xs = np.concatenate([
        mid, -mid, just_below, just_above,
        rng.standard_normal(50000).astype(np.float32) * np.float32(10.0) ** rng.integers(-30, 30, 50000).astype(np.float32),
        np.array([0.0, -0.0, 1.0, -1.0, 3.3895314e38, 3.4028235e38, np.inf, -np.inf, 1e-45, 9.1835e-41, 1.17549435e-38],
                 np.float32),
    ])
    want = torch_bf16_bits(xs)
    assert np.array_equal(oracle.f32_to_bf16_bits(xs), want)
    fn = oracle.lib().lo_f32_to_bf16
    sample = np.concatenate([mid[::7], -mid[::11], just_below[::13], just_above[::17], xs[-2000:]])
    got = np.array([fn(float(v)) for v in sample], np.uint16)
    assert np.array_equal(got, torch_bf16_bits(sample))
    # ties really are present and go to the even code
    assert np.array_equal(torch_bf16_bits(mid), np.where(codes & 1, codes + 1, codes).astype(np.uint16))


def test_moe_forward_bf16_activation_branch_vs_torch(oracle):
    rng = np.random.default_rng(12)
    T, H, I, E, topk = 5, 96, 64, 6, 3
    x = torch.from_numpy(rng.standard_normal((T, H)).astype(np.float32)).to(torch.bfloat16).float().numpy()
    w_gu = (rng.standard_normal((E, 2 * I, H)) * 0.1).astype(np.float32)
    w_dn = (rng.standard_normal((E, H, I)) * 0.1).astype(np.float32)
    sel, wts = oracle.moe_route(rng.standard_normal((T, E)).astype(np.float32), topk)
    got = oracle.moe_forward(x, w_gu, w_dn, sel, wts, act_bf16=True)
    plain = oracle.moe_forward(x, w_gu, w_dn, sel, wts, act_bf16=False)
    xt = torch.from_numpy(x).double()
    want = torch.zeros((T, H), dtype=torch.float64)
    flips = 0
    for t in range(T):
        for s in range(topk):
            e = int(sel[t, s])
            g = torch.from_numpy(w_gu[e, :I]).double() @ xt[t]
            u = torch.from_numpy(w_gu[e, I:]).double() @ xt[t]
            act64 = u * F.silu(g)
            act = act64.float().to(torch.bfloat16)  # the rounding the kernel pipeline applies between its two GEMMs
            # the oracle forms the product in f32 before it rounds: where that double rounding could tip the bf16
            # result, accept either neighbour by taking the oracle's side (counted, must be rare)
            act32 = (u.float() * (g.float() * (1.0 / (1.0 + torch.exp(-g.float()))))).to(torch.bfloat16)
            flips += int((act32 != act).sum())
            want[t] += float(wts[t, s]) * (torch.from_numpy(w_dn[e]).double() @ act32.double())
    assert flips <= 2
    assert np.max(np.abs(got - want.numpy())) < 2e-6 * np.max(np.abs(want.numpy()))
    # and the branch does something: it differs from the unrounded forward by about one bf16 rounding
    rel = np.linalg.norm(got - plain) / np.linalg.norm(plain)
    assert 1e-4 < rel < 4e-3


def torch_llama_forward(cfg, w, tokens, k_cache, v_cache, pos0):
    """Independent restatement in torch (f64): complex-number rotary embedding, repeat_interleave for the
    query groups, scaled_dot_product_attention for scores / mask / softmax, silu on the gate."""
    tw = {k: torch.from_numpy(v).double() for k, v in w.items()}
    hd, hq, hkv = cfg.head_dim, cfg.q_heads, cfg.kv_heads
    s = len(tokens)
    pos = torch.arange(pos0, pos0 + s, dtype=torch.float64)
    inv = 1.0 / cfg.theta ** (torch.arange(0, hd, 2, dtype=torch.float64) / hd)
    rot = torch.polar(torch.ones(s, hd // 2, dtype=torch.float64), pos[:, None] * inv[None, :])  # (s, hd/2)

    def norm(x, g):
        return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + cfg.eps) * g

    def rope(t):  # (s, heads, hd)
        z = torch.view_as_complex(t.reshape(s, -1, hd // 2, 2).contiguous())
        return torch.view_as_real(z * rot[:, None, :]).reshape(s, -1, hd)

    x = tw["embed"][torch.tensor(tokens)]
    for i in range(cfg.layers):
        n = norm(x, tw[f"{i}.attn_norm"])
        q = rope(F.linear(n, tw[f"{i}.q"]).view(s, hq, hd)).transpose(0, 1)      # (hq, s, hd)
        k = rope(F.linear(n, tw[f"{i}.k"]).view(s, hkv, hd)).transpose(0, 1)
        v = F.linear(n, tw[f"{i}.v"]).view(s, hkv, hd).transpose(0, 1)
        k_all = torch.cat([k_cache[i], k], dim=1)
        v_all = torch.cat([v_cache[i], v], dim=1)
        k_cache[i], v_cache[i] = k_all, v_all
        prev = k_all.shape[1] - s
        kk = k_all.repeat_interleave(hq // hkv, dim=0)
        vv = v_all.repeat_interleave(hq // hkv, dim=0)
        if prev == 0:
            att = F.scaled_dot_product_attention(q[None], kk[None], vv[None], is_causal=True)[0]
        else:
            allowed = torch.arange(prev + s)[None, :] <= (prev + torch.arange(s))[:, None]
            att = F.scaled_dot_product_attention(q[None], kk[None], vv[None], attn_mask=allowed)[0]
        x = x + F.linear(att.transpose(0, 1).reshape(s, hq * hd), tw[f"{i}.o"])
        n = norm(x, tw[f"{i}.ffn_norm"])
        x = x + F.linear(F.silu(F.linear(n, tw[f"{i}.gate"])) * F.linear(n, tw[f"{i}.up"]), tw[f"{i}.down"])
    return F.linear(norm(x, tw["out_norm"]), tw["lm_head"]).numpy()


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


@pytest.mark.parametrize("q_heads,kv_heads", [(4, 2), (8, 2), (4, 4), (6, 1)])
def test_llama_forward_vs_torch(q_heads, kv_heads):
    cfg = LlamaConfig(vocab=101, dim=q_heads * 16, layers=2, q_heads=q_heads, kv_heads=kv_heads, ffn=80)
    w = random_f32_weights(cfg, seed=q_heads * 10 + kv_heads)
    toks = [5, 17, 3, 100, 0, 42, 8, 77, 9]
    kc = [np.zeros((cfg.kv_heads, 0, cfg.head_dim)) for _ in range(cfg.layers)]
    vc = [np.zeros((cfg.kv_heads, 0, cfg.head_dim)) for _ in range(cfg.layers)]
    tkc = [torch.zeros((cfg.kv_heads, 0, cfg.head_dim), dtype=torch.float64) for _ in range(cfg.layers)]
    tvc = [torch.zeros((cfg.kv_heads, 0, cfg.head_dim), dtype=torch.float64) for _ in range(cfg.layers)]
    # a prompt pass from position 0, then a three-token continuation through the caches, then single tokens
    pos = 0
    for chunk in (toks[:5], toks[5:8], toks[8:]):
        got = lo.forward(cfg, w, chunk, kc, vc, pos)
        want = torch_llama_forward(cfg, w, chunk, tkc, tvc, pos)
        assert got.shape == want.shape == (len(chunk), cfg.vocab)
        assert np.max(np.abs(got - want)) < 1e-9 * max(1.0, np.max(np.abs(want)))
        pos += len(chunk)
    for i in range(cfg.layers):
        assert np.allclose(kc[i], tkc[i].numpy(), atol=1e-12) and np.allclose(vc[i], tvc[i].numpy(), atol=1e-12)


def test_llama_forward_mistakes_are_caught():
    """The comparison above is sensitive to the slips it is meant to exclude: each of these changes moves the
    torch forward away from the oracle by far more than the tolerance used there."""
    cfg = LlamaConfig(vocab=101, dim=64, layers=2, q_heads=4, kv_heads=2, ffn=80)
    w = random_f32_weights(cfg, seed=3)
    toks = [5, 17, 3, 100, 0, 42]
    empty = lambda: [np.zeros((cfg.kv_heads, 0, cfg.head_dim)) for _ in range(cfg.layers)]  # noqa: E731
    base = lo.forward(cfg, w, toks, empty(), empty(), 0)
    # gate and up exchanged (swish on the wrong branch)
    w2 = dict(w)
    for i in range(cfg.layers):
        w2[f"{i}.gate"], w2[f"{i}.up"] = w[f"{i}.up"], w[f"{i}.gate"]
    assert np.max(np.abs(lo.forward(cfg, w2, toks, empty(), empty(), 0) - base)) > 1e-3
    # KV heads exchanged (a wrong query-head -> KV-head map)
    w3 = dict(w)
    hd = cfg.head_dim
    for i in range(cfg.layers):
        for name in ("k", "v"):
            m = w[f"{i}.{name}"].reshape(cfg.kv_heads, hd, cfg.dim)
            w3[f"{i}.{name}"] = np.ascontiguousarray(m[::-1]).reshape(cfg.kv_heads * hd, cfg.dim)
    assert np.max(np.abs(lo.forward(cfg, w3, toks, empty(), empty(), 0) - base)) > 1e-3
