"""The Llama-3 decode loop through the C ABI against the numpy oracle, on small
configurations of the same architecture (the oracle cannot run 8B parameters in
test time): single operators, f32 prefill + decode logits within 2e-3, graph
replay equal to eager stepping, bf16 prefill within what its own roundings cost (measured in the test against a
restatement with the same roundings)."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from conftest import rel_err  # noqa: E402
from luminal_amd import capi, synth  # noqa: E402
from luminal_amd.llama import LlamaConfig, LlamaQ8, fuse_rows, interleave_rows, random_weights  # noqa: E402
from luminal_amd.quantized import Q8Weight  # noqa: E402
from oracle import llama_oracle as lo  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def s():
    return torch.cuda.current_stream().cuda_stream


def build_model(oracle, cfg, seed, max_seq=64):
    """Random Q8_0 model: returns (engine, dequantised f32 weights for the oracle)."""
    rng = np.random.default_rng(seed)
    hd = cfg.head_dim
    wf, raws = {}, {}

    def q8(name, n, k, i):
        qs, d = synth.q8_0_random(n, k, seed=seed * 1000 + i, scale_sigma=float(np.sqrt(3.0 / k) / 0.8))
        raw = synth.q8_0_raw_blocks(qs, d)
        raws[name] = raw
        wf[name] = oracle.q8_0_dequant(raw, n * k).reshape(n, k)

    wf["embed"] = rng.standard_normal((cfg.vocab, cfg.dim)).astype(np.float32)
    wf["out_norm"] = (1 + 0.05 * rng.standard_normal(cfg.dim)).astype(np.float32)
    q8("lm_head", cfg.vocab, cfg.dim, 0)
    for i in range(cfg.layers):
        wf[f"{i}.attn_norm"] = (1 + 0.05 * rng.standard_normal(cfg.dim)).astype(np.float32)
        wf[f"{i}.ffn_norm"] = (1 + 0.05 * rng.standard_normal(cfg.dim)).astype(np.float32)
        for j, (nm, n, k) in enumerate([("q", cfg.dim, cfg.dim), ("k", cfg.kv_heads * hd, cfg.dim),
                                        ("v", cfg.kv_heads * hd, cfg.dim), ("o", cfg.dim, cfg.dim),
                                        ("gate", cfg.ffn, cfg.dim), ("up", cfg.ffn, cfg.dim),
                                        ("down", cfg.dim, cfg.ffn)]):
            q8(f"{i}.{nm}", n, k, 10 * i + j + 1)
    w = {"embed": torch.from_numpy(wf["embed"]).to(DEV), "out_norm": torch.from_numpy(wf["out_norm"]).to(DEV),
         "lm_head": Q8Weight.from_raw(raws["lm_head"], cfg.vocab, cfg.dim, DEV)}
    for i in range(cfg.layers):
        w[f"{i}.attn_norm"] = torch.from_numpy(wf[f"{i}.attn_norm"]).to(DEV)
        w[f"{i}.ffn_norm"] = torch.from_numpy(wf[f"{i}.ffn_norm"]).to(DEV)
        w[f"{i}.qkv"] = Q8Weight.from_raw(fuse_rows(raws[f"{i}.q"], raws[f"{i}.k"], raws[f"{i}.v"]), cfg.qkv_rows,
                                          cfg.dim, DEV)
        w[f"{i}.o"] = Q8Weight.from_raw(raws[f"{i}.o"], cfg.dim, cfg.dim, DEV)
        w[f"{i}.gate_up"] = Q8Weight.from_raw(interleave_rows(raws[f"{i}.gate"], raws[f"{i}.up"], cfg.dim), 2 * cfg.ffn, cfg.dim, DEV)
        w[f"{i}.down"] = Q8Weight.from_raw(raws[f"{i}.down"], cfg.dim, cfg.ffn, DEV)
    return LlamaQ8(cfg, w, max_seq, DEV), wf


def empty_cache(cfg):
    return [np.zeros((cfg.kv_heads, 0, cfg.head_dim)) for _ in range(cfg.layers)]


# ------------------------------------------------------------------ single operators

def test_rms_norm_and_fused_residual():
    lib = capi.load_library()
    rng = np.random.default_rng(1)
    x = rng.standard_normal((5, 4096)).astype(np.float32)
    r = rng.standard_normal((5, 4096)).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(4096)).astype(np.float32)
    xd, rd, wd = (torch.from_numpy(a).to(DEV) for a in (x, r, w))
    y = torch.empty_like(xd)
    assert lib.lhip_rms_norm_f32(xd.data_ptr(), None, None, wd.data_ptr(), y.data_ptr(), 5, 4096, 1e-5, s()) == 0
    assert rel_err(y.cpu().numpy(), lo.rms_norm(x, w, 1e-5)) < 1e-5
    xo = torch.empty_like(xd)
    assert lib.lhip_rms_norm_f32(xd.data_ptr(), rd.data_ptr(), xo.data_ptr(), wd.data_ptr(), y.data_ptr(), 5, 4096,
                                 1e-5, s()) == 0
    assert np.array_equal(xo.cpu().numpy(), x + r)
    assert rel_err(y.cpu().numpy(), lo.rms_norm(x + r, w, 1e-5)) < 1e-5


def test_rope_attention_swiglu_gather_argmax():
    lib = capi.load_library()
    rng = np.random.default_rng(2)
    hq, hkv, hd, max_seq, S, pos0 = 8, 2, 128, 40, 6, 9
    qkv = rng.standard_normal((S, (hq + 2 * hkv) * hd)).astype(np.float32)
    kc = rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)
    vc = rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)
    qd, kd, vd = (torch.from_numpy(a.copy()).to(DEV) for a in (qkv, kc, vc))
    pos = torch.tensor([pos0], dtype=torch.int32, device=DEV)
    assert lib.lhip_rope_kv_append_f32(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), pos.data_ptr(), S, hq, hkv, hd,
                                       max_seq, 500000.0, s()) == 0
    rows = qkv.reshape(S, hq + 2 * hkv, hd)
    q_want = lo.rope(rows[:, :hq].astype(np.float64), pos0, 500000.0)
    k_want = lo.rope(rows[:, hq:hq + hkv].astype(np.float64), pos0, 500000.0)
    got = qd.cpu().numpy().reshape(S, hq + 2 * hkv, hd)
    assert np.max(np.abs(got[:, :hq] - q_want)) < 2e-5 and np.max(np.abs(got[:, hq:hq + hkv] - k_want)) < 2e-5
    assert np.array_equal(got[:, hq + hkv:], rows[:, hq + hkv:])  # v untouched
    kc2, vc2 = kd.cpu().numpy(), vd.cpu().numpy()
    assert np.max(np.abs(kc2[:, pos0:pos0 + S] - k_want.transpose(1, 0, 2))) < 2e-5
    assert np.array_equal(vc2[:, pos0:pos0 + S], rows[:, hq + hkv:].transpose(1, 0, 2))
    assert np.array_equal(kc2[:, :pos0], kc[:, :pos0]) and np.array_equal(kc2[:, pos0 + S:], kc[:, pos0 + S:])
    # attention over the updated cache
    out = torch.empty((S, hq * hd), dtype=torch.float32, device=DEV)
    assert lib.lhip_attention_f32(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(), pos.data_ptr(), S, hq,
                                  hkv, hd, max_seq, s()) == 0
    want = np.empty((S, hq, hd))
    for t in range(S):
        n_keys = pos0 + t + 1
        for h in range(hq):
            sc = kc2[h // (hq // hkv), :n_keys].astype(np.float64) @ got[t, h].astype(np.float64) / np.sqrt(hd)
            p = np.exp(sc - sc.max())
            want[t, h] = (p / p.sum()) @ vc2[h // (hq // hkv), :n_keys].astype(np.float64)
    assert rel_err(out.cpu().numpy(), want.reshape(S, -1)) < 1e-3
    # swiglu
    gu = rng.standard_normal((3, 2 * 96)).astype(np.float32)
    o = torch.empty((3, 96), dtype=torch.float32, device=DEV)
    assert lib.lhip_swiglu_f32(torch.from_numpy(gu).to(DEV).data_ptr(), o.data_ptr(), 3, 96, 0, s()) == 0
    assert rel_err(o.cpu().numpy(), gu[:, 96:] * lo.swish(gu[:, :96].astype(np.float64))) < 1e-5
    # fp32 row gather with f32 ids, argmax with the reference's tie rule (last maximum wins)
    table = rng.standard_normal((50, 64)).astype(np.float32)
    ids = torch.tensor([3.0, 49.0, 0.0, 7.9], device=DEV)
    g = torch.empty((4, 64), dtype=torch.float32, device=DEV)
    assert lib.lhip_gather_rows_f32(torch.from_numpy(table).to(DEV).data_ptr(), ids.data_ptr(), g.data_ptr(), 4, 50,
                                    64, s()) == 0
    assert np.array_equal(g.cpu().numpy(), table[[3, 49, 0, 7]])
    v = rng.standard_normal(5000).astype(np.float32)
    v[[17, 4021, 333]] = 9.5
    idf = torch.zeros(1, device=DEV)
    idi = torch.zeros(1, dtype=torch.int32, device=DEV)
    assert lib.lhip_argmax_f32(torch.from_numpy(v).to(DEV).data_ptr(), 5000, idf.data_ptr(), idi.data_ptr(),
                               pos.data_ptr(), 3, s()) == 0
    assert int(idi.item()) == 4021 == lo.argmax_last(v) and idf.item() == 4021.0 and int(pos.item()) == pos0 + 3


def test_attention_over_the_longest_cache():
    """max_seq = 12000 (the operator's limit): 48 000 bytes of scores on top of the kernel's static arrays is more
    LDS than a kernel gets without asking; three tokens at positions 11 990 .. 11 992 against a direct softmax."""
    lib = capi.load_library()
    rng = np.random.default_rng(8)
    hq, hkv, hd, max_seq, S, pos0 = 4, 2, 64, 12000, 3, 11990
    qkv = rng.standard_normal((S, (hq + 2 * hkv) * hd)).astype(np.float32)
    kc = rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)
    vc = rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)
    qd, kd, vd = (torch.from_numpy(a).to(DEV) for a in (qkv, kc, vc))
    pos = torch.tensor([pos0], dtype=torch.int32, device=DEV)
    out = torch.full((S, hq * hd), float("nan"), dtype=torch.float32, device=DEV)
    assert lib.lhip_attention_f32(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(), pos.data_ptr(), S, hq,
                                  hkv, hd, max_seq, s()) == 0
    torch.cuda.synchronize()
    q = qkv.reshape(S, hq + 2 * hkv, hd)[:, :hq].astype(np.float64)
    want = np.empty((S, hq, hd))
    for t in range(S):
        for h in range(hq):
            sc = kc[h // (hq // hkv), :pos0 + t + 1].astype(np.float64) @ q[t, h] / np.sqrt(hd)
            p = np.exp(sc - sc.max())
            want[t, h] = (p / p.sum()) @ vc[h // (hq // hkv), :pos0 + t + 1].astype(np.float64)
    assert rel_err(out.cpu().numpy(), want.reshape(S, -1)) < 1e-3
    assert lib.lhip_attention_f32(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(), pos.data_ptr(), S, hq,
                                  hkv, hd, max_seq + 1, s()) == capi.LHIP_ERR_INVALID_SHAPE


@pytest.mark.parametrize("n", [16384, 16387, 128256, 128259, 1 << 20])
def test_argmax_of_long_rows(n):
    """Rows long enough for the two-launch pick (partial picks over 64 workgroups, then one wave): ties in several
    workgroups' parts (the last index wins), the maximum among the n % 4 trailing entries, an unaligned row (the
    single-workgroup kernel), all entries equal, and rows of -inf / lowest finite values."""
    lib = capi.load_library()
    rng = np.random.default_rng(n)
    idi = torch.zeros(1, dtype=torch.int32, device=DEV)
    idf = torch.zeros(1, device=DEV)
    pos = torch.tensor([5], dtype=torch.int32, device=DEV)

    def pick(v, offset=0):
        buf = torch.zeros(len(v) + 4, device=DEV)
        buf[offset:offset + len(v)] = torch.from_numpy(v).to(DEV)
        assert lib.lhip_argmax_f32(buf.data_ptr() + 4 * offset, len(v), idf.data_ptr(), idi.data_ptr(), pos.data_ptr(), 1,
                                   s()) == 0
        assert idf.item() == float(idi.item())
        return int(idi.item())

    v = rng.standard_normal(n).astype(np.float32)
    assert pick(v) == lo.argmax_last(v)
    ties = rng.choice(n, 9, replace=False)
    v[ties] = 11.0
    assert pick(v) == int(ties.max()) == lo.argmax_last(v)
    assert pick(v, offset=1) == int(ties.max())            # row not 16-byte aligned
    v[n - 1] = 12.0                                        # in the trailing entries when n % 4 != 0
    assert pick(v) == n - 1
    v[0] = 13.0
    assert pick(v) == 0
    assert pick(np.full(n, 2.5, np.float32)) == n - 1
    assert pick(np.full(n, -np.inf, np.float32)) == n - 1
    low = np.full(n, np.finfo(np.float32).min, np.float32)
    low[n // 2] = -np.inf
    assert pick(low) == n - 1
    assert int(pos.item()) == 5 + 8


@pytest.mark.parametrize("hq,hkv,hd", [(8, 2, 128), (32, 8, 128), (4, 4, 64), (16, 2, 64), (4, 2, 128)])
@pytest.mark.parametrize("pos0", [0, 1, 63, 64, 200, 1500])
def test_decode_attention_equals_rope_append_attention(hq, hkv, hd, pos0):
    """The one-launch decode attention against an f64 restatement of rotary + append + softmax(QK)V, at positions
    that leave key ranges empty, ragged and many tiles long; three consecutive tokens share one workspace."""
    lib = capi.load_library()
    rng = np.random.default_rng(hq * 1000 + pos0)
    max_seq = 1600
    kc = rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)
    vc = rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)
    kd, vd = torch.from_numpy(kc.copy()).to(DEV), torch.from_numpy(vc.copy()).to(DEV)
    nws = lib.lhip_attention_decode_workspace_nbytes(hq, hkv, hd)
    assert nws > 0
    ws = torch.full((nws,), 0xFF, dtype=torch.uint8, device=DEV)  # contents on entry do not matter
    out = torch.empty(hq * hd, device=DEV)
    g = hq // hkv
    for step in range(3):
        p = pos0 + step
        qkv = (2.0 * rng.standard_normal((hq + 2 * hkv, hd))).astype(np.float32)
        pos = torch.tensor([p], dtype=torch.int32, device=DEV)
        qd = torch.from_numpy(qkv.copy()).to(DEV)
        assert lib.lhip_attention_decode_f32(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(),
                                             pos.data_ptr(), hq, hkv, hd, max_seq, 500000.0, ws.data_ptr(), s()) == 0
        assert np.array_equal(qd.cpu().numpy(), qkv)  # the input row is left alone
        q_r = lo.rope(qkv[None, :hq].astype(np.float64), p, 500000.0)[0]
        k_r = lo.rope(qkv[None, hq:hq + hkv].astype(np.float64), p, 500000.0)[0]
        kc[:, p], vc[:, p] = k_r, qkv[hq + hkv:]
        want = np.empty((hq, hd))
        for h in range(hq):
            sc = kc[h // g, :p + 1].astype(np.float64) @ q_r[h] / np.sqrt(hd)
            w = np.exp(sc - sc.max())
            want[h] = (w / w.sum()) @ vc[h // g, :p + 1].astype(np.float64)
        # f32 rotary angles and softmax: judged against the scale of the output vector (elements that cancel to
        # ~0 carry the same absolute rounding error as the rest)
        err = np.max(np.abs(out.cpu().numpy() - want.reshape(-1))) / np.sqrt(np.mean(want * want))
        # plus the f32 rotary angle: half an ulp of p turns q and k by p * 2^-24 rad, which moves a score by that
        # times |q||k|/sqrt(hd) (~25 here)
        assert err < 1e-4 + 25 * p * 2.0 ** -24, (step, p, err)
        kgot, vgot = kd.cpu().numpy(), vd.cpu().numpy()
        # the f32 angle p * inv_freq is off by up to half an ulp of p, which turns the pair by that much
        k_tol = 2e-5 + p * 2.0 ** -23 * float(np.max(np.abs(qkv)))
        assert np.max(np.abs(kgot[:, p] - k_r)) < k_tol and np.array_equal(vgot[:, p], qkv[hq + hkv:])
        kc[:, p] = kgot[:, p]  # continue from the device's f32 rounding of the new key
        assert np.array_equal(kgot, kc) and np.array_equal(vgot, vc)  # nothing else in the caches moved


@pytest.mark.parametrize("hq,hkv,hd", [(8, 2, 128), (32, 8, 128), (4, 4, 64), (16, 2, 64), (4, 2, 128), (8, 8, 128)])
@pytest.mark.parametrize("S,pos0", [(8, 0), (33, 0), (70, 5), (64, 64), (129, 31)])
def test_prompt_attention_on_matrix_cores(hq, hkv, hd, S, pos0):
    """Calls of 8 or more tokens take the matrix-core kernel: against the f64 softmax(QK)V over the cache, for
    query blocks and key tiles that are ragged, start mid-cache and span several tiles."""
    lib = capi.load_library()
    rng = np.random.default_rng(hq * 100 + S + pos0)
    max_seq = 200
    kc = rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)
    vc = rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)
    qkv = rng.standard_normal((S, hq + 2 * hkv, hd)).astype(np.float32)
    kd, vd, qd = (torch.from_numpy(a).to(DEV) for a in (kc, vc, qkv))
    pos = torch.tensor([pos0], dtype=torch.int32, device=DEV)
    out = torch.full((S, hq * hd), float("nan"), device=DEV)
    assert lib.lhip_attention_f32(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(), pos.data_ptr(), S, hq,
                                  hkv, hd, max_seq, s()) == 0
    g = hq // hkv
    want = np.empty((S, hq, hd))
    for t in range(S):
        n = pos0 + t + 1
        for h in range(hq):
            sc = kc[h // g, :n].astype(np.float64) @ qkv[t, h].astype(np.float64) / np.sqrt(hd)
            w = np.exp(sc - sc.max())
            want[t, h] = (w / w.sum()) @ vc[h // g, :n].astype(np.float64)
    err = np.max(np.abs(out.cpu().numpy() - want.reshape(S, -1))) / np.sqrt(np.mean(want * want))
    assert err < 1e-5, err


# ---- the bf16 prompt pass through a whole stack.
# oracle.llama_oracle.forward_prompt_bf16 is the pass in f64 with the bf16 roundings in the engine's places.  Its
# distance from the exact f64 pass is what bf16 operands cost (unit roundoff 2^-9 on every operand of every product:
# about 1.1e-3 of a product's rms each, nine per layer, added in quadrature along the residual stream, the maximum
# over a few thousand logits four to five deviations out: 1e-2 to 3e-2 of the logits' rms on these two-layer stacks),
# and the tests compute it.  The engine cannot be held to a tighter bar against that restatement than against the
# truth: measured stage by stage on the 4096 / 14336 layer, q, k and v of the first layer agree to 3e-4 of their rms
# (one element of the normed input lands on the other side of a rounding boundary under f32 arithmetic and moves a
# whole row by that), the attention given the engine's own q, k, v agrees bit for bit, but that 3e-4 flips 2 % of the
# attention's output roundings by one bf16 ulp each, those flip 38 % of the SwiGLU roundings, and after one layer two
# faithful implementations differ by about as much as either differs from the truth.  (Where no rounding tips - most of
# the small stacks below - the engine agrees with the restatement to 3e-7 ... 1.5e-6 of the logits' rms, which is what
# shows the restatement to be the engine's arithmetic; one tip and the figure is 7e-3 to 2e-2.)  Every operator is held tightly
# on its own inputs elsewhere in this file and in test_q8_gemm_gpu.py; the stack is held to: no further from the truth,
# and from the restatement, than 1.5 times what the roundings themselves cost.
BF16_STACK_FACTOR = 1.5


def uses_bf16_attention(cfg):
    """Head shapes for which the prompt pass takes lhip_attention_bf16 (else attention in f32, result rounded)."""
    return cfg.head_dim in (64, 128) and cfg.q_heads // cfg.kv_heads in (2, 4, 8)


def check_bf16_stack(got, exact, rounded, what=""):
    """got: the engine's logits; exact: the f64 pass; rounded: the f64 pass with the engine's bf16 roundings."""
    rms = float(np.sqrt(np.mean(exact * exact)))
    to_rounded = float(np.max(np.abs(got - rounded))) / rms
    budget = float(np.max(np.abs(rounded - exact))) / rms
    to_exact = float(np.max(np.abs(got - exact))) / rms
    print(f"[bf16 stack{what}] engine vs exact {to_exact:.2e}, restatement with the same roundings vs exact {budget:.2e}, "
          f"engine vs restatement {to_rounded:.2e} (of the logits' rms)")
    assert 1e-4 < budget < 5e-2, (what, budget)
    assert to_exact < BF16_STACK_FACTOR * budget, (what, to_exact, budget)
    assert to_rounded < BF16_STACK_FACTOR * budget, (what, to_rounded, budget)


def _bf16(x):
    """Round to bfloat16 (nearest even) and return as float64."""
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).bfloat16().double().numpy()


def _attention_with_bf16_roundings(qkv, kc, vc, hq, hkv, hd, pos0):
    """softmax(QK)V in f64 with the five roundings of the bf16 kernel placed where it places them: q / sqrt(hd), K and
    V rounded once; per 32-key tile the weights exp(s - running max) rounded and the running sum taken over the
    rounded weights; the quotient rounded at the store."""
    S, g = qkv.shape[0], hq // hkv
    q = _bf16(qkv[:, :hq].astype(np.float32) * (np.float32(1.0) / np.sqrt(np.float32(hd))))
    kb, vb = _bf16(kc), _bf16(vc)
    n_keys = pos0 + S
    out = np.empty((S, hq, hd))
    visible = np.arange(n_keys)[None, :] <= (pos0 + np.arange(S))[:, None]
    for h in range(hq):
        sc = np.where(visible, q[:, h] @ kb[h // g, :n_keys].T, -np.inf)
        m = np.full(S, -np.inf)
        l, acc = np.zeros(S), np.zeros((S, hd))
        for k0 in range(0, n_keys, 32):
            tile = sc[:, k0:k0 + 32]
            m_new = np.maximum(m, tile.max(axis=1))
            corr = np.exp(m - m_new)
            w = _bf16(np.exp(tile - m_new[:, None]))
            l = l * corr + w.sum(axis=1)
            acc = acc * corr[:, None] + w @ vb[h // g, k0:k0 + 32][:w.shape[1]]
            m = m_new
        out[:, h] = _bf16(acc / l[:, None])
    return out.reshape(S, -1)


@pytest.mark.parametrize("hq,hkv,hd", [(8, 2, 128), (32, 8, 128), (16, 2, 64), (4, 2, 128), (8, 4, 64), (16, 2, 128)])
@pytest.mark.parametrize("S,pos0", [(8, 0), (33, 0), (70, 5), (64, 64), (129, 31), (300, 0)])
def test_prompt_attention_with_bf16_operands(hq, hkv, hd, S, pos0):
    """The bf16 matrix-core form, for query blocks and key tiles that are ragged, start mid-cache and span several
    tiles, against two references.

    (1) f64 arithmetic with the kernel's five bf16 roundings (q, K, V, soft-max weights, result) in their places. What
        is left is f32 against f64 accumulation and the roundings it tips, of which one at the store moves an element
        by one bf16 ulp, at most 2^-7 of its size: max |y - r| / max(|r|, rms(r)) < 1e-2.
    (2) the exact f64 softmax(QK)V = sum_j p_j v_j, with the error measured against the sum before cancellation,
        a = sum_j p_j |v_j|, per element. bf16's unit roundoff is 2^-8: the roundings of V, of the weights and of
        the result bound the error by 3 * 2^-8 * a = 1.2e-2 * a between them, and the rounding of q and K adds the
        relative error of a weight that the soft-max makes of an error of a score (restated on the CPU, the five
        together reach 1.1e-2 * a on these inputs): |y - t| < 2e-2 * a.
    The f32-operand kernel behind lhip_attention_f32 and lhip_attention_f32_bf16out is the one held to 1e-5."""
    lib = capi.load_library()
    rng = np.random.default_rng(hq * 100 + S + pos0 + 7)
    max_seq = 384
    kc = rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)
    vc = rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)
    qkv = rng.standard_normal((S, hq + 2 * hkv, hd)).astype(np.float32)
    kd, vd, qd = (torch.from_numpy(a).to(DEV) for a in (kc, vc, qkv))
    pos = torch.tensor([pos0], dtype=torch.int32, device=DEV)
    out = torch.full((S, hq * hd), float("nan"), device=DEV, dtype=torch.bfloat16)
    assert lib.lhip_attention_bf16(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(), pos.data_ptr(), S, hq,
                                   hkv, hd, max_seq, s()) == 0
    got = out.double().cpu().numpy()
    g = hq // hkv
    exact, scale = np.empty((S, hq, hd)), np.empty((S, hq, hd))
    for t in range(S):
        n = pos0 + t + 1
        for h in range(hq):
            sc = kc[h // g, :n].astype(np.float64) @ qkv[t, h].astype(np.float64) / np.sqrt(hd)
            w = np.exp(sc - sc.max())
            w /= w.sum()
            exact[t, h] = w @ vc[h // g, :n].astype(np.float64)
            scale[t, h] = w @ np.abs(vc[h // g, :n].astype(np.float64))
    rounded = _attention_with_bf16_roundings(qkv, kc, vc, hq, hkv, hd, pos0)
    e1 = np.max(np.abs(got - rounded) / np.maximum(np.abs(rounded), np.sqrt(np.mean(rounded * rounded))))
    e2 = np.max(np.abs(got - exact.reshape(S, -1)) / scale.reshape(S, -1))
    assert e1 < 1e-2 and e2 < 2e-2, (e1, e2)
    # a query that sees one key returns that key's V row, rounded
    if pos0 == 0:
        assert np.array_equal(got[0].reshape(hq, hd), np.repeat(_bf16(vc[:, 0]), g, axis=0))
    # the caches are only read
    assert np.array_equal(kd.cpu().numpy(), kc) and np.array_equal(vd.cpu().numpy(), vc)


def test_bf16_prompt_attention_argument_errors():
    lib = capi.load_library()
    a = torch.zeros(1 << 16, device=DEV)
    pos = torch.zeros(1, dtype=torch.int32, device=DEV)

    def call(S=8, hq=8, hkv=2, hd=128, qkv=a.data_ptr(), out=a.data_ptr(), max_seq=8):
        return lib.lhip_attention_bf16(qkv, a.data_ptr(), a.data_ptr(), out, pos.data_ptr(), S, hq, hkv, hd, max_seq, s())

    assert call() == capi.LHIP_OK
    assert call(hq=4, hkv=4) == capi.LHIP_ERR_UNSUPPORTED  # one query head per key head has no bf16 kernel
    assert call(hq=32, hkv=2) == capi.LHIP_ERR_UNSUPPORTED and call(hd=32) == capi.LHIP_ERR_UNSUPPORTED
    assert call(hq=7, hkv=2) == capi.LHIP_ERR_INVALID_SHAPE and call(max_seq=0) == capi.LHIP_ERR_INVALID_SHAPE
    assert call(qkv=None) == capi.LHIP_ERR_NULL_PTR and call(out=None) == capi.LHIP_ERR_NULL_PTR
    assert call(S=0) == capi.LHIP_ERR_INVALID_SHAPE
    torch.cuda.synchronize()


def test_decode_attention_argument_errors():
    lib = capi.load_library()
    a = torch.zeros(4096, device=DEV)
    pos = torch.zeros(1, dtype=torch.int32, device=DEV)
    ws = torch.zeros(1 << 20, dtype=torch.uint8, device=DEV)

    def call(hq=8, hkv=2, hd=128, qkv=a.data_ptr(), w=ws.data_ptr(), max_seq=4):
        return lib.lhip_attention_decode_f32(qkv, a.data_ptr(), a.data_ptr(), a.data_ptr(), pos.data_ptr(), hq, hkv, hd,
                                             max_seq, 1e4, w, s())

    assert call() == capi.LHIP_OK
    assert call(hq=6, hkv=2) == capi.LHIP_ERR_UNSUPPORTED and lib.lhip_attention_decode_workspace_nbytes(6, 2, 128) == 0
    assert call(hd=256) == capi.LHIP_ERR_UNSUPPORTED
    assert call(hq=7, hkv=2) == capi.LHIP_ERR_INVALID_SHAPE
    assert call(max_seq=0) == capi.LHIP_ERR_INVALID_SHAPE
    assert call(qkv=None) == capi.LHIP_ERR_NULL_PTR and call(w=None) == capi.LHIP_ERR_NULL_PTR
    assert call(w=ws.data_ptr() + 16) == capi.LHIP_ERR_MISALIGNED
    torch.cuda.synchronize()


# ------------------------------------------------------------------ end to end

@pytest.mark.parametrize("cfg", [LlamaConfig(vocab=512, dim=256, layers=2, q_heads=4, kv_heads=2, ffn=512),
                                 LlamaConfig(vocab=1000, dim=1024, layers=3, q_heads=8, kv_heads=2, ffn=2048)])
def test_prefill_and_decode_logits_vs_oracle(oracle, cfg):
    eng, wf = build_model(oracle, cfg, seed=cfg.dim)
    assert eng.fused_decode == (cfg.dim == 1024)  # the second configuration decodes through the fused matvecs
    rng = np.random.default_rng(3)
    prompt = [int(t) for t in rng.integers(0, cfg.vocab, 12)]
    kc, vc = empty_cache(cfg), empty_cache(cfg)
    want = lo.forward(cfg, wf, prompt, kc, vc, 0)
    got = eng.forward(torch.tensor(prompt, dtype=torch.float32, device=DEV), len(prompt), all_logits=True)
    assert rel_err(got.cpu().numpy(), want) < 2e-3
    # generation loop: prefill picks a token, then teacher-forced comparison of every decode step's logits
    eng.reset()
    eng.prefill(prompt)
    tok = lo.argmax_last(want[-1])
    assert int(eng.tok_i.item()) == tok and int(eng.pos.item()) == len(prompt)
    for step in range(6):
        want_step = lo.forward(cfg, wf, [tok], kc, vc, len(prompt) + step)[0]
        logits = eng.decode_step()
        assert rel_err(logits.cpu().numpy(), want_step) < 2e-3, step
        tok = lo.argmax_last(want_step)
        # keep both sides on the oracle's token even if a near-tie flipped the pick
        eng.tok.fill_(float(tok))
        eng.tok_i.fill_(tok)


def test_llama3_8b_layer_dimensions_vs_oracle(oracle):
    """Two layers with the real Llama-3-8B dimensions (examples/llama/src/model.rs:5-14: dim 4096, 32 query and 8 KV
    heads of 128, FFN 14336; a small vocabulary keeps the oracle's lm_head cheap): the f32 prompt pass, the bf16
    prompt pass and fused-matvec decode steps (eager and replayed from a graph) against the numpy oracle."""
    cfg = LlamaConfig(vocab=2048, dim=4096, layers=2, q_heads=32, kv_heads=8, ffn=14336)
    eng, wf = build_model(oracle, cfg, seed=31, max_seq=64)
    assert eng.fused_decode
    rng = np.random.default_rng(5)
    prompt = [int(t) for t in rng.integers(0, cfg.vocab, 16)]
    kc, vc = empty_cache(cfg), empty_cache(cfg)
    want = lo.forward(cfg, wf, prompt, kc, vc, 0)
    got = eng.forward(torch.tensor(prompt, dtype=torch.float32, device=DEV), len(prompt), all_logits=True)
    assert rel_err(got.cpu().numpy(), want) < 2e-3
    gotb = eng.forward(torch.tensor(prompt, dtype=torch.float32, device=DEV), len(prompt), bf16=True, all_logits=True)
    assert uses_bf16_attention(cfg)
    check_bf16_stack(gotb.cpu().numpy(), want, lo.forward_prompt_bf16(cfg, wf, prompt)[0], " 4096/14336, 2 layers")
    eng.reset()
    eng.prefill(prompt)
    tok = lo.argmax_last(want[-1])
    assert int(eng.tok_i.item()) == tok and int(eng.pos.item()) == len(prompt)
    for step in range(3):
        want_step = lo.forward(cfg, wf, [tok], kc, vc, len(prompt) + step)[0]
        logits = eng.decode_step()
        assert rel_err(logits.cpu().numpy(), want_step) < 2e-3, step
        tok = lo.argmax_last(want_step)
        eng.tok.fill_(float(tok))
        eng.tok_i.fill_(tok)
    # greedy decode replayed from a graph picks the tokens eager stepping picks
    eng.reset()
    eng.prefill(prompt)
    eager = eng.decode(6, use_graph=False).cpu().numpy()
    eng.reset()
    eng.prefill(prompt)
    assert np.array_equal(eng.decode(6, use_graph=True).cpu().numpy(), eager)


@pytest.mark.parametrize("cfg", [LlamaConfig(vocab=512, dim=256, layers=2, q_heads=4, kv_heads=2, ffn=512),
                                 LlamaConfig(vocab=700, dim=1024, layers=2, q_heads=8, kv_heads=4, ffn=1024)])
def test_graph_replay_equals_eager_decode(oracle, cfg):
    eng, _ = build_model(oracle, cfg, seed=7)
    prompt = [1, 2, 3, 4, 5]
    eng.prefill(prompt)
    eager = eng.decode(10, use_graph=False).cpu().numpy()
    eng.reset()
    eng.prefill(prompt)
    graphed = eng.decode(10, use_graph=True).cpu().numpy()
    assert np.array_equal(eager, graphed)
    # a second run re-uses the captured graph
    eng.reset()
    eng.prefill(prompt)
    assert np.array_equal(eng.decode(10, use_graph=True).cpu().numpy(), eager)


@pytest.mark.parametrize("cfg", [LlamaConfig(vocab=512, dim=256, layers=2, q_heads=4, kv_heads=2, ffn=512),
                                 LlamaConfig(vocab=700, dim=1024, layers=2, q_heads=8, kv_heads=2, ffn=2048),
                                 LlamaConfig(vocab=300, dim=768, layers=1, q_heads=12, kv_heads=4, ffn=256)])
def test_bf16_prefill_then_f32_decode(oracle, cfg):
    """The prompt pass on the bf16 GEMM (the third configuration has 3 query heads per KV head, for which there is
    no matrix-core attention: it takes the f32 attention + cast branch)."""
    eng, wf = build_model(oracle, cfg, seed=9)
    prompt = [int(t) for t in np.random.default_rng(4).integers(0, cfg.vocab, 20)]
    kc, vc = empty_cache(cfg), empty_cache(cfg)
    want = lo.forward(cfg, wf, prompt, kc, vc, 0)
    bfa = uses_bf16_attention(cfg)
    assert bfa == (cfg.q_heads // cfg.kv_heads != 3)
    got = eng.prefill(prompt, bf16=True).cpu().numpy()
    last_rounded, kcb, vcb = lo.forward_prompt_bf16(cfg, wf, prompt, bf16_attention=bfa, all_logits=False)
    check_bf16_stack(got, np.asarray(want[-1]), last_rounded, " last position")
    eng.reset()
    allpos = eng.forward(torch.tensor(prompt, dtype=torch.float32, device=DEV), len(prompt), bf16=True,
                         all_logits=True).cpu().numpy()
    check_bf16_stack(allpos, want, lo.forward_prompt_bf16(cfg, wf, prompt, bf16_attention=bfa)[0], " all positions")
    # the f32 decode step continues from the cache the bf16 pass wrote: against the f32 oracle step over the exact
    # caches (the budget of the bf16 pass) and over the caches of the rounded restatement (the f32 tolerance)
    eng.reset()
    eng.prefill(prompt, bf16=True)
    tok = lo.argmax_last(want[-1])
    eng.tok.fill_(float(tok))
    step = lo.forward(cfg, wf, [tok], kc, vc, len(prompt))[0]
    step_rounded = lo.forward(cfg, wf, [tok], kcb, vcb, len(prompt))[0]
    check_bf16_stack(eng.decode_step().cpu().numpy(), step, step_rounded, " f32 step after the bf16 prompt")


def test_bf16_output_forms_equal_the_rounded_f32_forms():
    """rms norm, SwiGLU and prompt attention writing bf16 are the f32 operators followed by round-to-nearest-even."""
    lib = capi.load_library()
    rng = np.random.default_rng(8)

    def rounded(t):
        return t.to(torch.bfloat16)

    rows, dim = 5, 1024
    x = torch.from_numpy(rng.standard_normal((rows, dim)).astype(np.float32)).to(DEV)
    res = torch.from_numpy(rng.standard_normal((rows, dim)).astype(np.float32)).to(DEV)
    g = torch.from_numpy((1 + 0.1 * rng.standard_normal(dim)).astype(np.float32)).to(DEV)
    y32, xo32 = torch.empty_like(x), torch.empty_like(x)
    y16 = torch.empty((rows, dim), dtype=torch.bfloat16, device=DEV)
    xo16 = torch.empty_like(x)
    assert lib.lhip_rms_norm_f32(x.data_ptr(), res.data_ptr(), xo32.data_ptr(), g.data_ptr(), y32.data_ptr(), rows, dim,
                                 1e-5, s()) == 0
    assert lib.lhip_rms_norm_f32_bf16out(x.data_ptr(), res.data_ptr(), xo16.data_ptr(), g.data_ptr(), y16.data_ptr(),
                                         rows, dim, 1e-5, s()) == 0
    assert torch.equal(y16, rounded(y32)) and torch.equal(xo16, xo32)

    f = 96
    gu = torch.from_numpy(rng.standard_normal((3, 2 * f)).astype(np.float32)).to(DEV)
    for inter in (0, 1):
        o32 = torch.empty((3, f), device=DEV)
        o16 = torch.empty((3, f), dtype=torch.bfloat16, device=DEV)
        assert lib.lhip_swiglu_f32(gu.data_ptr(), o32.data_ptr(), 3, f, inter, s()) == 0
        assert lib.lhip_swiglu_f32_bf16out(gu.data_ptr(), o16.data_ptr(), 3, f, inter, s()) == 0
        assert torch.equal(o16, rounded(o32))

    hq, hkv, hd, S, max_seq = 8, 2, 128, 37, 64
    qkv = torch.from_numpy(rng.standard_normal((S, (hq + 2 * hkv) * hd)).astype(np.float32)).to(DEV)
    kc = torch.from_numpy(rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)).to(DEV)
    vc = torch.from_numpy(rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)).to(DEV)
    pos = torch.tensor([9], dtype=torch.int32, device=DEV)
    a32 = torch.empty((S, hq * hd), device=DEV)
    a16 = torch.empty((S, hq * hd), dtype=torch.bfloat16, device=DEV)
    assert lib.lhip_attention_f32(qkv.data_ptr(), kc.data_ptr(), vc.data_ptr(), a32.data_ptr(), pos.data_ptr(), S, hq,
                                  hkv, hd, max_seq, s()) == 0
    assert lib.lhip_attention_f32_bf16out(qkv.data_ptr(), kc.data_ptr(), vc.data_ptr(), a16.data_ptr(), pos.data_ptr(),
                                          S, hq, hkv, hd, max_seq, s()) == 0
    assert torch.equal(a16, rounded(a32))
    assert lib.lhip_attention_f32_bf16out(qkv.data_ptr(), kc.data_ptr(), vc.data_ptr(), a16.data_ptr(), pos.data_ptr(),
                                          S, 6, 2, hd, max_seq, s()) == capi.LHIP_ERR_UNSUPPORTED


def test_prompt_pass_replays_from_a_graph():
    """The bf16 prompt pass allocates nothing once its buffers exist (the K-sliced GEMMs keep their partial sums in
    the library's own scratch array), so it can be captured; every replay, with eager passes and synchronisations
    in between, gives the eager logits bit for bit."""
    cfg = LlamaConfig(vocab=1000, dim=1024, layers=3, q_heads=8, kv_heads=2, ffn=2048)
    eng = LlamaQ8(cfg, random_weights(cfg, seed=4, device=DEV), max_seq=128)
    n = 16
    t = torch.as_tensor(np.random.default_rng(0).integers(0, cfg.vocab, n).astype(np.float32)).to(DEV)
    eng.reset()
    ref = eng.forward(t, n, bf16=True).clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        eng.reset()
        eng.forward(t, n, bf16=True)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eng.reset()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        out = eng.forward(t, n, bf16=True)
    for _ in range(3):
        eng.reset()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref)
        eng.reset()
        other = eng.forward(t.flip(0).contiguous(), n, bf16=True).clone()  # eager work between the replays
        torch.cuda.synchronize()
        assert not torch.equal(other, ref)


@pytest.mark.parametrize("embed_dtype", ["F32", "Q8_0"])
def test_gguf_loader_gives_the_same_model(oracle, tmp_path, embed_dtype):
    """A synthetic GGUF with the reference's tensor names, read back through the loader
    (examples/llama/src/loader.rs:99-165), must produce exactly the engine built from the same blocks; with the
    embedding table in f32 or, as quantised checkpoints hold it, in Q8_0 (then gathered by lhip_q8_0_gather_f32)."""
    from luminal_amd import gguf

    cfg = LlamaConfig(vocab=256, dim=256, layers=2, q_heads=4, kv_heads=2, ffn=512)  # head_dim 64
    rng = np.random.default_rng(5)
    hd = cfg.head_dim
    tensors = {"token_embd.weight": ("F32", (cfg.dim, cfg.vocab), rng.standard_normal((cfg.vocab, cfg.dim)).astype("<f4").tobytes()),
               "output_norm.weight": ("F32", (cfg.dim,), (1 + 0.05 * rng.standard_normal(cfg.dim)).astype("<f4").tobytes())}
    if embed_dtype == "Q8_0":
        eq, ed = synth.q8_0_random(cfg.vocab, cfg.dim, seed=499, scale_sigma=1.0)
        tensors["token_embd.weight"] = ("Q8_0", (cfg.dim, cfg.vocab), synth.q8_0_raw_blocks(eq, ed).tobytes())

    def q8(name, n, k, i):
        qs, d = synth.q8_0_random(n, k, seed=500 + i, scale_sigma=float(np.sqrt(3.0 / k) / 0.8))
        tensors[name] = ("Q8_0", (k, n), synth.q8_0_raw_blocks(qs, d).tobytes())

    q8("output.weight", cfg.vocab, cfg.dim, 0)
    for i in range(cfg.layers):
        for nm in ("attn_norm", "ffn_norm"):
            tensors[f"blk.{i}.{nm}.weight"] = ("F32", (cfg.dim,), (1 + 0.05 * rng.standard_normal(cfg.dim)).astype("<f4").tobytes())
        for j, (nm, n, k) in enumerate([("attn_q", cfg.dim, cfg.dim), ("attn_k", cfg.kv_heads * hd, cfg.dim),
                                        ("attn_v", cfg.kv_heads * hd, cfg.dim), ("attn_output", cfg.dim, cfg.dim),
                                        ("ffn_gate", cfg.ffn, cfg.dim), ("ffn_up", cfg.ffn, cfg.dim),
                                        ("ffn_down", cfg.dim, cfg.ffn)]):
            q8(f"blk.{i}.{nm}.weight", n, k, 10 * i + j + 1)
    path = tmp_path / "tiny_llama.gguf"
    gguf.write_gguf(path, {"general.architecture": "llama"}, tensors)
    eng = LlamaQ8(cfg, gguf.q8_load(path, cfg, DEV), max_seq=32)
    # oracle weights straight from the same bytes
    wf = {}
    for name, (dt, dims, data) in tensors.items():
        arr = np.frombuffer(data, dtype="<f4") if dt == "F32" else oracle.q8_0_dequant(np.frombuffer(data, np.uint8), int(np.prod(dims)))
        wf[name] = arr
    ow = {"embed": wf["token_embd.weight"].reshape(cfg.vocab, cfg.dim), "out_norm": wf["output_norm.weight"],
          "lm_head": wf["output.weight"].reshape(cfg.vocab, cfg.dim)}
    for i in range(cfg.layers):
        b = f"blk.{i}."
        ow[f"{i}.attn_norm"], ow[f"{i}.ffn_norm"] = wf[b + "attn_norm.weight"], wf[b + "ffn_norm.weight"]
        ow[f"{i}.q"] = wf[b + "attn_q.weight"].reshape(cfg.dim, cfg.dim)
        ow[f"{i}.k"] = wf[b + "attn_k.weight"].reshape(cfg.kv_heads * hd, cfg.dim)
        ow[f"{i}.v"] = wf[b + "attn_v.weight"].reshape(cfg.kv_heads * hd, cfg.dim)
        ow[f"{i}.o"] = wf[b + "attn_output.weight"].reshape(cfg.dim, cfg.dim)
        ow[f"{i}.gate"] = wf[b + "ffn_gate.weight"].reshape(cfg.ffn, cfg.dim)
        ow[f"{i}.up"] = wf[b + "ffn_up.weight"].reshape(cfg.ffn, cfg.dim)
        ow[f"{i}.down"] = wf[b + "ffn_down.weight"].reshape(cfg.dim, cfg.ffn)
    assert isinstance(eng.w["embed"], Q8Weight) == (embed_dtype == "Q8_0")
    prompt = [3, 200, 17, 5]
    kc, vc = empty_cache(cfg), empty_cache(cfg)
    want = lo.forward(cfg, ow, prompt, kc, vc, 0)
    got = eng.forward(torch.tensor(prompt, dtype=torch.float32, device=DEV), len(prompt), all_logits=True)
    assert rel_err(got.cpu().numpy(), want) < 2e-3
    gotb = eng.forward(torch.tensor(prompt, dtype=torch.float32, device=DEV), len(prompt), bf16=True, all_logits=True)
    check_bf16_stack(gotb.cpu().numpy(), want, lo.forward_prompt_bf16(cfg, ow, prompt, bf16_attention=uses_bf16_attention(cfg))[0],
                     " model read from GGUF")
    eng.prefill(prompt)
    tok = lo.argmax_last(want[-1])
    assert int(eng.tok_i.item()) == tok
    step = lo.forward(cfg, ow, [tok], kc, vc, len(prompt))[0]
    assert rel_err(eng.decode_step().cpu().numpy(), step) < 2e-3


def test_running_past_max_seq_is_refused_on_the_host(oracle):
    cfg = LlamaConfig(vocab=64, dim=128, layers=1, q_heads=2, kv_heads=1, ffn=128)
    eng, _ = build_model(oracle, cfg, seed=3, max_seq=8)
    with pytest.raises(capi.LhipError) as e:
        eng.prefill(list(range(9)))
    assert e.value.status == capi.LHIP_ERR_INVALID_SHAPE
    eng.prefill([1, 2, 3, 4, 5, 6])
    eng.decode_step()
    eng.decode_step()  # position 8 = max_seq reached
    with pytest.raises(capi.LhipError):
        eng.decode_step()
    with pytest.raises(capi.LhipError):
        eng.decode(1, use_graph=False)
    eng.reset()
    eng.prefill([1, 2, 3])
    with pytest.raises(capi.LhipError):
        eng.decode(6, use_graph=False)
    assert eng.decode(5, use_graph=False).numel() == 5


def test_decode_of_the_last_free_position(oracle):
    """A decode of exactly the last free cache position fits and is not refused: capturing the graph needs two free
    positions (its warm-up and captured steps write real K/V rows), so with fewer the steps run eagerly; one step
    more is refused on the host."""
    cfg = LlamaConfig(vocab=512, dim=1024, layers=2, q_heads=8, kv_heads=2, ffn=1024)
    eng, _ = build_model(oracle, cfg, seed=9, max_seq=6)
    eng.prefill([1, 2, 3, 4, 5])
    toks = eng.decode(1, use_graph=True).cpu().numpy()
    assert toks.shape == (1,) and eng._pos_host == 6 and int(eng.pos.item()) == 6
    with pytest.raises(capi.LhipError):
        eng.decode(1, use_graph=True)
    # the same tokens as a roomier engine picks
    eng2, _ = build_model(oracle, cfg, seed=9, max_seq=32)
    eng2.prefill([1, 2, 3, 4, 5])
    assert np.array_equal(eng2.decode(1, use_graph=True).cpu().numpy(), toks)


def test_argmax_with_the_callers_workspace():
    """lhip_argmax_f32_ws: the same pick as lhip_argmax_f32 with the partial picks in the caller's 512 bytes."""
    lib = capi.load_library()
    torch.manual_seed(3)
    x = torch.randn(128256, device=DEV)
    x[77777] = x.max() + 1.0
    x[99999] = x[77777]  # an exact tie: the last index wins
    ws = torch.zeros(512, dtype=torch.uint8, device=DEV)
    outs = []
    for use_ws in (False, True):
        f, i, pos = torch.zeros(1, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV), torch.zeros(1, dtype=torch.int32, device=DEV)
        if use_ws:
            capi.check(lib.lhip_argmax_f32_ws(x.data_ptr(), x.numel(), f.data_ptr(), i.data_ptr(), pos.data_ptr(), 2, ws.data_ptr(), s()), "ws")
        else:
            capi.check(lib.lhip_argmax_f32(x.data_ptr(), x.numel(), f.data_ptr(), i.data_ptr(), pos.data_ptr(), 2, s()), "plain")
        torch.cuda.synchronize()
        outs.append((float(f.item()), int(i.item()), int(pos.item())))
    assert outs[0] == outs[1] == (99999.0, 99999, 2)
    assert lib.lhip_argmax_f32_ws(x.data_ptr(), x.numel(), None, None, None, 0, ws.data_ptr(), s()) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_argmax_f32_ws(x.data_ptr(), x.numel(), ws.data_ptr(), None, None, 0, None, s()) == capi.LHIP_ERR_NULL_PTR


@pytest.mark.parametrize("hq,hkv,hd", [(32, 8, 128), (16, 2, 128), (32, 32, 64), (16, 8, 128)])
def test_output_projection_that_merges_the_key_ranges_itself(hq, hkv, hd):
    """lhip_attention_decode_partial_f32 + lhip_q8_0_matvec_attn_merge_f32 against lhip_attention_decode_few_ranges_f32
    followed by the fused matvec with the residual: the same bits, at positions that give one key range, a ragged last
    range, eight ranges and (beyond 2048 keys) sixteen; the caches are appended to alike.  The few-range attention
    itself against the many-range one: the operator's tolerance (other partial sums)."""
    lib = capi.load_library()
    dim = hq * hd
    max_seq = 2600
    rng = np.random.default_rng(hq + hkv)
    qs, d = synth.q8_0_random(dim, dim, seed=hq * hd, scale_sigma=float(np.sqrt(3.0 / dim) / 0.8))
    w = Q8Weight.from_raw(synth.q8_0_raw_blocks(qs, d), dim, dim, DEV)
    ws_n = lib.lhip_attention_decode_workspace_nbytes(hq, hkv, hd)
    assert ws_n > 0
    kc0 = torch.from_numpy(rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)).to(DEV)
    vc0 = torch.from_numpy(rng.standard_normal((hkv, max_seq, hd)).astype(np.float32)).to(DEV)
    for p in (0, 5, 63, 64, 200, 511, 700, 2047, 2048, 2599):
        qkv = torch.from_numpy(rng.standard_normal((hq + 2 * hkv) * hd).astype(np.float32)).to(DEV)
        res = torch.from_numpy(rng.standard_normal(dim).astype(np.float32)).to(DEV)
        pos = torch.tensor([p], dtype=torch.int32, device=DEV)
        # reference: attention with its merge launch, then y = res + W att
        kc, vc = kc0.clone(), vc0.clone()
        ws = torch.zeros(ws_n, dtype=torch.uint8, device=DEV)
        att = torch.empty(dim, device=DEV)
        capi.check(lib.lhip_attention_decode_few_ranges_f32(qkv.data_ptr(), kc.data_ptr(), vc.data_ptr(), att.data_ptr(),
                                                            pos.data_ptr(), hq, hkv, hd, max_seq, 500000.0, ws.data_ptr(),
                                                            s()), "decode, few ranges")
        kc3, vc3, att3 = kc0.clone(), vc0.clone(), torch.empty(dim, device=DEV)
        capi.check(lib.lhip_attention_decode_f32(qkv.data_ptr(), kc3.data_ptr(), vc3.data_ptr(), att3.data_ptr(),
                                                 pos.data_ptr(), hq, hkv, hd, max_seq, 500000.0, ws.data_ptr(), s()), "decode")
        torch.cuda.synchronize()
        assert rel_err(att.cpu().numpy(), att3.cpu().numpy().astype(np.float64)) < 2e-3, p  # two f32 paths, other partial sums
        assert torch.equal(kc3, kc) and torch.equal(vc3, vc), p
        y_ref = res.clone()
        from luminal_amd.quantized import FusedMatvec
        FusedMatvec([w], [y_ref], residual=y_ref, epilogue=FusedMatvec.EPI_ADD).run(att)
        # the folded form
        kc2, vc2 = kc0.clone(), vc0.clone()
        ws2 = torch.full((ws_n,), 0xFF, dtype=torch.uint8, device=DEV)  # stale contents: NaN patterns
        capi.check(lib.lhip_attention_decode_partial_f32(qkv.data_ptr(), kc2.data_ptr(), vc2.data_ptr(), pos.data_ptr(), hq,
                                                         hkv, hd, max_seq, 500000.0, ws2.data_ptr(), s()), "partial")
        y = res.clone()
        capi.check(lib.lhip_q8_0_matvec_attn_merge_f32(w.planar.data_ptr(), y.data_ptr(), dim, dim, ws2.data_ptr(),
                                                       pos.data_ptr(), hq, hkv, hd, max_seq, y.data_ptr(), s()), "merge")
        y_plain = torch.empty(dim, device=DEV)
        capi.check(lib.lhip_q8_0_matvec_attn_merge_f32(w.planar.data_ptr(), y_plain.data_ptr(), dim, dim, ws2.data_ptr(),
                                                       pos.data_ptr(), hq, hkv, hd, max_seq, None, s()), "merge, no residual")
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int32), y_ref.view(torch.int32)), p
        assert torch.equal((y_plain + res).view(torch.int32), y_ref.view(torch.int32)) or torch.allclose(y_plain + res, y_ref), p
        assert torch.equal(kc2, kc) and torch.equal(vc2, vc), p
    p8 = w.planar.data_ptr()
    assert lib.lhip_q8_0_matvec_attn_merge_f32(p8, y.data_ptr(), dim, dim, None, pos.data_ptr(), hq, hkv, hd, max_seq, None, s()) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_q8_0_matvec_attn_merge_f32(p8, y.data_ptr(), dim, dim, ws2.data_ptr(), pos.data_ptr(), hq, hkv, hd + 64, max_seq, None, s()) == capi.LHIP_ERR_INVALID_SHAPE


def test_engine_with_the_merge_inside_the_output_projection(oracle):
    """LlamaQ8.merge_in_o_proj: decode steps through lhip_attention_decode_partial_f32 and
    lhip_q8_0_matvec_attn_merge_f32 against the oracle, and graph replay against eager stepping."""
    cfg = LlamaConfig(vocab=1000, dim=2048, layers=2, q_heads=16, kv_heads=4, ffn=2048)
    eng, wf = build_model(oracle, cfg, seed=77, max_seq=128)
    eng.merge_in_o_proj = True
    assert eng.fused_decode and eng._can_merge_in_o_proj
    prompt = [int(t) for t in np.random.default_rng(2).integers(0, cfg.vocab, 70)]
    kc, vc = empty_cache(cfg), empty_cache(cfg)
    want = lo.forward(cfg, wf, prompt, kc, vc, 0)
    eng.prefill(prompt)
    tok = lo.argmax_last(want[-1])
    assert int(eng.tok_i.item()) == tok
    for step in range(4):
        want_step = lo.forward(cfg, wf, [tok], kc, vc, len(prompt) + step)[0]
        logits = eng.decode_step()
        assert rel_err(logits.cpu().numpy(), want_step) < 2e-3, step
        tok = lo.argmax_last(want_step)
        eng.tok.fill_(float(tok))
        eng.tok_i.fill_(tok)
    eng.reset()
    eng.prefill(prompt)
    eager = eng.decode(6, use_graph=False).cpu().numpy()
    eng.reset()
    eng.prefill(prompt)
    assert np.array_equal(eng.decode(6, use_graph=True).cpu().numpy(), eager)
