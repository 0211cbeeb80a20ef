"""Pins the CPU oracle: against the reference's literal test operands, against
IEEE/numpy for the format conversions, and against closed forms."""
import json
import os

import numpy as np
import pytest

from luminal_amd import synth

HERE = os.path.dirname(os.path.abspath(__file__))


def test_f16_to_f32_exhaustive(oracle):
    codes = np.arange(65536, dtype=np.uint16)
    want = codes.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(c)) for c in codes], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_matches_numpy(oracle):
    rng = np.random.default_rng(1)
    xs = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-9, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 65504.0, 65519.9, 65520.0, 1e-8, 2.0 ** -25, 2.0 ** -24, 3 * 2.0 ** -25,
                  6.1e-5, 6.0975e-5, np.inf, -np.inf, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11], np.float32),
        # every f16 value and every midpoint between neighbours (ties)
        np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32),
        ((np.arange(0, 0x7bff, dtype=np.uint16).view(np.float16).astype(np.float64)
          + np.arange(1, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)) / 2).astype(np.float32),
    ])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(float(x)) for x in xs], np.uint16)
    assert np.array_equal(got, want)


def test_bf16_round_trip(oracle):
    rng = np.random.default_rng(2)
    x = rng.standard_normal(4096).astype(np.float32)
    bits = oracle.f32_to_bf16_bits(x)
    c = np.array([oracle.lib().lo_f32_to_bf16(float(v)) for v in x], np.uint16)
    assert np.array_equal(bits, c)
    back = oracle.bf16_bits_to_f32(bits)
    assert np.max(np.abs(back - x) / np.abs(x)) <= 2.0 ** -8
    # exact for bf16-representable values
    assert np.array_equal(oracle.f32_to_bf16_bits(back), bits)


def test_q8_0_size_law(oracle):
    # n + n/16 bytes (examples/llama/src/loader.rs:128)
    assert oracle.q8_0_nbytes(32) == 34
    assert oracle.q8_0_nbytes(4096 * 4096) == 17825792
    assert oracle.q8_0_nbytes(128256 * 4096) == 558170112


def test_q8_0_pack_layout_and_dequant_closed_form(oracle):
    qs, d = synth.q8_0_random(8, 96, seed=3)
    raw = oracle.q8_0_pack(qs, d.view(np.uint16))
    # layout: little-endian f16 first, then 32 int8
    blk = raw.reshape(-1, 34)
    assert np.array_equal(blk[:, :2].copy().view("<f2").reshape(-1), d.reshape(-1))
    assert np.array_equal(blk[:, 2:].view(np.int8).reshape(8, 96), qs)
    # numpy packer used by the benchmark agrees with the C one
    assert np.array_equal(synth.q8_0_raw_blocks(qs, d), raw)
    w = oracle.q8_0_dequant(raw, qs.size).reshape(8, 96)
    want = qs.astype(np.float32) * np.repeat(d.astype(np.float32), 32, axis=1)
    assert np.array_equal(w.view(np.uint32), want.view(np.uint32))
    # exactness: the f32 product equals the f64 product
    want64 = qs.astype(np.float64) * np.repeat(d.astype(np.float64), 32, axis=1)
    assert np.array_equal(w.astype(np.float64), want64)


def test_q8_0_dequant_all_quant_values_subnormal_scales(oracle):
    qs = np.tile(np.arange(-128, 128, dtype=np.int8), 4).reshape(4, 256)
    d = np.array([[2.0 ** -24] * 8, [6e-5] * 8, [1.0] * 8, [65504.0] * 8], np.float16)
    raw = oracle.q8_0_pack(qs, d.view(np.uint16))
    w = oracle.q8_0_dequant(raw, qs.size).reshape(4, 256)
    want = qs.astype(np.float64) * np.repeat(d.astype(np.float64), 32, axis=1)
    assert np.array_equal(w.astype(np.float64), want)


def test_matmul_reference_literals(oracle):
    with open(os.path.join(HERE, "golden", "reference_matmul_literals.json")) as f:
        cases = json.load(f)["cases"]
    for c in cases:
        a = np.array(c["a"], np.float32).reshape(c["a_shape"])
        b = np.array(c["b"], np.float32).reshape(c["b_shape"])
        want = np.array(c["c"], np.float32).reshape(a.shape[0], b.shape[1])
        w = np.ascontiguousarray(b.T)  # the oracle takes W = (N, K)
        for fn in (oracle.matmul_seq_f32, oracle.matmul_f64, oracle.matmul_fast_f32):
            got = fn(a, w)
            assert np.array_equal(got.astype(np.float64), want.astype(np.float64)), c["source"]


def test_matmul_reference_sweep_vs_numpy(oracle):
    # the reference's dynamic-shape sweep (crates/luminal_cpu/src/lib.rs:145-175),
    # U(-0.5, 0.5) operands (src/tests/mod.rs:117-119), tolerance 1e-2 there
    for m in range(1, 23, 4):
        for k in range(1, 35, 3):
            for n in range(1, 70, 7):
                rng = np.random.default_rng(0)
                a = rng.uniform(-0.5, 0.5, (m, k)).astype(np.float32)
                b = rng.uniform(-0.5, 0.5, (k, n)).astype(np.float32)
                want = a.astype(np.float64) @ b.astype(np.float64)
                w = np.ascontiguousarray(b.T)
                assert np.max(np.abs(oracle.matmul_seq_f32(a, w) - want)) < 1e-5
                assert np.max(np.abs(oracle.matmul_f64(a, w) - want)) < 1e-12
                assert np.max(np.abs(oracle.matmul_fast_f32(a, w) - want)) < 1e-5


def test_matmul_seq_is_sequential_unfused(oracle):
    # A case where order and fusing matter: 1e8 + 1 - 1e8 in f32 = 0 when added
    # left to right; and a product that an FMA would keep exact.
    a = np.array([[1e8, 1.0, -1e8]], np.float32)
    w = np.ones((1, 3), np.float32)
    assert oracle.matmul_seq_f32(a, w)[0, 0] == 0.0
    assert oracle.matmul_f64(a, w)[0, 0] == 1.0
    x = np.float32(1.0 + 2.0 ** -12)
    a = np.array([[x, -1.0]], np.float32)
    w = np.array([[x, np.float32(x * x)]], np.float32)  # x*x rounded - round(x*x) = 0 unfused
    assert oracle.matmul_seq_f32(a, w)[0, 0] == 0.0


def test_matmul_metal_quantized_test_shape(oracle):
    # crates/luminal_metal/src/quantized.rs:888-935: W 512x1024 ints in 0..5, d = 1.0,
    # x in U(-0.5, 0.5); quantized result vs f32 graph within 1e-3 absolute.
    rng = np.random.default_rng(4)
    qs = rng.integers(0, 5, (512, 1024), dtype=np.int8)
    d = np.ones((512, 32), np.float16)
    x = rng.uniform(-0.5, 0.5, (1, 1024)).astype(np.float32)
    w = oracle.q8_0_dequant(oracle.q8_0_pack(qs, d.view(np.uint16)), qs.size).reshape(512, 1024)
    assert np.array_equal(w, qs.astype(np.float32))
    y = oracle.matmul_seq_f32(x, w)
    assert np.max(np.abs(y - x.astype(np.float64) @ qs.T.astype(np.float64))) < 1e-3


def test_q8_0_gather_equals_dequant_rows(oracle):
    qs, d = synth.q8_0_random(50, 64, seed=5)
    raw = oracle.q8_0_pack(qs, d.view(np.uint16))
    w = oracle.q8_0_dequant(raw, qs.size).reshape(50, 64)
    idx = np.array([0, 49, 7, 7, 13.9], np.float32)  # f32 indices truncate
    got = oracle.q8_0_gather(raw, idx, 64)
    assert np.array_equal(got, w[[0, 49, 7, 7, 13]])


def test_mxfp4_value_table_and_scale(oracle):
    # OCP MX e2m1 magnitudes {0,.5,1,1.5,2,3,4,6}; low nibble = even element.
    blk = np.zeros(17, np.uint8)
    blk[:8] = [(2 * i + 1) << 4 | (2 * i) for i in range(8)]
    blk[8:16] = 0
    blk[16] = 127
    w = oracle.mxfp4_dequant(blk, 32)
    assert list(w[:16]) == [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]
    assert np.signbit(w[8])
    for e in (0, 1, 119, 127, 128, 254):
        blk[16] = e
        w2 = oracle.mxfp4_dequant(blk, 32)
        with np.errstate(over="ignore"):  # 4 * 2^127 and 6 * 2^127 overflow f32 to inf
            want = (w.astype(np.float64) * 2.0 ** (e - 127)).astype(np.float32)
        assert np.array_equal(w2, want)
    blk[16] = 255
    assert np.all(np.isnan(oracle.mxfp4_dequant(blk, 32)))


def test_moe_route_top4_softmax(oracle):
    rng = np.random.default_rng(6)
    logits = rng.standard_normal((16, 32)).astype(np.float32)
    sel, wts = oracle.moe_route(logits, 4)
    order = np.argsort(-logits, axis=1, kind="stable")[:, :4]
    assert np.array_equal(sel, order)
    picked = np.take_along_axis(logits.astype(np.float64), order, axis=1)
    e = np.exp(picked - picked.max(axis=1, keepdims=True))
    assert np.allclose(wts, e / e.sum(axis=1, keepdims=True), rtol=1e-6, atol=0)
    assert np.allclose(wts.sum(axis=1), 1.0, atol=1e-6)


def test_moe_forward_vs_numpy(oracle):
    rng = np.random.default_rng(7)
    T, H, I, E, topk = 3, 64, 32, 4, 2
    x = rng.standard_normal((T, H)).astype(np.float32)
    w_gu = rng.standard_normal((E, 2 * I, H)).astype(np.float32) * 0.1
    w_dn = rng.standard_normal((E, H, I)).astype(np.float32) * 0.1
    sel, wts = oracle.moe_route(rng.standard_normal((T, E)).astype(np.float32), topk)
    got = oracle.moe_forward(x, w_gu, w_dn, sel, wts, act_bf16=False)
    want = np.zeros((T, H))
    for t in range(T):
        for s in range(topk):
            e = sel[t, s]
            g = w_gu[e, :I].astype(np.float64) @ x[t]
            u = w_gu[e, I:].astype(np.float64) @ x[t]
            act = u * (g / (1 + np.exp(-g)))
            want[t] += wts[t, s] * (w_dn[e].astype(np.float64) @ act)
    assert np.max(np.abs(got - want)) < 1e-5
