"""The f32 / f16 quantized matmul for several activation rows on the matrix cores
(lhip_q8_0_matmul_f32_gemm, lhip_q8_0_matmul_f16_gemm), through the C ABI.

The reference's operator (QuantizedMatmul<T>::process, crates/luminal_cuda/src/quantized.rs:116-168) runs one
matvec per activation row; this form streams the weights once per 64 rows: the codes enter the matrix cores as
exact bf16, x as three bf16 limbs whose sum is the f32 value (an f16 x: two), and each block's f32 sum is scaled as in the matvec
kernels.  Bars: the operator's own (conftest.rel_err < 2e-3: every element, with a floor of 1e-3 rms) and
max |y - t| / rms(t) < 5e-6 against the f64 product (measured 1e-6, like the matvec kernels; two limbs of x and of
q * d give 2e-5, bf16 operands alone 5e-3); integer cases exact; a one-hot row returns the weight column bit for
bit; the f16 form is bit-equal to the f32 form on the widened inputs rounded once.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from conftest import rel_err  # noqa: E402
from luminal_amd import capi, synth  # noqa: E402
from luminal_amd.quantized import Q8Weight, QuantizedMatmul  # noqa: E402

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
BAR = 5e-6


def upload(qs, d):
    n, k = qs.shape
    return Q8Weight.from_raw(synth.q8_0_raw_blocks(qs, d), n, k, DEV)


def stream():
    return torch.cuda.current_stream().cuda_stream


def gemm_f32(w, x):
    lib = capi.load_library()
    xd = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(DEV)
    y = torch.full((x.shape[0], w.n), float("nan"), device=DEV)
    capi.check(lib.lhip_q8_0_matmul_f32_gemm(w.planar.data_ptr(), xd.data_ptr(), y.data_ptr(), x.shape[0], w.n, w.k,
                                             stream()), "lhip_q8_0_matmul_f32_gemm")
    torch.cuda.synchronize()
    return y.cpu().numpy()


def gemm_f16(w, x16):
    lib = capi.load_library()
    xd = torch.from_numpy(np.ascontiguousarray(x16)).to(DEV)
    y = torch.zeros((x16.shape[0], w.n), device=DEV, dtype=torch.float16)
    capi.check(lib.lhip_q8_0_matmul_f16_gemm(w.planar.data_ptr(), xd.data_ptr(), y.data_ptr(), x16.shape[0], w.n, w.k,
                                             stream()), "lhip_q8_0_matmul_f16_gemm")
    torch.cuda.synchronize()
    return y.cpu().numpy()


def rms_err(y, t):
    return float(np.max(np.abs(y - t)) / np.sqrt(np.mean(t * t)))


@pytest.mark.parametrize("m,n,k", [(1, 128, 512), (4, 128, 512), (12, 256, 512), (16, 512, 1024), (33, 260, 1024),
                                   (64, 4, 1536), (100, 1024, 4096), (128, 512, 14336), (129, 1024, 512),
                                   (300, 132, 1536)])
def test_rows_gemm_vs_oracle(oracle, m, n, k):
    """Every activation-row bracket, ragged strips, K slices, and more than 64 rows (several passes)."""
    qs, d = synth.q8_0_random(n, k, seed=m + n + k)
    x = synth.activations(m, k, seed=m * n + 3)
    w = upload(qs, d)
    wf = oracle.q8_0_dequant(synth.q8_0_raw_blocks(qs, d), qs.size).reshape(qs.shape)
    y = gemm_f32(w, x)
    truth = oracle.matmul_f64(x, wf)
    assert y.shape == (m, n) and rms_err(y.astype(np.float64), truth) < BAR and rel_err(y, truth) < 2e-3
    # f16 in / out: the f32 form on the widened inputs, rounded once
    x16 = x.astype(np.float16)
    y16 = gemm_f16(w, x16)
    y32 = gemm_f32(w, x16.astype(np.float32))
    assert np.array_equal(y16.view(np.uint16), y32.astype(np.float16).view(np.uint16))
    assert rel_err(y16.astype(np.float32), oracle.matmul_f64(x16.astype(np.float32), wf)) < 2e-3


def test_rows_gemm_integer_exact_and_wide_dynamic_range(oracle):
    """Small integers with power-of-two scales: every product and partial sum is exact.  Then activations whose
    magnitudes span twelve binades in one row: the limbs are taken per element, so the bar holds."""
    rng = np.random.default_rng(5)
    m, n, k = 70, 152, 2048
    qi = rng.integers(-8, 9, (n, k), dtype=np.int8)
    di = (2.0 ** rng.integers(-2, 2, (n, k // 32))).astype(np.float16)
    x = rng.integers(-4, 5, (m, k)).astype(np.float32)
    want = x.astype(np.float64) @ (qi.astype(np.float64) * np.repeat(di.astype(np.float64), 32, axis=1)).T
    assert np.array_equal(gemm_f32(upload(qi, di), x).astype(np.float64), want)
    qs, d = synth.q8_0_random(256, 1024, seed=9)
    xw = (rng.standard_normal((40, 1024)) * 2.0 ** rng.integers(-6, 7, (40, 1024))).astype(np.float32)
    wf = oracle.q8_0_dequant(synth.q8_0_raw_blocks(qs, d), qs.size).reshape(qs.shape)
    assert rms_err(gemm_f32(upload(qs, d), xw).astype(np.float64), oracle.matmul_f64(xw, wf)) < BAR


def test_rows_gemm_full_size_one_hot(oracle):
    """gate (14336 x 4096) at 128 rows (two passes): zero rows give zero, a one-hot row gives the weight column
    exactly (one exact product, one exact scaling)."""
    n, k = synth.LLAMA3_8B_PROJ["gate"]
    qs, d = synth.q8_0_random(n, k, seed=77)
    w = upload(qs, d)
    e = np.zeros((128, k), np.float32)
    e[64, 1234] = 1.0
    e[127, 4095] = -2.0
    y = gemm_f32(w, e)
    col = lambda j: qs[:, j].astype(np.float64) * d[:, j // 32].astype(np.float64)  # noqa: E731
    assert np.array_equal(y[64].astype(np.float64), col(1234))
    assert np.array_equal(y[127].astype(np.float64), -2.0 * col(4095))
    rest = np.ones(128, bool)
    rest[[64, 127]] = False
    assert not y[rest].any()


def test_plain_operator_takes_the_matrix_core_form(oracle):
    """lhip_q8_0_matmul_f32 / _f16 (and so QuantizedMatmul.process): from six rows on (small matrices; large ones earlier) the matrix-core form where
    the shape allows it, the matvec form below that, for other shapes, and whenever a launch shape is given."""
    lib = capi.load_library()
    qs, d = synth.q8_0_random(512, 1024, seed=21)
    w = upload(qs, d)
    x = synth.activations(16, 1024, seed=22)
    xd = torch.from_numpy(x).to(DEV)
    y = QuantizedMatmul().process(xd, w).cpu().numpy()
    assert np.array_equal(y, gemm_f32(w, x))
    ymv = QuantizedMatmul(1, 1, 0, 4).process(xd, w).cpu().numpy()  # a launch shape: one matvec per row group
    assert not np.array_equal(y, ymv) and rel_err(ymv, y) < 1e-3   # another order of additions, the same product
    y5 = torch.empty(5, 512, device=DEV)  # under six rows: the matvec form, another order of additions
    capi.check(lib.lhip_q8_0_matmul_f32(w.planar.data_ptr(), xd.data_ptr(), y5.data_ptr(), 5, 512, 1024, stream()), "mv")
    assert not np.array_equal(y5.cpu().numpy(), y[:5]) and rel_err(y5.cpu().numpy(), y[:5]) < 1e-3
    assert np.array_equal(QuantizedMatmul().process(xd.reshape(2, 8, 1024), w).cpu().numpy().reshape(16, 512), y)
    x16 = x.astype(np.float16)
    y16 = QuantizedMatmul().process(torch.from_numpy(x16).to(DEV), w).cpu().numpy()
    assert np.array_equal(y16.view(np.uint16), gemm_f16(w, x16).view(np.uint16))
    # K not a multiple of 512: not covered, the plain operator keeps the matvec form
    q2, d2 = synth.q8_0_random(64, 96, seed=2)
    w2 = upload(q2, d2)
    x2 = torch.from_numpy(synth.activations(8, 96, seed=4)).to(DEV)
    y2 = torch.empty(8, 64, device=DEV)
    assert lib.lhip_q8_0_matmul_f32_gemm(w2.planar.data_ptr(), x2.data_ptr(), y2.data_ptr(), 8, 64, 96,
                                         stream()) == capi.LHIP_ERR_UNSUPPORTED
    wf2 = oracle.q8_0_dequant(synth.q8_0_raw_blocks(q2, d2), q2.size).reshape(q2.shape)
    assert rel_err(QuantizedMatmul().process(x2, w2).cpu().numpy(), oracle.matmul_f64(x2.cpu().numpy(), wf2)) < 2e-3


def test_large_matrices_take_the_matrix_core_form_earlier(oracle):
    """4096 x 4096 (2^24 codes): the plain operator is the matvec form at three rows and the matrix-core form at
    four (bit-equal to the _gemm entry), both within the operator's bar."""
    lib = capi.load_library()
    n = k = 4096
    qs, d = synth.q8_0_random(n, k, seed=31)
    w = upload(qs, d)
    wf = oracle.q8_0_dequant(synth.q8_0_raw_blocks(qs, d), qs.size).reshape(qs.shape)
    for m, same in ((3, False), (4, True)):
        x = synth.activations(m, k, seed=40 + m)
        xd = torch.from_numpy(x).to(DEV)
        y = torch.empty(m, n, device=DEV)
        capi.check(lib.lhip_q8_0_matmul_f32(w.planar.data_ptr(), xd.data_ptr(), y.data_ptr(), m, n, k, stream()), "plain")
        y = y.cpu().numpy()
        assert np.array_equal(y, gemm_f32(w, x)) == same
        assert rel_err(y, oracle.matmul_f64(x, wf)) < 2e-3


def test_rows_gemm_argument_errors():
    lib = capi.load_library()
    w = upload(*synth.q8_0_random(64, 512, seed=1))
    x = torch.zeros((8, 512), device=DEV)
    y = torch.zeros((8, 64), device=DEV)
    xh, yh = x.half(), y.half()
    s = stream()
    f32, f16 = lib.lhip_q8_0_matmul_f32_gemm, lib.lhip_q8_0_matmul_f16_gemm
    assert f32(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 8, 64, 512, s) == capi.LHIP_OK
    assert f16(w.planar.data_ptr(), xh.data_ptr(), yh.data_ptr(), 8, 64, 512, s) == capi.LHIP_OK
    assert f32(None, x.data_ptr(), y.data_ptr(), 8, 64, 512, s) == capi.LHIP_ERR_NULL_PTR
    assert f16(w.planar.data_ptr(), None, yh.data_ptr(), 8, 64, 512, s) == capi.LHIP_ERR_NULL_PTR
    assert f32(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 0, 64, 512, s) == capi.LHIP_ERR_INVALID_SHAPE
    assert f32(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 8, 64, 500, s) == capi.LHIP_ERR_INVALID_SHAPE
    assert f32(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 8, 62, 512, s) == capi.LHIP_ERR_UNSUPPORTED
    assert f32(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 8, 64, 1024 + 32, s) == capi.LHIP_ERR_UNSUPPORTED
    assert f16(w.planar.data_ptr(), xh.data_ptr() + 8, yh.data_ptr(), 7, 64, 512, s) == capi.LHIP_ERR_UNSUPPORTED
    assert f16(w.planar.data_ptr(), xh.data_ptr() + 2, yh.data_ptr(), 7, 64, 512, s) == capi.LHIP_ERR_MISALIGNED
    torch.cuda.synchronize()


@pytest.mark.parametrize("m,n,k", [(4, 4096, 4096), (6, 1024, 1024), (16, 1024, 4096), (64, 2048, 2048), (200, 512, 1536)])
def test_workspace_forms_give_the_plain_calls_bits_and_overlap_safely(oracle, m, n, k):
    """lhip_q8_0_matmul_f32_ws / _f16_ws keep K-slice partial sums in the caller's workspace: with the recommended
    size the plan and the bits are those of the plain call; without a workspace K is not sliced (operator's bar
    still holds); two streams with workspaces of their own run interleaved and each gets its own result."""
    lib = capi.load_library()
    qs, d = synth.q8_0_random(n, k, seed=7 * m + n + k)
    w = upload(qs, d)
    wf = oracle.q8_0_dequant(synth.q8_0_raw_blocks(qs, d), qs.size).reshape(qs.shape)
    xs = [torch.from_numpy(synth.activations(m, k, seed=s)).to(DEV) for s in (1, 2)]
    nbytes = lib.lhip_q8_0_matmul_workspace_nbytes(m, n, k)
    assert nbytes % 4 == 0 and nbytes <= 32 << 20
    plain = []
    for x in xs:
        y = torch.empty((m, n), device=DEV)
        capi.check(lib.lhip_q8_0_matmul_f32(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), m, n, k, stream()), "plain")
        plain.append(y)
    torch.cuda.synchronize()
    spaces = [torch.empty(max(nbytes, 256), dtype=torch.uint8, device=DEV) for _ in xs]
    y_ws = torch.empty((m, n), device=DEV)
    capi.check(lib.lhip_q8_0_matmul_f32_ws(w.planar.data_ptr(), xs[0].data_ptr(), y_ws.data_ptr(), m, n, k,
                                           spaces[0].data_ptr() if nbytes else None, nbytes, stream()), "ws")
    y_none = torch.empty((m, n), device=DEV)
    capi.check(lib.lhip_q8_0_matmul_f32_ws(w.planar.data_ptr(), xs[0].data_ptr(), y_none.data_ptr(), m, n, k, None, 0,
                                           stream()), "ws none")
    torch.cuda.synchronize()
    assert torch.equal(y_ws.view(torch.int32), plain[0].view(torch.int32))
    truth = oracle.matmul_f64(xs[0].cpu().numpy(), wf)
    assert rel_err(y_none.cpu().numpy(), truth) < 2e-3 and rms_err(y_none.cpu().numpy().astype(np.float64), truth) < BAR
    # f16 form: same plan, bits of the plain f16 call
    x16 = xs[0].to(torch.float16)
    y16_plain = torch.empty((m, n), device=DEV, dtype=torch.float16)
    y16_ws = torch.empty_like(y16_plain)
    capi.check(lib.lhip_q8_0_matmul_f16(w.planar.data_ptr(), x16.data_ptr(), y16_plain.data_ptr(), m, n, k, stream()), "f16")
    capi.check(lib.lhip_q8_0_matmul_f16_ws(w.planar.data_ptr(), x16.data_ptr(), y16_ws.data_ptr(), m, n, k,
                                           spaces[0].data_ptr() if nbytes else None, nbytes, stream()), "f16 ws")
    torch.cuda.synchronize()
    assert torch.equal(y16_ws.view(torch.int16), y16_plain.view(torch.int16))
    # two streams, a workspace each, launches interleaved
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [torch.empty((m, n), device=DEV) for _ in xs]
    for _ in range(20):
        for i, s in enumerate(streams):
            capi.check(lib.lhip_q8_0_matmul_f32_ws(w.planar.data_ptr(), xs[i].data_ptr(), outs[i].data_ptr(), m, n, k,
                                                   spaces[i].data_ptr() if nbytes else None, nbytes, s.cuda_stream), "ws 2")
    torch.cuda.synchronize()
    for i in range(2):
        assert torch.equal(outs[i].view(torch.int32), plain[i].view(torch.int32))


def test_workspace_form_argument_checks():
    lib = capi.load_library()
    w = upload(*synth.q8_0_random(1024, 1024, seed=3))
    x = torch.zeros((8, 1024), device=DEV)
    y = torch.empty((8, 1024), device=DEV)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=DEV)
    assert lib.lhip_q8_0_matmul_workspace_nbytes(1, 1024, 1024) == 0       # a matvec needs none
    assert lib.lhip_q8_0_matmul_workspace_nbytes(8, 1024, 1000) == 0       # invalid shape
    assert lib.lhip_q8_0_matmul_workspace_nbytes(8, 1024, 1024) > 0
    assert lib.lhip_q8_0_matmul_f32_ws(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 8, 1024, 1024, ws.data_ptr() + 64,
                                       1 << 19, stream()) == capi.LHIP_ERR_MISALIGNED
    assert lib.lhip_q8_0_matmul_f32_ws(None, x.data_ptr(), y.data_ptr(), 8, 1024, 1024, ws.data_ptr(), 1 << 20,
                                       stream()) == capi.LHIP_ERR_NULL_PTR
    # one row goes to the matvec kernels, workspace or not
    capi.check(lib.lhip_q8_0_matmul_f32_ws(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 1, 1024, 1024, None, 0,
                                           stream()), "one row")
    torch.cuda.synchronize()
