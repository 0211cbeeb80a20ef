"""Parity of the Q8_0 prefill GEMM (bf16 activations, f32 accumulate on MFMA,
bf16 out) with the CPU oracle, through the C ABI.

Bar: max |y - t| / max(|t|, 1e-3 rms(t)) (conftest.rel_err, the metric of the f32
operators) <= 1e-2 for the bf16 output and <= 2e-3 for the f32 output, against the
f64 truth computed from the same bf16 activations and the exactly dequantised
weights.  The kernels keep the weights exact (codes on the matrix cores, block
scales applied in f32), so the bf16 figure is the rounding of the store alone.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from conftest import rel_err  # noqa: E402
from luminal_amd import capi, synth  # noqa: E402
from luminal_amd.quantized import Q8Weight, QuantizedMatmulBf16  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = 1e-2      # bf16 output
TOL_F32 = 2e-3  # f32 output


def bf16_err(y, truth):
    """(element-wise error with the 1e-3 rms floor, norm-wise error)"""
    y = np.asarray(y, np.float64)
    t = np.asarray(truth, np.float64)
    return rel_err(y, t), float(np.linalg.norm(y - t) / (np.linalg.norm(t) + 1e-300))


def upload(qs, d):
    n, k = qs.shape
    return Q8Weight.from_raw(synth.q8_0_raw_blocks(qs, d), n, k, DEV)


def bf16_activations(oracle, m, k, seed):
    x = synth.activations(m, k, seed)
    bits = oracle.f32_to_bf16_bits(x)
    return oracle.bf16_bits_to_f32(bits), bits


def run(w, bits, tile=None):
    x = torch.from_numpy(bits.view(np.int16)).to(DEV).view(torch.bfloat16)
    y = QuantizedMatmulBf16(tile).process(x, w)
    torch.cuda.synchronize()
    return y.float().cpu().numpy()


def truth_for(oracle, qs, d, xf):
    wf = oracle.q8_0_dequant(synth.q8_0_raw_blocks(qs, d), qs.size).reshape(qs.shape)
    return oracle.matmul_f64(xf, wf)


@pytest.mark.parametrize("tile", [None, 0, 1, 2, 3])
@pytest.mark.parametrize("m,n,k", [(1, 64, 64), (16, 512, 1024), (33, 67, 128), (130, 200, 256), (257, 129, 4096),
                                   (128, 1024, 4096), (300, 96, 14336), (513, 600, 2048), (70, 130, 192)])
def test_gemm_vs_oracle_all_tiles_ragged(oracle, tile, m, n, k):
    # K = 64 / 192: one-tile register prefetch; 128: two tiles; multiples of 256: four
    qs, d = synth.q8_0_random(n, k, seed=m + n + k)
    xf, bits = bf16_activations(oracle, m, k, seed=m * n)
    y = run(upload(qs, d), bits, tile)
    assert y.shape == (m, n)
    elem, norm = bf16_err(y, truth_for(oracle, qs, d, xf))
    assert elem < TOL and norm < 4e-3, (elem, norm)


def test_gemm_integer_exact():
    # small integers, power-of-two scales: q*d is exact in bf16 and every partial sum exact in f32,
    # so the output must equal the bf16 rounding of the exact integer result bit for bit
    rng = np.random.default_rng(5)
    m, n, k = 70, 150, 512
    qs = rng.integers(-8, 9, (n, k), dtype=np.int8)
    d = (2.0 ** rng.integers(-2, 2, (n, k // 32))).astype(np.float16)
    x = rng.integers(-4, 5, (m, k)).astype(np.float32)
    bits = (x.view(np.uint32) >> 16).astype(np.uint16)  # small ints are bf16-exact
    want = x.astype(np.float64) @ (qs.astype(np.float64) * np.repeat(d.astype(np.float64), 32, axis=1)).T
    want_bf16 = torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16).float().numpy()
    w = upload(qs, d)
    for tile in (None, 0, 1, 2, 3):
        assert np.array_equal(run(w, bits, tile), want_bf16), tile


def test_reference_metal_matmul_case(oracle):
    """crates/luminal_metal/src/quantized.rs:937-986: W 512x1024 ints in 0..5, d = 1.0, x 16x1024 in
    U(-0.5, 0.5); its fp16 variant (:988-1038) accepts an absolute error of 1.0 because it accumulates in
    half; with f32 accumulation the bf16 result stays within bf16 rounding of the truth."""
    rng = np.random.default_rng(6)
    qs = rng.integers(0, 5, (512, 1024), dtype=np.int8)
    d = np.ones((512, 32), np.float16)
    x = rng.uniform(-0.5, 0.5, (16, 1024)).astype(np.float32)
    bits = oracle.f32_to_bf16_bits(x)
    xf = oracle.bf16_bits_to_f32(bits)
    truth = xf.astype(np.float64) @ qs.T.astype(np.float64)
    y = run(upload(qs, d), bits)
    assert np.max(np.abs(y - truth) / np.maximum(np.abs(truth), 1.0)) < 2.0 ** -8


FULL_CELLS = [(name, m) for name in ("q", "k", "v", "o", "gate", "up", "down", "lm_head") for m in (128, 512, 2048)
              if not (name in ("v", "up") and m != 512)]  # v / up have the shapes of k / gate: one cell each
FULL_CELLS += [("gate", 40), ("lm_head", 100), ("down", 300)]


@pytest.mark.parametrize("name,m", FULL_CELLS)
def test_full_size_prefill_shapes(oracle, name, m):
    """Every Llama-3-8B prefill shape at M in {128, 512, 2048} (and three off-grid M); the oracle runs on a sample
    of weight rows, the first and last forty among them."""
    n, k = synth.LLAMA3_8B_PROJ[name]
    qs, d = synth.q8_0_random(n, k, seed=300 + m)
    xf, bits = bf16_activations(oracle, m, k, seed=301)
    w = upload(qs, d)
    x = torch.from_numpy(bits.view(np.int16)).to(DEV).view(torch.bfloat16)
    y = QuantizedMatmulBf16().process(x, w)
    rows = np.unique(np.concatenate([np.arange(40), np.arange(n - 40, n),
                                     np.random.default_rng(7).integers(0, n, 112)]))
    got = y[:, torch.from_numpy(rows).to(DEV)].float().cpu().numpy()
    truth = truth_for(oracle, qs[rows], d[rows], xf)
    elem, norm = bf16_err(got, truth)
    assert elem < TOL and norm < 4e-3, (elem, norm)
    # the f32 output of the same product
    y32 = torch.empty((m, n), dtype=torch.float32, device=DEV)
    capi.check(capi.load_library().lhip_q8_0_matmul_bf16_f32out(w.planar.data_ptr(), x.data_ptr(), y32.data_ptr(), m, n, k,
                                                                torch.cuda.current_stream().cuda_stream), "f32out")
    assert rel_err(y32[:, torch.from_numpy(rows).to(DEV)].cpu().numpy(), truth) < TOL_F32
    del y, y32
    # zero activations give exactly zero; one-hot activation row gives the bf16-rounded weight column
    e = np.zeros((m, k), np.float32)
    e[m // 2, 77] = 1.0
    xe = torch.from_numpy((e.view(np.uint32) >> 16).astype(np.uint16).view(np.int16)).to(DEV).view(torch.bfloat16)
    ye = QuantizedMatmulBf16().process(xe, w)
    col = (qs[:, 77].astype(np.float32) * d[:, 77 // 32].astype(np.float32))
    want = torch.from_numpy(col).to(torch.bfloat16).float().numpy()
    assert np.array_equal(ye[m // 2].float().cpu().numpy(), want)
    ye[m // 2] = 0
    assert not bool(ye.any())


# ---- the weight-streaming kernel for at most 128 activation rows (K % 512 == 0, N % 4 == 0): tile id 5 lets
# the library choose the number of K slices, 50 + S asks for S of them

SKINNY_AUTO, SKINNY_SLICES = 5, 50


@pytest.mark.parametrize("m,n,k", [(1, 128, 512), (15, 100, 1024), (16, 260, 512), (17, 4, 1536), (33, 1024, 2048),
                                   (64, 132, 4096), (100, 516, 1024), (127, 128, 512), (128, 256, 14336)])
def test_weight_streaming_gemm_vs_oracle(oracle, m, n, k):
    """Every activation-row bracket (16, 32, 64, 128), ragged strips of weight rows, one to eight K slices (more
    slices than K has 512-element units are clamped).  The f32 output is held to the bar against the f64 product;
    the bf16 output is that result rounded once; another number of K slices only changes the order of the f32
    additions, which may tip the final rounding of a few elements by one bf16 step (or, where a sum cancelled,
    show the f32 rounding of its terms)."""
    lib = capi.load_library()
    st = torch.cuda.current_stream().cuda_stream
    qs, d = synth.q8_0_random(n, k, seed=m + n + k)
    xf, bits = bf16_activations(oracle, m, k, seed=m * n + 1)
    w = upload(qs, d)
    x = torch.from_numpy(bits.view(np.int16)).to(DEV).view(torch.bfloat16)
    y32 = torch.full((m, n), float("nan"), device=DEV)
    capi.check(lib.lhip_q8_0_matmul_bf16_f32out(w.planar.data_ptr(), x.data_ptr(), y32.data_ptr(), m, n, k, st), "f32out")
    elem, norm = bf16_err(y32.cpu().numpy(), truth_for(oracle, qs, d, xf))
    assert elem < TOL_F32 and norm < 1e-5, (elem, norm)
    auto = run(w, bits, SKINNY_AUTO)
    assert np.array_equal(auto, y32.to(torch.bfloat16).float().cpu().numpy())
    for slices in (1, 2, 3, 8):
        y = run(w, bits, SKINNY_SLICES + slices)
        # one bf16 step where the rounding tipped, and f32 rounding of the terms where the sum cancelled
        step = np.abs(auto) * 2.0 ** -7 + 1e-4 * float(np.sqrt(np.mean(auto * auto)))
        assert np.all(np.abs(y - auto) <= step) and np.mean(y == auto) > 0.98, slices


@pytest.mark.parametrize("m,n,k", [(129, 260, 1024), (300, 128, 512), (512, 1024, 4096)])
def test_weight_streaming_gemm_in_passes(oracle, m, n, k):
    """More than 128 rows through the weight-streaming kernel (tile id 5): passes of 128 rows in one launch."""
    qs, d = synth.q8_0_random(n, k, seed=m + n)
    xf, bits = bf16_activations(oracle, m, k, seed=5)
    y = run(upload(qs, d), bits, SKINNY_AUTO)
    elem, norm = bf16_err(y, truth_for(oracle, qs, d, xf))
    assert elem < TOL and norm < 4e-3, (elem, norm)


def test_weight_streaming_gemm_is_the_one_chosen_and_is_repeatable(oracle):
    """For m <= 128 the plain entry point takes the weight-streaming kernel (same bits as asking for it), K slices
    are added in a fixed order (two runs agree bit for bit, and a product that is exact in f32 is the same for
    every number of slices), and shapes it does not cover fall back to the tiled kernels."""
    lib = capi.load_library()
    s = torch.cuda.current_stream().cuda_stream
    m, n, k = 48, 4096, 4096
    qs, d = synth.q8_0_random(n, k, seed=77)
    w = upload(qs, d)
    _, bits = bf16_activations(oracle, m, k, seed=78)
    a = run(w, bits)
    assert np.array_equal(a, run(w, bits, SKINNY_AUTO)) and np.array_equal(a, run(w, bits))
    assert not np.array_equal(a, run(w, bits, 2))  # the tiled kernel adds in another order
    # small integers and power-of-two scales: every partial sum is exact
    rng = np.random.default_rng(5)
    m, n, k = 70, 152, 2048
    qi = rng.integers(-8, 9, (n, k), dtype=np.int8)
    di = (2.0 ** rng.integers(-2, 2, (n, k // 32))).astype(np.float16)
    x = rng.integers(-4, 5, (m, k)).astype(np.float32)
    xb = (x.view(np.uint32) >> 16).astype(np.uint16)
    want = x.astype(np.float64) @ (qi.astype(np.float64) * np.repeat(di.astype(np.float64), 32, axis=1)).T
    want_bf16 = torch.from_numpy(want.astype(np.float32)).to(torch.bfloat16).float().numpy()
    wi = upload(qi, di)
    for tile in (None, SKINNY_AUTO, SKINNY_SLICES + 1, SKINNY_SLICES + 2, SKINNY_SLICES + 4):
        assert np.array_equal(run(wi, xb, tile), want_bf16), tile
    # not covered: K not a multiple of 512, N not a multiple of 4, more than 64 passes of 128 rows
    xd = torch.zeros((129, 4096), dtype=torch.bfloat16, device=DEV)
    yd = torch.zeros((129, 4096), dtype=torch.bfloat16, device=DEV)

    def cfg(mm, nn, kk):
        return lib.lhip_q8_0_matmul_bf16_cfg(w.planar.data_ptr(), xd.data_ptr(), yd.data_ptr(), mm, nn, kk, SKINNY_AUTO, s)

    assert cfg(128 * 64 + 1, 64, 512) == capi.LHIP_ERR_UNSUPPORTED and cfg(8, 64, 576) == capi.LHIP_ERR_UNSUPPORTED
    assert cfg(8, 66, 512) == capi.LHIP_ERR_UNSUPPORTED and cfg(8, 64, 512) == capi.LHIP_OK
    assert cfg(129, 64, 512) == capi.LHIP_OK  # asked for by name it takes more rows, in passes of 128
    torch.cuda.synchronize()


def test_weight_streaming_gemm_output_forms(oracle):
    """f32, bf16 and SwiGLU outputs of the same product, with and without K slices: bf16 is the f32 result rounded
    once, SwiGLU is lhip_swiglu_f32_bf16out of it."""
    lib = capi.load_library()
    s = torch.cuda.current_stream().cuda_stream
    for (m, n, k) in ((24, 28672 // 4, 4096), (128, 512, 4096), (9, 4096, 14336)):  # one slice, then several
        qs, d = synth.q8_0_random(n, k, seed=m + n)
        w = upload(qs, d)
        x = torch.from_numpy(synth.activations(m, k, seed=3)).to(DEV).to(torch.bfloat16)
        y32 = torch.empty(m, n, device=DEV)
        y16 = torch.empty(m, n, device=DEV, dtype=torch.bfloat16)
        act = torch.empty(m, n // 2, device=DEV, dtype=torch.bfloat16)
        want = torch.empty_like(act)
        capi.check(lib.lhip_q8_0_matmul_bf16_f32out(w.planar.data_ptr(), x.data_ptr(), y32.data_ptr(), m, n, k, s), "f32")
        capi.check(lib.lhip_q8_0_matmul_bf16(w.planar.data_ptr(), x.data_ptr(), y16.data_ptr(), m, n, k, s), "bf16")
        capi.check(lib.lhip_q8_0_matmul_bf16_swiglu(w.planar.data_ptr(), x.data_ptr(), act.data_ptr(), m, n, k, s), "swiglu")
        capi.check(lib.lhip_swiglu_f32_bf16out(y32.data_ptr(), want.data_ptr(), m, n // 2, 1, s), "swiglu of f32")
        torch.cuda.synchronize()
        assert torch.equal(y32.to(torch.bfloat16), y16)
        assert torch.equal(act.view(torch.int16), want.view(torch.int16))


def test_k_sliced_tiled_gemm(oracle):
    """Long K and few output tiles: the 256x128 tile runs over slices of K (tile id 120 + slices) and the f32 planes
    are added in slice order.  Against the f64 product on the f32 output; bf16 and SwiGLU outputs are that result's
    forms; the plain entry point picks the sliced form for such shapes (same bits) and two runs agree."""
    lib = capi.load_library()
    st = torch.cuda.current_stream().cuda_stream
    m, n, k = 300, 512, 8192
    qs, d = synth.q8_0_random(n, k, seed=41)
    xf, bits = bf16_activations(oracle, m, k, seed=42)
    w = upload(qs, d)
    x = torch.from_numpy(bits.view(np.int16)).to(DEV).view(torch.bfloat16)
    y32 = torch.full((m, n), float("nan"), device=DEV)
    capi.check(lib.lhip_q8_0_matmul_bf16_f32out(w.planar.data_ptr(), x.data_ptr(), y32.data_ptr(), m, n, k, st), "f32out")
    elem, norm = bf16_err(y32.cpu().numpy(), truth_for(oracle, qs, d, xf))
    assert elem < TOL_F32 and norm < 1e-5, (elem, norm)
    auto = run(w, bits)
    assert np.array_equal(auto, y32.to(torch.bfloat16).float().cpu().numpy())
    assert np.array_equal(auto, run(w, bits, 120 + 8)) and np.array_equal(auto, run(w, bits))
    ref = run(w, bits, 0)  # the same tile over all of K: another order of the f32 additions
    for tile in (120 + 2, 120 + 4):
        y = run(w, bits, tile)
        step = np.abs(ref) * 2.0 ** -7 + 1e-4 * float(np.sqrt(np.mean(ref * ref)))
        assert np.all(np.abs(y - ref) <= step) and np.mean(y == ref) > 0.98, tile
    act = torch.empty(m, n // 2, device=DEV, dtype=torch.bfloat16)
    want = torch.empty_like(act)
    capi.check(lib.lhip_q8_0_matmul_bf16_swiglu(w.planar.data_ptr(), x.data_ptr(), act.data_ptr(), m, n, k, st), "swiglu")
    capi.check(lib.lhip_swiglu_f32_bf16out(y32.data_ptr(), want.data_ptr(), m, n // 2, 1, st), "swiglu of f32")
    torch.cuda.synchronize()
    assert torch.equal(act.view(torch.int16), want.view(torch.int16))
    # slices must divide K into whole rounds of four 64-wide tiles
    yd = torch.empty(m, n, device=DEV, dtype=torch.bfloat16)
    assert lib.lhip_q8_0_matmul_bf16_cfg(w.planar.data_ptr(), x.data_ptr(), yd.data_ptr(), m, n, k, 120 + 3,
                                         st) == capi.LHIP_ERR_UNSUPPORTED
    assert lib.lhip_q8_0_matmul_bf16_cfg(w.planar.data_ptr(), x.data_ptr(), yd.data_ptr(), m, n, k, 120 + 32,
                                         st) == capi.LHIP_ERR_UNSUPPORTED


def test_whole_rounds_plus_k_sliced_remainder(oracle):
    """More than 256 tiles of 256x128 whose last round would be partly filled: the plain entry points run the leading
    column tiles in whole rounds with the plain kernel and the remaining ones over K slices (tile id 200).  Here 4 row
    tiles x 81 column tiles (the last one ragged): 64 column tiles in one round, 17 over two K slices.  The leading
    columns carry the bits of the plain tile, the others are another order of the f32 additions; every output form
    is held to its bar against f64, the workspace form gives the same bits, and a product with no remainder
    refuses the plan."""
    lib = capi.load_library()
    st = torch.cuda.current_stream().cuda_stream
    m, n, k = 1024, 80 * 128 + 36, 2048
    n_main = 64 * 128
    qs, d = synth.q8_0_random(n, k, seed=51)
    xf, bits = bf16_activations(oracle, m, k, seed=52)
    w = upload(qs, d)
    x = torch.from_numpy(bits.view(np.int16)).to(DEV).view(torch.bfloat16)
    truth = truth_for(oracle, qs, d, xf)
    y32 = torch.full((m, n), float("nan"), device=DEV)
    capi.check(lib.lhip_q8_0_matmul_bf16_f32out(w.planar.data_ptr(), x.data_ptr(), y32.data_ptr(), m, n, k, st), "f32out")
    elem, norm = bf16_err(y32.cpu().numpy(), truth)
    assert elem < TOL_F32 and norm < 1e-5, (elem, norm)
    auto = run(w, bits)
    assert bf16_err(auto, truth)[0] < TOL
    assert np.array_equal(auto, y32.to(torch.bfloat16).float().cpu().numpy())
    assert np.array_equal(auto, run(w, bits, 200)) and np.array_equal(auto, run(w, bits))
    ref = run(w, bits, 0)  # the plain tile everywhere
    assert np.array_equal(auto[:, :n_main], ref[:, :n_main])
    tail, tail_ref = auto[:, n_main:], ref[:, n_main:]
    step = np.abs(tail_ref) * 2.0 ** -7 + 1e-4 * float(np.sqrt(np.mean(tail_ref * tail_ref)))
    assert np.all(np.abs(tail - tail_ref) <= step) and np.mean(tail == tail_ref) > 0.98
    act = torch.empty(m, n // 2, device=DEV, dtype=torch.bfloat16)
    want = torch.empty_like(act)
    capi.check(lib.lhip_q8_0_matmul_bf16_swiglu(w.planar.data_ptr(), x.data_ptr(), act.data_ptr(), m, n, k, st), "swiglu")
    capi.check(lib.lhip_swiglu_f32_bf16out(y32.data_ptr(), want.data_ptr(), m, n // 2, 1, st), "swiglu of f32")
    torch.cuda.synchronize()
    assert torch.equal(act.view(torch.int16), want.view(torch.int16))
    # the caller's workspace instead of the library's array: two planes of the trailing columns
    for form, dtype, cols, plain in ((0, torch.bfloat16, n, None), (1, torch.float32, n, y32), (2, torch.bfloat16, n // 2, act)):
        nbytes = lib.lhip_q8_0_matmul_bf16_workspace_nbytes(m, n, k, form)
        assert nbytes == 2 * m * (n - n_main) * 4
        space = torch.empty(nbytes, dtype=torch.uint8, device=DEV)
        y_ws = torch.empty((m, cols), dtype=dtype, device=DEV)
        capi.check(lib.lhip_q8_0_matmul_bf16_ws(w.planar.data_ptr(), x.data_ptr(), y_ws.data_ptr(), m, n, k, form,
                                                space.data_ptr(), nbytes, st), "ws")
        torch.cuda.synchronize()
        if plain is None:
            assert np.array_equal(y_ws.float().cpu().numpy(), auto)
        else:
            assert torch.equal(y_ws.view(torch.uint8), plain.view(torch.uint8)), form
    # no remainder (64 column tiles are exactly one round), or a K that two slices do not cut into rounds of four tiles
    yd = torch.empty(m, n_main, device=DEV, dtype=torch.bfloat16)
    w2 = upload(*synth.q8_0_random(n_main, k, seed=53))
    assert lib.lhip_q8_0_matmul_bf16_cfg(w2.planar.data_ptr(), x.data_ptr(), yd.data_ptr(), m, n_main, k, 200,
                                         st) == capi.LHIP_ERR_UNSUPPORTED


def test_gemm_argument_errors():
    lib = capi.load_library()
    w = upload(*synth.q8_0_random(64, 96, seed=1))
    x = torch.zeros((4, 96), dtype=torch.bfloat16, device=DEV)
    y = torch.zeros((4, 64), dtype=torch.bfloat16, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    # K = 96 is not a multiple of 64
    assert lib.lhip_q8_0_matmul_bf16(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 4, 64, 96, s) == \
        capi.LHIP_ERR_UNSUPPORTED
    assert lib.lhip_q8_0_matmul_bf16(w.planar.data_ptr(), None, y.data_ptr(), 4, 64, 128, s) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_q8_0_matmul_bf16(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 0, 64, 128, s) == \
        capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_q8_0_matmul_bf16_cfg(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 4, 64, 128, 9, s) == \
        capi.LHIP_ERR_UNSUPPORTED


@pytest.mark.parametrize("m,n,k", [(70, 150, 512), (300, 700, 1024), (513, 600, 2048)])
def test_f32_output_is_the_unrounded_accumulator(oracle, m, n, k):
    """lhip_q8_0_matmul_bf16_f32out: same kernel, accumulators stored as f32 — rounding them gives the bf16 form bit
    for bit, and they sit within the f32 bar of the f64 truth."""
    lib = capi.load_library()
    qs, d = synth.q8_0_random(n, k, seed=m + n)
    xf, bits = bf16_activations(oracle, m, k, seed=3)
    w = upload(qs, d)
    x = torch.from_numpy(bits.view(np.int16)).to(DEV).view(torch.bfloat16)
    y16 = torch.empty((m, n), dtype=torch.bfloat16, device=DEV)
    y32 = torch.empty((m, n), dtype=torch.float32, device=DEV)
    st = torch.cuda.current_stream().cuda_stream
    assert lib.lhip_q8_0_matmul_bf16(w.planar.data_ptr(), x.data_ptr(), y16.data_ptr(), m, n, k, st) == 0
    assert lib.lhip_q8_0_matmul_bf16_f32out(w.planar.data_ptr(), x.data_ptr(), y32.data_ptr(), m, n, k, st) == 0
    assert torch.equal(y32.to(torch.bfloat16), y16)
    elem, norm = bf16_err(y32.cpu().numpy(), truth_for(oracle, qs, d, xf))
    assert elem < TOL_F32 and norm < 1e-5, (elem, norm)
    assert lib.lhip_q8_0_matmul_bf16_f32out(w.planar.data_ptr(), x.data_ptr(), y32.data_ptr() + 2, m, n, k,
                                            st) == capi.LHIP_ERR_MISALIGNED


@pytest.mark.parametrize("m,n,k", [(5, 64, 64), (130, 200, 128), (512, 1024, 256), (300, 28672 // 8, 512),
                                   (16, 384, 512), (100, 4096, 1024), (128, 28672 // 8, 4096)])
def test_swiglu_epilogue_equals_gemm_then_swiglu(m, n, k):
    """lhip_q8_0_matmul_bf16_swiglu == lhip_q8_0_matmul_bf16_f32out followed by lhip_swiglu_f32_bf16out on
    interleaved (gate, up) columns, bit for bit, on every tile the library would pick and on ragged edges."""
    lib = capi.load_library()
    qs, d = synth.q8_0_random(n, k, seed=m + n + k)
    w = upload(qs, d)
    x = torch.from_numpy(synth.activations(m, k, seed=9)).to(DEV).to(torch.bfloat16)
    s = torch.cuda.current_stream().cuda_stream
    y32 = torch.empty(m, n, device=DEV)
    capi.check(lib.lhip_q8_0_matmul_bf16_f32out(w.planar.data_ptr(), x.data_ptr(), y32.data_ptr(), m, n, k, s), "gemm")
    want = torch.empty(m, n // 2, device=DEV, dtype=torch.bfloat16)
    capi.check(lib.lhip_swiglu_f32_bf16out(y32.data_ptr(), want.data_ptr(), m, n // 2, 1, s), "swiglu")
    got = torch.full((m, n // 2), 7.0, device=DEV, dtype=torch.bfloat16)
    capi.check(lib.lhip_q8_0_matmul_bf16_swiglu(w.planar.data_ptr(), x.data_ptr(), got.data_ptr(), m, n, k, s), "fused")
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # pairs are stored two at a time: N must be a multiple of 4
    assert lib.lhip_q8_0_matmul_bf16_swiglu(w.planar.data_ptr(), x.data_ptr(), got.data_ptr(), m, n - 2, k, s) \
        == capi.LHIP_ERR_INVALID_SHAPE


def _stream():
    return torch.cuda.current_stream().cuda_stream


@pytest.mark.parametrize("m,n,k", [(16, 4096, 4096), (128, 1024, 4096), (512, 4096, 4096), (512, 1024, 4096),
                                   (300, 600, 2048)])
def test_bf16_workspace_form_gives_the_plain_calls_bits_and_overlaps_safely(oracle, m, n, k):
    """lhip_q8_0_matmul_bf16_ws keeps the partial planes of a K-sliced plan in the caller's workspace: with the
    recommended size it gives the bits of the plain call for every output form (weight-streaming kernel with K
    slices, tiled kernel with K slices, plans without slices); without a workspace K is not sliced and the bar still
    holds; two streams with a workspace each run interleaved and each gets its own result."""
    lib = capi.load_library()
    qs, d = synth.q8_0_random(n, k, seed=m + n + k)
    w = upload(qs, d)
    xfs, xds = [], []
    for seed in (1, 2):
        xf, bits = bf16_activations(oracle, m, k, seed=seed)
        xfs.append(xf)
        xds.append(torch.from_numpy(bits.view(np.int16)).to(DEV).view(torch.bfloat16))
    forms = [(capi_form, plain, dtype, cols) for capi_form, plain, dtype, cols in
             ((0, lib.lhip_q8_0_matmul_bf16, torch.bfloat16, n), (1, lib.lhip_q8_0_matmul_bf16_f32out, torch.float32, n),
              (2, lib.lhip_q8_0_matmul_bf16_swiglu, torch.bfloat16, n // 2))]
    sliced = False
    for form, plain_fn, dtype, cols in forms:
        nbytes = lib.lhip_q8_0_matmul_bf16_workspace_nbytes(m, n, k, form)
        sliced = sliced or nbytes > 0
        assert nbytes % 4 == 0 and nbytes <= 32 << 20
        spaces = [torch.empty(max(nbytes, 256), dtype=torch.uint8, device=DEV) for _ in xds]
        plain = []
        for x in xds:
            y = torch.empty((m, cols), dtype=dtype, device=DEV)
            capi.check(plain_fn(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), m, n, k, _stream()), "plain")
            plain.append(y)
        y_ws = torch.empty((m, cols), dtype=dtype, device=DEV)
        capi.check(lib.lhip_q8_0_matmul_bf16_ws(w.planar.data_ptr(), xds[0].data_ptr(), y_ws.data_ptr(), m, n, k, form,
                                                spaces[0].data_ptr() if nbytes else None, nbytes, _stream()), "ws")
        y_none = torch.empty((m, cols), dtype=dtype, device=DEV)
        capi.check(lib.lhip_q8_0_matmul_bf16_ws(w.planar.data_ptr(), xds[0].data_ptr(), y_none.data_ptr(), m, n, k, form,
                                                None, 0, _stream()), "ws none")
        torch.cuda.synchronize()
        assert torch.equal(y_ws.view(torch.uint8), plain[0].view(torch.uint8)), form
        if form != 2:
            truth = truth_for(oracle, qs, d, xfs[0])
            assert rel_err(y_none.float().cpu().numpy(), truth) < (TOL if form == 0 else TOL_F32), form
        streams = [torch.cuda.Stream(), torch.cuda.Stream()]
        outs = [torch.empty((m, cols), dtype=dtype, device=DEV) for _ in xds]
        torch.cuda.synchronize()
        for _ in range(10):
            for i, st in enumerate(streams):
                capi.check(lib.lhip_q8_0_matmul_bf16_ws(w.planar.data_ptr(), xds[i].data_ptr(), outs[i].data_ptr(), m, n, k,
                                                        form, spaces[i].data_ptr() if nbytes else None, nbytes,
                                                        st.cuda_stream), "ws 2")
        torch.cuda.synchronize()
        for i in range(2):
            assert torch.equal(outs[i].view(torch.uint8), plain[i].view(torch.uint8)), (form, i)
    assert sliced  # every shape here has a K-sliced plan in at least one output form


def test_bf16_workspace_form_argument_checks():
    lib = capi.load_library()
    w = upload(*synth.q8_0_random(1024, 1024, seed=3))
    x = torch.zeros((8, 1024), device=DEV, dtype=torch.bfloat16)
    y = torch.empty((8, 1024), device=DEV, dtype=torch.bfloat16)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=DEV)
    p, xp, yp = w.planar.data_ptr(), x.data_ptr(), y.data_ptr()
    assert lib.lhip_q8_0_matmul_bf16_workspace_nbytes(8, 1024, 1000, 0) == 0   # invalid shape
    assert lib.lhip_q8_0_matmul_bf16_workspace_nbytes(8, 1024, 1024, 3) == 0   # no such output form
    assert lib.lhip_q8_0_matmul_bf16_ws(p, xp, yp, 8, 1024, 1024, 3, None, 0, _stream()) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_q8_0_matmul_bf16_ws(p, xp, yp, 8, 1024, 1024, 0, ws.data_ptr() + 64, 1 << 19, _stream()) == capi.LHIP_ERR_MISALIGNED
    assert lib.lhip_q8_0_matmul_bf16_ws(None, xp, yp, 8, 1024, 1024, 0, None, 0, _stream()) == capi.LHIP_ERR_NULL_PTR


def test_result_of_a_row_depends_on_the_row_count_only_through_the_plan(oracle):
    """The contract on M: a row's result does not depend on the other rows of the call (equal bits whatever they
    hold), calls with the same M take the same plan (equal bits), and calls whose M selects another plan - the
    weight-streaming kernel up to 128 rows, K slices of the tiled kernel, the tiled kernel - agree within the
    operator's tolerance, not bit for bit (another order of the f32 additions)."""
    n, k = 4096, 4096
    qs, d = synth.q8_0_random(n, k, seed=77)
    w = upload(qs, d)
    xf, bits = bf16_activations(oracle, 2048, k, seed=5)
    truth0 = truth_for(oracle, qs, d, xf[:1])
    x_all = torch.from_numpy(bits.view(np.int16)).to(DEV).view(torch.bfloat16)
    row0 = {}
    for m in (1, 16, 128, 512, 2048):
        y = QuantizedMatmulBf16().process(x_all[:m].contiguous(), w)
        other = x_all[:m].clone()
        if m > 1:
            other[1:] = torch.flip(other[1:], dims=[0]) * 3.0  # the same first row among different rows
        y2 = QuantizedMatmulBf16().process(other, w)
        torch.cuda.synchronize()
        assert torch.equal(y[0].view(torch.int16), y2[0].view(torch.int16)), m
        row0[m] = y[0].float().cpu().numpy()
        assert rel_err(row0[m][None, :], truth0) < TOL, m
    differing = sum(not np.array_equal(row0[a], row0[b]) for a, b in ((1, 16), (16, 128), (128, 512), (512, 2048)))
    print(f"[M contract] pairs of neighbouring plans whose first rows differ in some bit: {differing} of 4")
