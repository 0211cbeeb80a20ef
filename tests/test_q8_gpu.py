"""Parity of the Q8_0 HIP path with the CPU oracle, through the C ABI.

Bars: storage transforms and dequantised weights bit-exact; matmul outputs
within max relative error 2e-3 of the f64 truth (floor 1e-3*rms, see
conftest.rel_err), and within the reference's own absolute 1e-3 convention
(src/tests/mod.rs:67-69) on O(1) data.
"""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from conftest import rel_err  # noqa: E402
from luminal_amd import capi, synth  # noqa: E402
from luminal_amd.quantized import Q8Weight, QuantizedGather, QuantizedMatmul  # noqa: E402

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = 2e-3


def upload(qs, d):
    n, k = qs.shape
    return Q8Weight.from_raw(synth.q8_0_raw_blocks(qs, d), n, k, DEV)


def dequant_truth(oracle, qs, d):
    raw = synth.q8_0_raw_blocks(qs, d)
    return oracle.q8_0_dequant(raw, qs.size).reshape(qs.shape)


# ---------------------------------------------------------------- storage

@pytest.mark.parametrize("n,k", [(1, 32), (3, 32), (7, 96), (64, 1024), (129, 1056), (1024, 4096)])
def test_repack_unpack_round_trip_bit_exact(n, k):
    qs, d = synth.q8_0_random(n, k, seed=n * 131 + k)
    raw = synth.q8_0_raw_blocks(qs, d)
    w = Q8Weight.from_raw(raw, n, k, DEV)
    planar = w.planar.cpu().numpy()
    off = capi.load_library().lhip_q8_0_planar_scale_offset(n, k)
    assert np.array_equal(planar[: n * k].view(np.int8).reshape(n, k), qs)
    assert np.array_equal(planar[off:].view(np.float16).reshape(n, k // 32), d)
    assert np.array_equal(w.to_raw().cpu().numpy(), raw)


@pytest.mark.parametrize("n,k", [(3, 96), (129, 1056), (1024, 4096)])
def test_planar_form_depends_on_the_block_count_only(n, k):
    # a loader that knows a tensor's element count but not its (n, k), as the reference's loader does
    # (examples/llama/src/loader.rs:121-130), may repack it as (n_elements / 32, 32)
    qs, d = synth.q8_0_random(n, k, seed=n + k)
    raw = synth.q8_0_raw_blocks(qs, d)
    by_shape = Q8Weight.from_raw(raw, n, k, DEV).planar.cpu().numpy()
    by_count = Q8Weight.from_raw(raw, n * k // 32, 32, DEV).planar.cpu().numpy()
    assert np.array_equal(by_shape, by_count)


@pytest.mark.parametrize("n,k", [(1, 32), (5, 96), (129, 1056), (2048, 1024)])
def test_interleaved_rows_are_the_sources_rows_bit_for_bit(n, k):
    qa, da = synth.q8_0_random(n, k, seed=3 * n + k)
    qb, db = synth.q8_0_random(n, k, seed=5 * n + k)
    both = Q8Weight.interleave_rows(upload(qa, da), upload(qb, db))
    assert (both.n, both.k) == (2 * n, k)
    qs = np.empty((2 * n, k), dtype=np.int8)
    d = np.empty((2 * n, k // 32), dtype=np.float16)
    qs[0::2], qs[1::2], d[0::2], d[1::2] = qa, qb, da, db
    planar = both.planar.cpu().numpy()
    off = capi.load_library().lhip_q8_0_planar_scale_offset(2 * n, k)
    assert np.array_equal(planar[:2 * n * k].view(np.int8).reshape(2 * n, k), qs)  # the padding behind it is not written
    assert np.array_equal(planar[off:].view(np.float16).reshape(2 * n, k // 32), d)
    assert np.array_equal(both.to_raw().cpu().numpy(), synth.q8_0_raw_blocks(qs, d))


def test_interleave_rows_rejects_bad_arguments():
    lib = capi.load_library()
    a = upload(*synth.q8_0_random(4, 64, seed=1))
    out = torch.empty(Q8Weight.planar_nbytes(8, 64) + 256, dtype=torch.uint8, device=DEV)
    p = a.planar.data_ptr()
    assert lib.lhip_q8_0_interleave_rows(None, p, out.data_ptr(), 4, 64, None) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_q8_0_interleave_rows(p, p, out.data_ptr() + 16, 4, 64, None) == capi.LHIP_ERR_MISALIGNED
    assert lib.lhip_q8_0_interleave_rows(p, p, out.data_ptr(), 4, 48, None) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_q8_0_interleave_rows(p, p, out.data_ptr(), 0, 64, None) == capi.LHIP_ERR_INVALID_SHAPE
    with pytest.raises(capi.LhipError):
        Q8Weight.interleave_rows(a, upload(*synth.q8_0_random(4, 96, seed=2)))


def test_dequant_bit_exact_every_quant_times_every_scale(oracle):
    # all 256 int8 values x all 65536 f16 codes (NaN codes compared as NaN)
    n, k = 65536, 256
    qs = np.broadcast_to(np.arange(-128, 128, dtype=np.int8), (n, k)).copy()
    d = np.repeat(np.arange(65536, dtype=np.uint16).view(np.float16)[:, None], k // 32, axis=1)
    got = upload(qs, d).dequantize().cpu().numpy()
    want = dequant_truth(oracle, qs, d)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_dequant_bit_exact_benchmark_distribution(oracle):
    qs, d = synth.q8_0_random(1024, 4096, seed=11)
    got = upload(qs, d).dequantize().cpu().numpy()
    assert np.array_equal(got.view(np.uint32), dequant_truth(oracle, qs, d).view(np.uint32))


def test_gather_bit_exact(oracle):
    qs, d = synth.q8_0_random(1000, 4096, seed=12)
    w = upload(qs, d)
    idx = np.array([0, 999, 5, 5, 123.7, 998.99], np.float32)
    got = QuantizedGather(4096).process(torch.from_numpy(idx), w).cpu().numpy()
    want = oracle.q8_0_gather(synth.q8_0_raw_blocks(qs, d), idx, 4096)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # out-of-range and non-finite indices give zero rows
    bad = QuantizedGather(4096).process(torch.tensor([-1.0, 1000.0, float("nan"), 3e9]), w).cpu().numpy()
    assert not bad.any()


# ---------------------------------------------------------------- matvec / matmul

def run_matmul(w, x, cfg=None):
    op = QuantizedMatmul(*cfg) if cfg else QuantizedMatmul()
    y = op.process(torch.from_numpy(x).to(DEV), w)
    torch.cuda.synchronize()
    return y.cpu().numpy()


def test_config0_single_matvec_4096(oracle):
    """The single-matvec benchmark case: W 4096x4096, x 1x4096 N(0,1), y = x W^T in f32."""
    qs, d = synth.q8_0_random(4096, 4096, seed=0x5EED)
    x = synth.activations(1, 4096, seed=0x5EED + 1)
    w = upload(qs, d)
    wf = dequant_truth(oracle, qs, d)
    truth = oracle.matmul_f64(x, wf)
    y = run_matmul(w, x)
    assert y.shape == (1, 4096)
    assert rel_err(y, truth) < TOL
    # the oracle's own f32 path (sequential, unfused) is no closer to the truth than we must be
    seq = oracle.matmul_seq_f32(x, wf)
    assert rel_err(seq, truth) < TOL
    assert np.max(np.abs(y - seq)) < 1e-3 * max(1.0, float(np.max(np.abs(seq))))


# (rows_per_wave, k_unroll, blocks_per_cu): blocks_per_cu == 0 is the one-shot kernel
ONESHOT = [(r, u, 0) for r, u in [(1, 1), (1, 2), (1, 4), (2, 1), (2, 2), (2, 4), (4, 1), (4, 2), (4, 4), (8, 1),
                                  (8, 2)]]
PIPE = [(r, s, b, w) for r in (1, 2, 4) for s in (1, 2, 4) for b, w in ((1, 4), (3, 4), (2, 8), (1, 16))
        if not (w == 16 and r * s > 8)]


@pytest.mark.parametrize("n,k", [(1, 32), (5, 64), (33, 1024), (37, 1056), (64, 2048), (130, 3104), (257, 4096),
                                 (2051, 4096), (96, 14336), (1029, 8192), (70, 16384), (9, 20480)])
def test_matvec_every_launch_shape_ragged(oracle, n, k):
    qs, d = synth.q8_0_random(n, k, seed=n + k)
    x = synth.activations(1, k, seed=n * k)
    w = upload(qs, d)
    truth = oracle.matmul_f64(x, dequant_truth(oracle, qs, d))
    for cfg in [None] + ONESHOT:
        y = run_matmul(w, x, cfg)
        assert rel_err(y, truth) < TOL, (n, k, cfg)
    for cfg in PIPE:
        if k % (cfg[1] * 1024) == 0 and k <= 16384:
            assert rel_err(run_matmul(w, x, cfg), truth) < TOL, (n, k, cfg)
        else:  # the pipelined kernel needs K to be a whole number of steps that fits its LDS stage
            with pytest.raises(capi.LhipError) as e:
                run_matmul(w, x, cfg)
            assert e.value.status == capi.LHIP_ERR_UNSUPPORTED


def test_unbuilt_launch_shape_is_reported():
    qs, d = synth.q8_0_random(4, 32, seed=1)
    w = upload(qs, d)
    with pytest.raises(capi.LhipError) as e:
        run_matmul(w, synth.activations(1, 32, 2), cfg=(3, 1, 0))
    assert e.value.status == capi.LHIP_ERR_UNSUPPORTED


@pytest.mark.parametrize("m", [2, 5, 16])
def test_matmul_rows_of_x(oracle, m):
    # the reference runs its matvec once per activation row (grid z = m*batch,
    # crates/luminal_cuda/src/quantized.rs:159); M=16 is its test_quantized_matmul shape
    qs, d = synth.q8_0_random(512, 1024, seed=21)
    x = synth.activations(m, 1024, seed=22)
    w = upload(qs, d)
    truth = oracle.matmul_f64(x, dequant_truth(oracle, qs, d))
    y = run_matmul(w, x)
    assert y.shape == (m, 512)
    assert rel_err(y, truth) < TOL
    # leading batch dims fold into M
    y3 = QuantizedMatmul().process(torch.from_numpy(x).to(DEV).reshape(1, m, 1024), w).cpu().numpy()
    assert y3.shape == (1, m, 512) and np.array_equal(y3[0], y)


def test_more_activation_rows_than_one_grid_dimension_holds():
    """The matvec form puts the rows of x on the grid's y axis (at most 65 535): a taller x goes in several passes.
    K = 32 keeps the call on the matvec form (the matrix-core form wants K % 512 == 0)."""
    n, k, m = 8, 32, 70001
    qs, d = synth.q8_0_random(n, k, seed=5)
    w = upload(qs, d)
    x = torch.randn(m, k, device=DEV)
    for dt, fn in ((torch.float32, "lhip_q8_0_matmul_f32"), (torch.float16, "lhip_q8_0_matmul_f16")):
        xs = x.to(dt)
        y = torch.full((m, n), float("nan"), device=DEV, dtype=dt)
        lib = capi.load_library()
        capi.check(getattr(lib, fn)(w.planar.data_ptr(), xs.data_ptr(), y.data_ptr(), m, n, k, None), fn)
        # every row equals the same row computed in a call of its own size class (bit for bit: one arithmetic)
        for rows in (slice(0, 3), slice(65533, 65538), slice(m - 2, m)):
            part = torch.empty((rows.stop - rows.start, n), device=DEV, dtype=dt)
            capi.check(getattr(lib, fn)(w.planar.data_ptr(), xs[rows].contiguous().data_ptr(), part.data_ptr(),
                                        rows.stop - rows.start, n, k, None), fn)
            as_int = torch.int32 if dt == torch.float32 else torch.int16
            assert torch.equal(y[rows].view(as_int), part.view(as_int))
        assert not torch.isnan(y.float()).any()


def test_reference_metal_matvec_case(oracle):
    """crates/luminal_metal/src/quantized.rs:888-935: W 512x1024 ints in 0..5,
    d = 1.0, x in U(-0.5,0.5), absolute 1e-3 against the f32 graph."""
    rng = np.random.default_rng(31)
    qs = rng.integers(0, 5, (512, 1024), dtype=np.int8)
    d = np.ones((512, 32), np.float16)
    x = rng.uniform(-0.5, 0.5, (1, 1024)).astype(np.float32)
    w = upload(qs, d)
    want = oracle.matmul_seq_f32(x, qs.astype(np.float32))
    assert np.max(np.abs(run_matmul(w, x) - want)) < 1e-3
    # M = 16 (test_quantized_matmul, :937-986)
    x16 = rng.uniform(-0.5, 0.5, (16, 1024)).astype(np.float32)
    want16 = oracle.matmul_seq_f32(x16, qs.astype(np.float32))
    assert np.max(np.abs(run_matmul(w, x16) - want16)) < 1e-3


def test_integer_exact_any_order():
    # small integers and power-of-two scales: every partial sum is exact in f32,
    # so any summation order must give the integer answer bit for bit
    rng = np.random.default_rng(32)
    n, k = 300, 2048
    qs = rng.integers(-8, 9, (n, k), dtype=np.int8)
    d = (2.0 ** rng.integers(-3, 3, (n, k // 32))).astype(np.float16)
    x = rng.integers(-4, 5, (1, k)).astype(np.float32)
    want = (qs.astype(np.float64) * np.repeat(d.astype(np.float64), 32, axis=1)) @ x[0].astype(np.float64)
    w = upload(qs, d)
    for cfg in [None, (1, 1, 0), (2, 2, 0), (4, 4, 0), (8, 2, 0), (1, 2, 2), (2, 1, 1), (4, 2, 4), (2, 2, 1, 8),
                (1, 2, 2, 16)]:
        assert np.array_equal(run_matmul(w, x, cfg)[0].astype(np.float64), want), cfg


def test_zero_scale_blocks_and_extreme_quants(oracle):
    n, k = 64, 1024
    qs = np.full((n, k), -128, np.int8)
    qs[::2] = 127
    d = np.full((n, k // 32), 0.01, np.float16)
    d[:, ::3] = 0.0  # these blocks must contribute nothing
    x = synth.activations(1, k, seed=33)
    w = upload(qs, d)
    truth = oracle.matmul_f64(x, dequant_truth(oracle, qs, d))
    assert rel_err(run_matmul(w, x), truth) < TOL


# ---------------------------------------------------------------- full-size properties

@pytest.mark.parametrize("name", ["q", "k", "gate", "down", "lm_head"])
def test_full_size_projection_vs_oracle(oracle, name):
    """The Llama-3-8B decode projection shapes at full size against the f64 truth."""
    n, k = synth.LLAMA3_8B_PROJ[name]
    qs, d = synth.q8_0_random(n, k, seed=100 + sorted(synth.LLAMA3_8B_PROJ).index(name))
    x = synth.activations(1, k, seed=77)
    w = upload(qs, d)
    y = run_matmul(w, x)
    # oracle on a bounded sample of rows keeps the CPU side to seconds
    rows = np.unique(np.concatenate([np.arange(0, 64), np.arange(n - 64, n),
                                     np.random.default_rng(5).integers(0, n, 2048)]))
    wf = dequant_truth(oracle, qs[rows], d[rows])
    truth = oracle.matmul_f64(x, wf)
    assert rel_err(y[:, rows], truth) < TOL
    # one-hot activation: y is exactly a dequantised column (size-independent)
    col = 1234
    e = np.zeros((1, k), np.float32)
    e[0, col] = 1.0
    ycol = run_matmul(w, e)[0]
    want = qs[:, col].astype(np.float32) * d[:, col // 32].astype(np.float32)
    assert np.array_equal(ycol, want)
    # linearity: W(2x) == 2 W(x) exactly (power-of-two scaling commutes with rounding)
    assert np.array_equal(run_matmul(w, 2.0 * x), 2.0 * y)


def test_error_statuses_on_device():
    lib = capi.load_library()
    w = upload(*synth.q8_0_random(8, 64, seed=3))
    x = torch.zeros(64, device=DEV)
    y = torch.zeros(8, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.lhip_q8_0_matmul_f32(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 1, 8, 64, s) == 0
    assert lib.lhip_q8_0_matmul_f32(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 1, 8, 65, s) == 2
    assert lib.lhip_q8_0_matmul_f32(w.planar.data_ptr(), x.data_ptr() + 4, y.data_ptr(), 1, 8, 64, s) == 3
    assert lib.lhip_init(0) == 0
    assert lib.lhip_init(1 << 20) == capi.LHIP_ERR_INVALID_SHAPE
    torch.cuda.synchronize()


def test_plumbing_malloc_copy_round_trip():
    import ctypes as C

    lib = capi.load_library()
    p = C.c_void_p()
    assert lib.lhip_malloc(C.byref(p), 4096) == 0
    src = np.arange(1024, dtype=np.int32)
    dst = np.zeros_like(src)
    assert lib.lhip_memcpy_h2d(p, src.ctypes.data, 4096, None) == 0
    assert lib.lhip_memcpy_d2h(dst.ctypes.data, p, 4096, None) == 0
    assert lib.lhip_stream_sync(None) == 0
    assert np.array_equal(src, dst)
    assert lib.lhip_free(p) == 0
