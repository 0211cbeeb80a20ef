"""The reference's second activation type, T = f16 (QuantizedMatmul<f16> / QuantizedGather<f16>,
crates/luminal_cuda/src/quantized.rs:42-109,170-233), through the C ABI.

Bars: the f16 matvec equals the f32 matvec on the same (f16-representable) activations rounded once to f16, bit
for bit, because both run the same f32 arithmetic in the same order; it is within 2e-3 of the f64 truth; the f16
gather equals the exact dequantised row rounded once to f16.
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


def both(w, x16):
    """(f16 result, f32 result on the same activation values)."""
    xd = torch.from_numpy(x16).to(DEV)
    y16 = QuantizedMatmul().process(xd, w)
    y32 = QuantizedMatmul().process(xd.float(), w)
    torch.cuda.synchronize()
    assert y16.dtype == torch.float16 and y32.dtype == torch.float32
    return y16.cpu().numpy(), y32.cpu().numpy()


# one shape per launch choice of the library: one-shot kernel with 1 / 2 / 4 rows per wave (ragged K),
# pipelined kernel 1x1, 1x2 (3 workgroups per CU), 1x1 and 1x2 with 16 waves (long K), 2x4 (very tall)
@pytest.mark.parametrize("n,k", [(1, 32), (37, 1056), (4100, 96), (8200, 64), (33, 1024), (64, 2048), (257, 4096),
                                 (96, 14336), (70, 16384), (33000, 4096)])
def test_f16_matvec_equals_rounded_f32_matvec(oracle, n, k):
    qs, d = synth.q8_0_random(n, k, seed=n + k)
    x16 = synth.activations(1, k, seed=n * k).astype(np.float16)
    w = upload(qs, d)
    y16, y32 = both(w, x16)
    assert y16.shape == (1, n)
    assert np.array_equal(y16.view(np.uint16), y32.astype(np.float16).view(np.uint16))
    truth = oracle.matmul_f64(x16.astype(np.float32), dequant_truth(oracle, qs, d))
    assert rel_err(y16.astype(np.float32), truth) < TOL


@pytest.mark.parametrize("m", [2, 16])
def test_f16_matmul_rows_of_x(oracle, m):
    qs, d = synth.q8_0_random(512, 1024, seed=21)
    x16 = synth.activations(m, 1024, seed=22).astype(np.float16)
    w = upload(qs, d)
    y16, y32 = both(w, x16)
    assert y16.shape == (m, 512)
    assert np.array_equal(y16.view(np.uint16), y32.astype(np.float16).view(np.uint16))
    truth = oracle.matmul_f64(x16.astype(np.float32), dequant_truth(oracle, qs, d))
    assert rel_err(y16.astype(np.float32), truth) < TOL


def test_reference_fp16_case(oracle):
    """crates/luminal_metal/src/quantized.rs:988-1038 restated: W 512x1024 of integers 0..4 with d = 1.0, x 16x1024
    uniform in (-0.5, 0.5) in f16, checked there against an f32 matmul to an absolute 1.0 (it accumulated in f16);
    here accumulation is f32, so the result is the f32 product rounded to f16."""
    rng = np.random.default_rng(7)
    qs = rng.integers(0, 5, (512, 1024)).astype(np.int8)
    d = np.ones((512, 32), np.float16)
    x16 = (rng.random((16, 1024), dtype=np.float32) - 0.5).astype(np.float16)
    w = upload(qs, d)
    y16, _ = both(w, x16)
    want = x16.astype(np.float64) @ qs.astype(np.float64).T
    assert np.max(np.abs(y16.astype(np.float64) - want)) < 1.0              # the reference's bar
    assert np.max(np.abs(y16.astype(np.float64) - want)) <= np.max(np.abs(want)) * 2.0 ** -10  # half an f16 ulp and change


def test_f16_gather_is_the_exact_row_rounded_once(oracle):
    qs, d = synth.q8_0_random(1000, 4096, seed=12)
    w = upload(qs, d)
    idx = np.array([0, 999, 5, 5, 123.7, 998.99], np.float32)
    got = QuantizedGather(4096, torch.float16).process(torch.from_numpy(idx), w).cpu().numpy()
    want = oracle.q8_0_gather(synth.q8_0_raw_blocks(qs, d), idx, 4096).astype(np.float16)
    assert got.dtype == np.float16 and np.array_equal(got.view(np.uint16), want.view(np.uint16))
    bad = QuantizedGather(4096, torch.float16).process(torch.tensor([-1.0, 1000.0, float("nan")]), w).cpu().numpy()
    assert not bad.any()


def test_f16_argument_errors():
    lib = capi.load_library()
    qs, d = synth.q8_0_random(8, 64, seed=3)
    w = upload(qs, d)
    x = torch.zeros(64, dtype=torch.float16, device=DEV)
    y = torch.zeros(8, dtype=torch.float16, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.lhip_q8_0_matmul_f16(None, x.data_ptr(), y.data_ptr(), 1, 8, 64, s) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_q8_0_matmul_f16(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), 1, 8, 48, s) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_q8_0_matmul_f16(w.planar.data_ptr(), x.data_ptr() + 2, y.data_ptr(), 1, 8, 64, s) == capi.LHIP_ERR_MISALIGNED
    assert lib.lhip_q8_0_gather_f16(w.planar.data_ptr(), None, y.data_ptr(), 1, 8, 64, s) == capi.LHIP_ERR_NULL_PTR
    with pytest.raises(TypeError):
        QuantizedMatmul(1, 1, 0).process(x.reshape(1, 64), w)  # launch shapes are an f32-only knob
