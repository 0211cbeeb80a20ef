"""Parity of the fused batch-1 matvec (grouped sibling weights, RMS-norm prologue, residual and SwiGLU epilogues)
with the CPU oracle, through the C ABI.

Bars: with no prologue/epilogue the fused launch equals the plain matvec bit for bit (same per-row arithmetic);
with them, max relative error 2e-3 against the f64 composition of the oracle's pieces (conftest.rel_err).
"""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from conftest import rel_err  # noqa: E402
from luminal_amd import capi, synth  # noqa: E402
from luminal_amd.quantized import FusedMatvec, Q8Weight, QuantizedMatmul  # noqa: E402
from oracle import llama_oracle as lo  # noqa: E402

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
TOL = 2e-3
CFGS = [(2, 4, 4, 1), (1, 2, 4, 3), (2, 2, 4, 2), (1, 1, 4, 3), (2, 1, 4, 2), (1, 2, 16, 1), (2, 2, 8, 1), (1, 1, 16, 1),
        (2, 1, 8, 1)]


def make(n, k, seed):
    qs, d = synth.q8_0_random(n, k, seed=seed)
    raw = synth.q8_0_raw_blocks(qs, d)
    return Q8Weight.from_raw(raw, n, k, DEV), raw


def dense(oracle, raw, n, k):
    return oracle.q8_0_dequant(raw, n * k).reshape(n, k)


@pytest.mark.parametrize("k,ns", [(4096, (4096, 1024, 1024)), (4096, (14336, 14336)), (2048, (77, 1, 300, 5)),
                                  (1024, (130,)), (14336, (4096,)), (4096, (128256,))])
def test_grouped_launch_equals_plain_matvec_bitwise(k, ns):
    ws = [make(n, k, 31 * i + n % 97)[0] for i, n in enumerate(ns)]
    x = torch.from_numpy(synth.activations(1, k, seed=k + len(ns))).to(DEV).reshape(k)
    ys = [torch.full((n,), float("nan"), device=DEV) for n in ns]
    FusedMatvec(ws, ys).run(x)
    for w, y in zip(ws, ys):
        want = QuantizedMatmul().process(x.reshape(1, k), w).reshape(-1)
        assert torch.equal(y, want)


@pytest.mark.parametrize("cfg", CFGS)
def test_every_launch_shape_grouped(oracle, cfg):
    k = 4096
    ns = (70, 1026, 3)
    made = [make(n, k, 7 + i) for i, n in enumerate(ns)]
    x = synth.activations(1, k, seed=3)
    ys = [torch.full((n,), float("nan"), device=DEV) for n in ns]
    FusedMatvec([m[0] for m in made], ys, cfg=cfg).run(torch.from_numpy(x).to(DEV).reshape(k))
    for (w, raw), y, n in zip(made, ys, ns):
        truth = oracle.matmul_f64(x, dense(oracle, raw, n, k)).reshape(-1)
        assert rel_err(y.cpu().numpy(), truth) < TOL


def test_longest_staged_k(oracle):
    """K = 16384: 64 KiB of staged activations plus the reduction array is more LDS than a kernel gets without
    asking; with and without the norm prologue, and the plain operator's kernel at the same K."""
    k, n = 16384, 520
    w, raw = make(n, k, 3)
    rng = np.random.default_rng(1)
    x = rng.standard_normal(k).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    wd = dense(oracle, raw, n, k)
    y = torch.full((n,), float("nan"), device=DEV)
    FusedMatvec([w], [y]).run(torch.from_numpy(x).to(DEV))
    assert rel_err(y.cpu().numpy(), oracle.matmul_f64(x[None, :], wd).reshape(-1)) < TOL
    assert torch.equal(y, QuantizedMatmul().process(torch.from_numpy(x).to(DEV).reshape(1, k), w).reshape(-1))
    y.fill_(float("nan"))
    FusedMatvec([w], [y], norm_weight=torch.from_numpy(g).to(DEV), eps=1e-5).run(torch.from_numpy(x).to(DEV))
    assert rel_err(y.cpu().numpy(), lo.rms_norm(x[None, :], g, 1e-5) @ wd.astype(np.float64).T) < TOL


@pytest.mark.parametrize("k,n", [(4096, 6144), (1024, 200), (2048, 4096), (4096, 32768)])
def test_rms_norm_prologue(oracle, k, n):
    w, raw = make(n, k, 5)
    rng = np.random.default_rng(k + n)
    x = (3.0 * rng.standard_normal(k)).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    eps = 1e-5
    y = torch.empty(n, device=DEV)
    FusedMatvec([w], [y], norm_weight=torch.from_numpy(g).to(DEV), eps=eps).run(torch.from_numpy(x).to(DEV))
    xn = lo.rms_norm(x[None, :], g, eps)
    truth = xn @ dense(oracle, raw, n, k).astype(np.float64).T
    assert rel_err(y.cpu().numpy(), truth) < TOL


@pytest.mark.parametrize("k,n", [(4096, 4096), (14336, 4096), (1024, 130), (2048, 77)])
def test_residual_epilogue_in_place(oracle, k, n):
    w, raw = make(n, k, 9)
    x = synth.activations(1, k, seed=2)
    res = np.random.default_rng(n).standard_normal(n).astype(np.float32)
    h = torch.from_numpy(res.copy()).to(DEV)
    FusedMatvec([w], [h], residual=h, epilogue=FusedMatvec.EPI_ADD).run(torch.from_numpy(x).to(DEV).reshape(k))
    truth = res.astype(np.float64) + oracle.matmul_f64(x, dense(oracle, raw, n, k)).reshape(-1)
    assert rel_err(h.cpu().numpy(), truth) < TOL


@pytest.mark.parametrize("k,f,cfg", [(4096, 14336, None), (1024, 65, None), (2048, 512, (2, 2, 8, 1)),
                                     (4096, 700, (2, 4, 4, 1)), (1024, 300, (2, 1, 4, 2)), (1024, 300, (2, 1, 8, 1))])
def test_norm_prologue_and_swiglu_epilogue_on_interleaved_rows(oracle, k, f, cfg):
    w, raw = make(2 * f, k, 13)
    rng = np.random.default_rng(f)
    x = rng.standard_normal(k).astype(np.float32)
    g = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    y = torch.empty(f, device=DEV)
    FusedMatvec([w], [y], norm_weight=torch.from_numpy(g).to(DEV), eps=1e-5, epilogue=FusedMatvec.EPI_SWIGLU,
                cfg=cfg).run(torch.from_numpy(x).to(DEV))
    gu = lo.rms_norm(x[None, :], g, 1e-5) @ dense(oracle, raw, 2 * f, k).astype(np.float64).T
    truth = lo.swish(gu[0, 0::2]) * gu[0, 1::2]
    assert rel_err(y.cpu().numpy(), truth) < TOL


def test_swiglu_operator_reads_interleaved_rows():
    lib = capi.load_library()
    rng = np.random.default_rng(0)
    gu = rng.standard_normal((3, 2 * 96)).astype(np.float32)
    out = torch.empty((3, 96), device=DEV)
    st = lib.lhip_swiglu_f32(torch.from_numpy(gu).to(DEV).data_ptr(), out.data_ptr(), 3, 96, 1,
                             torch.cuda.current_stream().cuda_stream)
    assert st == 0
    want = lo.swish(gu[:, 0::2].astype(np.float64)) * gu[:, 1::2]
    assert rel_err(out.cpu().numpy(), want) < 1e-5


def test_argument_errors():
    lib = capi.load_library()
    w, _ = make(64, 1024, 1)
    x = torch.zeros(1024, device=DEV)
    y = torch.zeros(64, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    wp, yp, n = (C.c_void_p * 1)(w.planar.data_ptr()), (C.c_void_p * 1)(y.data_ptr()), (C.c_int64 * 1)(64)

    def call(count=1, k=1024, norm=None, res=None, epi=0, wp=wp, yp=yp, n=n, xp=x.data_ptr()):
        return lib.lhip_q8_0_matvec_fused_f32(wp, yp, n, count, xp, k, norm, 0.0, res, epi, s)

    assert call() == capi.LHIP_OK
    assert call(count=0) == capi.LHIP_ERR_INVALID_SHAPE
    assert call(count=5) == capi.LHIP_ERR_INVALID_SHAPE
    assert call(k=1000) == capi.LHIP_ERR_INVALID_SHAPE
    assert call(k=1056) == capi.LHIP_ERR_UNSUPPORTED      # legal Q8_0 width the fused kernel does not take
    assert call(k=32768) == capi.LHIP_ERR_UNSUPPORTED
    assert call(epi=1) == capi.LHIP_ERR_NULL_PTR          # residual missing
    assert call(epi=3) == capi.LHIP_ERR_UNSUPPORTED
    assert call(xp=None) == capi.LHIP_ERR_NULL_PTR
    assert call(xp=x.data_ptr() + 4) == capi.LHIP_ERR_MISALIGNED
    assert call(wp=(C.c_void_p * 1)(None)) == capi.LHIP_ERR_NULL_PTR
    assert call(n=(C.c_int64 * 1)(63), epi=2) == capi.LHIP_ERR_INVALID_SHAPE  # odd row count has no pairs
    two_w, two_y, two_n = (C.c_void_p * 2)(w.planar.data_ptr(), w.planar.data_ptr()), (C.c_void_p * 2)(
        y.data_ptr(), y.data_ptr()), (C.c_int64 * 2)(64, 64)
    assert call(count=2, wp=two_w, yp=two_y, n=two_n, res=y.data_ptr(), epi=1) == capi.LHIP_ERR_UNSUPPORTED
    assert lib.lhip_q8_0_matvec_fused_f32_cfg(wp, yp, n, 1, x.data_ptr(), 1024, None, 0.0, None, 0, 3, 1, 4, 1,
                                              s) == capi.LHIP_ERR_UNSUPPORTED
    assert lib.lhip_q8_0_matvec_fused_f32_cfg(wp, yp, n, 1, x.data_ptr(), 1024, None, 0.0, None, 2, 1, 1, 4, 1,
                                              s) == capi.LHIP_ERR_UNSUPPORTED  # pairs need two rows per wave
    torch.cuda.synchronize()
