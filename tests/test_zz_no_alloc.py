"""lhip_mxfp4_moe_bf16_static, the entry point that allocates nothing (its workspace is a scratch array inside the
library): same bits as lhip_mxfp4_moe_bf16 on two calls in a row, the second with a smaller input that leaves part
of the scratch array holding the first call's contents; sizes beyond the array are refused."""
import numpy as np
import pytest

torch = pytest.importorskip("torch")

from luminal_amd import capi, synth  # noqa: E402
from luminal_amd.moe import Mxfp4Weight, MoEExperts, route_topk  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_static_workspace_entry_point_equals_the_workspace_one():
    lib = capi.load_library()
    e, h, i, topk = 8, 256, 192, 4
    gu_c, gu_s = synth.mxfp4_random(e * 2 * i, h, seed=11)
    dn_c, dn_s = synth.mxfp4_random(e * h, i, seed=12)
    gu = Mxfp4Weight.from_raw(synth.mxfp4_raw_blocks(gu_c, gu_s), e * 2 * i, h, DEV)
    dn = Mxfp4Weight.from_raw(synth.mxfp4_raw_blocks(dn_c, dn_s), e * h, i, DEV)
    layer = MoEExperts(gu, dn, e, h, i)
    rng = np.random.default_rng(13)
    st = torch.cuda.current_stream().cuda_stream
    for t in (300, 37):  # two calls in a row, the second smaller
        assert 0 < lib.lhip_mxfp4_moe_workspace_nbytes(t, h, i, e, topk) <= 8 << 20
        x = torch.from_numpy(rng.standard_normal((t, h)).astype(np.float32)).to(DEV).to(torch.bfloat16)
        sel, wts = route_topk(torch.from_numpy(rng.standard_normal((t, e)).astype(np.float32)).to(DEV), topk)
        want = layer.process(x, sel, wts)
        got = torch.full((t, h), 7.0, dtype=torch.bfloat16, device=DEV)
        capi.check(lib.lhip_mxfp4_moe_bf16_static(gu.planar.data_ptr(), dn.planar.data_ptr(), x.data_ptr(), sel.data_ptr(),
                                                  wts.data_ptr(), got.data_ptr(), t, h, i, e, topk, st), "static")
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), t
        assert bool(torch.isfinite(got.float()).all()) and float(got.float().abs().max()) > 0
    # the two-launch direct form for at most four routed rows (batch-1 decode, what the entry point is aimed at): one
    # token with top-4 and two tokens with top-2, each with one routed entry that names no expert (its activation
    # rows in the scratch array are never written and must not be used)
    for t, k in ((1, 4), (2, 2)):
        x = torch.from_numpy(rng.standard_normal((t, h)).astype(np.float32)).to(DEV).to(torch.bfloat16)
        sel, wts = route_topk(torch.from_numpy(rng.standard_normal((t, e)).astype(np.float32)).to(DEV), k)
        sel[0, 1] = e + 3
        want = layer.process(x, sel, wts)
        got = torch.full((t, h), 7.0, dtype=torch.bfloat16, device=DEV)
        capi.check(lib.lhip_mxfp4_moe_bf16_static(gu.planar.data_ptr(), dn.planar.data_ptr(), x.data_ptr(), sel.data_ptr(),
                                                  wts.data_ptr(), got.data_ptr(), t, h, i, e, k, st), "static")
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (t, k)
        assert bool(torch.isfinite(got.float()).all()) and float(got.float().abs().max()) > 0
    # beyond the scratch array: refused, nothing launched
    big_t = 4096
    assert lib.lhip_mxfp4_moe_workspace_nbytes(big_t, h, i, e, topk) > 8 << 20
    p = gu.planar.data_ptr()
    assert lib.lhip_mxfp4_moe_bf16_static(p, p, p, p, p, p, big_t, h, i, e, topk, st) == capi.LHIP_ERR_UNSUPPORTED
    assert lib.lhip_mxfp4_moe_bf16_static(p, p, p, p, p, p, 4, h, 48, e, topk, st) == capi.LHIP_ERR_INVALID_SHAPE
    assert lib.lhip_mxfp4_moe_bf16_static(None, p, p, p, p, p, 4, h, i, e, topk, st) == capi.LHIP_ERR_NULL_PTR
