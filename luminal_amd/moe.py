"""Host-side wrappers of the MXFP4 mixture-of-experts entry points (no
counterpart in the reference; see include/luminal_hip.h).  torch provides
device memory and the current stream only."""
from __future__ import annotations

import numpy as np
import torch

from . import capi


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


class Mxfp4Weight:
    """A (N, K) MXFP4 weight resident on the device in planar form."""

    def __init__(self, planar: torch.Tensor, n: int, k: int):
        self.planar, self.n, self.k = planar, n, k

    @classmethod
    def from_raw(cls, raw, n: int, k: int, device="cuda:0") -> "Mxfp4Weight":
        lib = capi.load_library()
        if isinstance(raw, np.ndarray):
            raw = torch.from_numpy(np.ascontiguousarray(raw, dtype=np.uint8))
        raw = raw.reshape(-1)
        expect = lib.lhip_mxfp4_raw_nbytes(n, k)
        if expect == 0 or raw.numel() != expect:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "Mxfp4Weight.from_raw",
                                 f"expected {expect} bytes for ({n}, {k}), got {raw.numel()}")
        raw_dev = raw.to(device)
        planar = torch.empty(lib.lhip_mxfp4_planar_nbytes(n, k), dtype=torch.uint8, device=device)
        with torch.cuda.device(planar.device):
            capi.check(lib.lhip_mxfp4_repack(raw_dev.data_ptr(), planar.data_ptr(), n, k, _stream()),
                       "lhip_mxfp4_repack")
            torch.cuda.current_stream().synchronize()
        return cls(planar, n, k)

    def to_raw(self) -> torch.Tensor:
        lib = capi.load_library()
        raw = torch.empty(lib.lhip_mxfp4_raw_nbytes(self.n, self.k), dtype=torch.uint8, device=self.planar.device)
        with torch.cuda.device(raw.device):
            capi.check(lib.lhip_mxfp4_unpack(self.planar.data_ptr(), raw.data_ptr(), self.n, self.k, _stream()),
                       "lhip_mxfp4_unpack")
        return raw

    def dequantize_bf16(self) -> torch.Tensor:
        """The weight as the bf16 numbers the exact expert GEMMs multiply (lhip_mxfp4_dequant_bf16)."""
        lib = capi.load_library()
        out = torch.empty((self.n, self.k), dtype=torch.bfloat16, device=self.planar.device)
        with torch.cuda.device(out.device):
            capi.check(lib.lhip_mxfp4_dequant_bf16(self.planar.data_ptr(), out.data_ptr(), self.n, self.k, _stream()),
                       "lhip_mxfp4_dequant_bf16")
        return out

    def dequantize(self) -> torch.Tensor:
        lib = capi.load_library()
        out = torch.empty((self.n, self.k), dtype=torch.float32, device=self.planar.device)
        with torch.cuda.device(out.device):
            capi.check(lib.lhip_mxfp4_dequant_f32(self.planar.data_ptr(), out.data_ptr(), self.n, self.k, _stream()),
                       "lhip_mxfp4_dequant_f32")
        return out


def route_topk(logits: torch.Tensor, topk: int):
    """(T, E) f32 logits -> (sel int32 (T, topk), wts f32 (T, topk))."""
    lib = capi.load_library()
    logits = logits.contiguous()
    t, e = logits.shape
    sel = torch.empty((t, topk), dtype=torch.int32, device=logits.device)
    wts = torch.empty((t, topk), dtype=torch.float32, device=logits.device)
    with torch.cuda.device(logits.device):
        capi.check(lib.lhip_moe_route_topk(logits.data_ptr(), sel.data_ptr(), wts.data_ptr(), t, e, topk, _stream()),
                   "lhip_moe_route_topk")
    return sel, wts


class MoEExperts:
    """E experts of hidden H, intermediate I: gate/up fused (E*2I, H) and down (E*H, I), both MXFP4."""

    def __init__(self, w_gate_up: Mxfp4Weight, w_down: Mxfp4Weight, experts: int, hidden: int, inter: int):
        assert w_gate_up.n == experts * 2 * inter and w_gate_up.k == hidden
        assert w_down.n == experts * hidden and w_down.k == inter
        self.gu, self.dn, self.e, self.h, self.i = w_gate_up, w_down, experts, hidden, inter
        self._ws = None

    def process(self, x: torch.Tensor, sel: torch.Tensor, wts: torch.Tensor, mode: int = capi.LHIP_MOE_EXACT) -> torch.Tensor:
        """mode: capi.LHIP_MOE_EXACT (bf16 matrix instruction on exactly expanded weights, the default) or
        capi.LHIP_MOE_FAST (block-scaled fp4 x fp8 instruction)."""
        lib = capi.load_library()
        if x.dtype != torch.bfloat16 or not x.is_cuda:
            raise TypeError("MoEExperts expects bf16 activations on the GPU")
        x = x.contiguous()
        t = x.shape[0]
        topk = sel.shape[1]
        need = lib.lhip_mxfp4_moe_workspace_nbytes(t, self.h, self.i, self.e, topk)
        if need == 0:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "MoEExperts", "invalid MoE shape")
        if self._ws is None or self._ws.numel() < need:
            self._ws = torch.empty(need, dtype=torch.uint8, device=x.device)
        y = torch.empty((t, self.h), dtype=torch.bfloat16, device=x.device)
        with torch.cuda.device(x.device):
            st = lib.lhip_mxfp4_moe_bf16_mode(self.gu.planar.data_ptr(), self.dn.planar.data_ptr(), x.data_ptr(),
                                              sel.contiguous().data_ptr(), wts.contiguous().data_ptr(), y.data_ptr(), t,
                                              self.h, self.i, self.e, topk, mode, self._ws.data_ptr(), _stream())
        capi.check(st, "lhip_mxfp4_moe_bf16_mode")
        self._last = (t, topk, mode)
        return y

    def intermediates(self):
        """(act (T*topk, I) f32, down (T*topk, H) f32) of the last `process` call: the SwiGLU activations as the down
        projection consumed them and every routed entry's down projection (lhip_mxfp4_moe_read_intermediates)."""
        lib = capi.load_library()
        t, topk, mode = self._last
        dev = self._ws.device
        act = torch.empty((t * topk, self.i), dtype=torch.float32, device=dev)
        down = torch.empty((t * topk, self.h), dtype=torch.float32, device=dev)
        with torch.cuda.device(dev):
            st = lib.lhip_mxfp4_moe_read_intermediates_mode(self._ws.data_ptr(), act.data_ptr(), down.data_ptr(), t,
                                                            self.h, self.i, self.e, topk, mode, _stream())
        capi.check(st, "lhip_mxfp4_moe_read_intermediates_mode")
        return act, down
