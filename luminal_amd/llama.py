"""Llama-3 decode loop over the luminal_hip C ABI.

Host-side counterpart of examples/llama/src/{model.rs,main.rs}: the same layer
stack and generation loop (prefill, then greedy decode with a KV cache), with
every tensor op running in libluminal_hip.so.  torch holds the device buffers
and, optionally, replays a captured HIP graph of one decode step.  Linear
weights are Q8_0; q|k|v are stored row-concatenated and gate/up row-interleaved
(row 2j = gate_j, row 2j+1 = up_j) so each is one matvec (row-wise the same
arithmetic as the reference's separate matmuls).  Batch-1 decode runs six
launches per layer: RMS norm is folded into the qkv and gate/up matvecs, SwiGLU
into the gate/up epilogue and the residual adds into the o and down epilogues.
"""
from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from . import capi
from .quantized import DecodeProgram, FusedMatvec, Q8Weight


@dataclass(frozen=True)
class LlamaConfig:
    """Constants of examples/llama/src/model.rs:5-14."""
    vocab: int = 128256
    dim: int = 4096
    layers: int = 32
    q_heads: int = 32
    kv_heads: int = 8
    ffn: int = 14336
    eps: float = 1e-5
    theta: float = 500000.0

    @property
    def head_dim(self) -> int:
        return self.dim // self.q_heads

    @property
    def qkv_rows(self) -> int:
        return (self.q_heads + 2 * self.kv_heads) * self.head_dim


LLAMA3_8B = LlamaConfig()


def _s() -> int:
    return torch.cuda.current_stream().cuda_stream


class LlamaQ8:
    def __init__(self, cfg: LlamaConfig, weights: dict, max_seq: int, device="cuda:0"):
        """weights: 'embed' f32 (vocab, dim) or Q8Weight (vocab, dim); 'out_norm' f32 (dim); 'lm_head' Q8Weight (vocab, dim); and per
        layer i: f'{i}.attn_norm', f'{i}.ffn_norm' f32 (dim); f'{i}.qkv' Q8Weight (qkv_rows, dim);
        f'{i}.o' (dim, dim); f'{i}.gate_up' (2*ffn, dim), gate and up rows interleaved; f'{i}.down' (dim, ffn)."""
        self.cfg, self.w, self.max_seq, self.dev = cfg, weights, max_seq, torch.device(device)
        self.lib = capi.load_library()
        kv = (cfg.kv_heads, max_seq, cfg.head_dim)
        self.k_cache = [torch.zeros(kv, dtype=torch.float32, device=self.dev) for _ in range(cfg.layers)]
        self.v_cache = [torch.zeros(kv, dtype=torch.float32, device=self.dev) for _ in range(cfg.layers)]
        self.pos = torch.zeros(1, dtype=torch.int32, device=self.dev)
        self._pos_host = 0  # host copy of the position, for the max_seq check
        self.tok = torch.zeros(1, dtype=torch.float32, device=self.dev)      # next token id, as f32
        self.tok_i = torch.zeros(1, dtype=torch.int32, device=self.dev)
        self._bufs = {}
        self._graph = None
        # The fused matvec stages K activations in LDS in slices of 1024.
        self.fused_decode = all(k % 1024 == 0 and k <= 16384 for k in (cfg.dim, cfg.ffn))
        self._plans = None
        # persistent_decode = True runs a decode step as one persistent launch (lhip_decode_program_*) where the
        # library builds it for these shapes.  Same bits; measured slower on MI355X than one launch per fused operator
        # replayed from a graph (2.9 against 2.2 ms per token at Llama-3-8B), so it is off unless asked for.
        self.persistent_decode = False
        self._program = None
        ws = self.lib.lhip_attention_decode_workspace_nbytes(cfg.q_heads, cfg.kv_heads, cfg.head_dim)
        self._attn_ws = torch.empty(ws, dtype=torch.uint8, device=self.dev) if ws else None
        # merge_in_o_proj = True lets the output projection merge the attention's key ranges while it stages its
        # activations (lhip_attention_decode_partial_f32 + lhip_q8_0_matvec_attn_merge_f32: one launch fewer per
        # layer).  Measured slower on MI355X than the three launches (21.0 against 17.6 us per layer at 512-768
        # keys: with few key ranges the attention kernel takes two tiles of dependent memory trips per range, and
        # the merge inside the projection's prologue delays its weight stream), so it is off unless asked for.
        self.merge_in_o_proj = False
        self._can_merge_in_o_proj = (self._attn_ws is not None and cfg.dim % 2048 == 0 and cfg.dim <= 16384
                                     and max_seq <= 2048)

    # ---- buffers -----------------------------------------------------------
    def _buf(self, name, shape, dtype=torch.float32):
        key = (name, tuple(shape), dtype)
        if key not in self._bufs:
            self._bufs[key] = torch.empty(shape, dtype=dtype, device=self.dev)
        return self._bufs[key]

    def reset(self):
        self.pos.zero_()
        self._pos_host = 0

    def _room(self, n: int):
        """The KV caches hold max_seq positions (the reference's caches grow instead, model.rs:108-110): a pass that
        would run past them is refused here, on the host, before anything is launched."""
        if self._pos_host + n > self.max_seq:
            raise capi.LhipError(capi.LHIP_ERR_INVALID_SHAPE, "LlamaQ8",
                                 f"position {self._pos_host} + {n} tokens exceeds max_seq {self.max_seq}")

    def _embed(self, tokens_f32, out, n):
        """Embedding rows of n token ids (f32, on the device): an f32 table (crates/luminal_nn/src/embedding.rs:40-58) or
        a Q8_0 one (QuantizedGather, crates/luminal_cuda/src/quantized.rs:170-233)."""
        cfg, lib, e = self.cfg, self.lib, self.w["embed"]
        if isinstance(e, Q8Weight):
            capi.check(lib.lhip_q8_0_gather_f32(e.planar.data_ptr(), tokens_f32.data_ptr(), out.data_ptr(), n, cfg.vocab,
                                                cfg.dim, _s()), "lhip_q8_0_gather_f32")
        else:
            capi.check(lib.lhip_gather_rows_f32(e.data_ptr(), tokens_f32.data_ptr(), out.data_ptr(), n, cfg.vocab,
                                                cfg.dim, _s()), "lhip_gather_rows_f32")

    # ---- ops ---------------------------------------------------------------
    def _matmul(self, w: Q8Weight, x, y, m, bf16):
        lib = self.lib
        if not bf16:
            capi.check(lib.lhip_q8_0_matmul_f32(w.planar.data_ptr(), x.data_ptr(), y.data_ptr(), m, w.n, w.k, _s()),
                       "lhip_q8_0_matmul_f32")
            return
        xb = self._buf("xb", (m, w.k), torch.bfloat16)
        yb = self._buf("yb", (m, w.n), torch.bfloat16)
        capi.check(lib.lhip_cast_f32_to_bf16(x.data_ptr(), xb.data_ptr(), m * w.k, _s()), "cast")
        capi.check(lib.lhip_q8_0_matmul_bf16(w.planar.data_ptr(), xb.data_ptr(), yb.data_ptr(), m, w.n, w.k, _s()),
                   "lhip_q8_0_matmul_bf16")
        capi.check(lib.lhip_cast_bf16_to_f32(yb.data_ptr(), y.data_ptr(), m * w.n, _s()), "cast")

    def _norm(self, x, res, x_out, w, y, rows):
        capi.check(self.lib.lhip_rms_norm_f32(x.data_ptr(), res.data_ptr() if res is not None else None,
                                              x_out.data_ptr() if x_out is not None else None, w.data_ptr(),
                                              y.data_ptr(), rows, self.cfg.dim, self.cfg.eps, _s()), "lhip_rms_norm_f32")

    def forward(self, tokens_f32: torch.Tensor, s: int, bf16: bool = False, all_logits: bool = False):
        """Runs s tokens (ids as f32 on the device) at positions pos .. pos+s-1, appends to the KV cache and
        returns the logits of the last position ((vocab,)), or of all positions ((s, vocab)).
        Does not advance the position."""
        self._room(s)
        if bf16 and s > 1:
            return self._forward_prompt_bf16(tokens_f32, s, all_logits)
        cfg, lib, w = self.cfg, self.lib, self.w
        d, hd = cfg.dim, cfg.head_dim
        h = self._buf("h", (s, d))
        n = self._buf("n", (s, d))
        qkv = self._buf("qkv", (s, cfg.qkv_rows))
        att = self._buf("att", (s, d))
        o = self._buf("o", (s, d))
        gu = self._buf("gu", (s, 2 * cfg.ffn))
        act = self._buf("act", (s, cfg.ffn))
        dn = self._buf("dn", (s, d))
        self._embed(tokens_f32, h, s)
        for i in range(cfg.layers):
            if i == 0:
                self._norm(h, None, None, w["0.attn_norm"], n, s)
            else:  # residual of the previous layer's MLP, fused into this norm
                self._norm(h, dn, h, w[f"{i}.attn_norm"], n, s)
            self._matmul(w[f"{i}.qkv"], n, qkv, s, bf16)
            if s == 1:
                self._attend_one(i, qkv, att)
            else:
                capi.check(lib.lhip_rope_kv_append_f32(qkv.data_ptr(), self.k_cache[i].data_ptr(),
                                                       self.v_cache[i].data_ptr(), self.pos.data_ptr(), s, cfg.q_heads,
                                                       cfg.kv_heads, hd, self.max_seq, cfg.theta, _s()), "rope")
                capi.check(lib.lhip_attention_f32(qkv.data_ptr(), self.k_cache[i].data_ptr(),
                                                  self.v_cache[i].data_ptr(), att.data_ptr(), self.pos.data_ptr(), s,
                                                  cfg.q_heads, cfg.kv_heads, hd, self.max_seq, _s()), "attention")
            self._matmul(w[f"{i}.o"], att, o, s, bf16)
            self._norm(h, o, h, w[f"{i}.ffn_norm"], n, s)          # h += attn out; n = norm(h)
            self._matmul(w[f"{i}.gate_up"], n, gu, s, bf16)
            capi.check(lib.lhip_swiglu_f32(gu.data_ptr(), act.data_ptr(), s, cfg.ffn, 1, _s()), "swiglu")
            self._matmul(w[f"{i}.down"], act, dn, s, bf16)
        self._norm(h, dn, h, w["out_norm"], n, s)                    # last residual + final norm
        if all_logits:
            logits = self._buf("logits_all", (s, cfg.vocab))
            self._matmul(w["lm_head"], n, logits, s, bf16)
            return logits
        logits = self._buf("logits", (cfg.vocab,))
        last = n[s - 1]
        self._matmul(w["lm_head"], last, logits, 1, False)  # only the last position is read (main.rs:58-61)
        return logits

    def _forward_prompt_bf16(self, tokens_f32: torch.Tensor, s: int, all_logits: bool):
        """Prompt pass with the linears on the bf16 matrix-core GEMM.  The residual stream, rotary, attention and
        softmax stay f32; the operators in front of a GEMM write bf16 and the GEMM stores its f32 accumulators, so
        there is no cast kernel anywhere."""
        cfg, lib, w = self.cfg, self.lib, self.w
        d, hd = cfg.dim, cfg.head_dim
        bf = torch.bfloat16
        h = self._buf("h", (s, d))
        nb = self._buf("nb", (s, d), bf)
        qkv = self._buf("qkv", (s, cfg.qkv_rows))
        attb = self._buf("attb", (s, d), bf)
        att = self._buf("att", (s, d))
        o = self._buf("o", (s, d))
        actb = self._buf("actb", (s, cfg.ffn), bf)
        dn = self._buf("dn", (s, d))

        def norm(res, wt):
            capi.check(lib.lhip_rms_norm_f32_bf16out(h.data_ptr(), res.data_ptr() if res is not None else None,
                                                     h.data_ptr() if res is not None else None, wt.data_ptr(),
                                                     nb.data_ptr(), s, d, cfg.eps, _s()), "lhip_rms_norm_f32_bf16out")

        def gemm(wq, x, y, m):
            capi.check(lib.lhip_q8_0_matmul_bf16_f32out(wq.planar.data_ptr(), x.data_ptr(), y.data_ptr(), m, wq.n, wq.k,
                                                        _s()), "lhip_q8_0_matmul_bf16_f32out")

        self._embed(tokens_f32, h, s)
        for i in range(cfg.layers):
            norm(None if i == 0 else dn, w[f"{i}.attn_norm"])       # h += previous MLP out; nb = norm(h)
            gemm(w[f"{i}.qkv"], nb, qkv, s)
            capi.check(lib.lhip_rope_kv_append_f32(qkv.data_ptr(), self.k_cache[i].data_ptr(),
                                                   self.v_cache[i].data_ptr(), self.pos.data_ptr(), s, cfg.q_heads,
                                                   cfg.kv_heads, hd, self.max_seq, cfg.theta, _s()), "rope")
            a_args = (qkv.data_ptr(), self.k_cache[i].data_ptr(), self.v_cache[i].data_ptr())
            a_dims = (self.pos.data_ptr(), s, cfg.q_heads, cfg.kv_heads, hd, self.max_seq, _s())
            # bf16 matrix-core operands where the head shape has that kernel, else the f32 matrix-core kernel
            # writing bf16, else (no matrix-core kernel at all) the f32 attention and a cast
            st = lib.lhip_attention_bf16(*a_args, attb.data_ptr(), *a_dims)
            if st == capi.LHIP_ERR_UNSUPPORTED:
                st = lib.lhip_attention_f32_bf16out(*a_args, attb.data_ptr(), *a_dims)
            if st == capi.LHIP_ERR_UNSUPPORTED:
                capi.check(lib.lhip_attention_f32(*a_args, att.data_ptr(), *a_dims), "attention")
                capi.check(lib.lhip_cast_f32_to_bf16(att.data_ptr(), attb.data_ptr(), s * d, _s()), "cast")
            else:
                capi.check(st, "prompt attention")
            gemm(w[f"{i}.o"], attb, o, s)
            norm(o, w[f"{i}.ffn_norm"])                              # h += attention out; nb = norm(h)
            gw = w[f"{i}.gate_up"]                                   # rows are (gate, up) pairs: SwiGLU in the epilogue
            capi.check(lib.lhip_q8_0_matmul_bf16_swiglu(gw.planar.data_ptr(), nb.data_ptr(), actb.data_ptr(), s, gw.n,
                                                        gw.k, _s()), "lhip_q8_0_matmul_bf16_swiglu")
            gemm(w[f"{i}.down"], actb, dn, s)
        if all_logits:
            norm(dn, w["out_norm"])
            logits = self._buf("logits_all", (s, cfg.vocab))
            gemm(w["lm_head"], nb, logits, s)
            return logits
        n = self._buf("n", (s, d))
        self._norm(h, dn, h, w["out_norm"], n, s)                   # last residual + final norm, f32
        logits = self._buf("logits", (cfg.vocab,))
        self._matmul(w["lm_head"], n[s - 1], logits, 1, False)      # only the last position is read (main.rs:58-61)
        return logits

    def _build_plans(self):
        cfg, w = self.cfg, self.w
        h = self._buf("h", (1, cfg.dim)).view(-1)
        qkv = self._buf("qkv", (1, cfg.qkv_rows)).view(-1)
        att = self._buf("att", (1, cfg.dim)).view(-1)
        act = self._buf("act", (1, cfg.ffn)).view(-1)
        logits = self._buf("logits", (cfg.vocab,))
        plans = []
        for i in range(cfg.layers):
            plans.append((
                FusedMatvec([w[f"{i}.qkv"]], [qkv], norm_weight=w[f"{i}.attn_norm"], eps=cfg.eps),
                FusedMatvec([w[f"{i}.o"]], [h], residual=h, epilogue=FusedMatvec.EPI_ADD),
                FusedMatvec([w[f"{i}.gate_up"]], [act], norm_weight=w[f"{i}.ffn_norm"], eps=cfg.eps,
                            epilogue=FusedMatvec.EPI_SWIGLU),
                FusedMatvec([w[f"{i}.down"]], [h], residual=h, epilogue=FusedMatvec.EPI_ADD)))
        head = FusedMatvec([w["lm_head"]], [logits], norm_weight=w["out_norm"], eps=cfg.eps)
        self._plans = (plans, head, h, qkv, att, act, logits)
        self._program = None
        if self.persistent_decode and self._attn_ws is not None:
            # the same operations as one persistent launch (lhip_decode_program_*)
            prog = DecodeProgram(cfg.q_heads, cfg.kv_heads, cfg.head_dim, self.max_seq, cfg.theta, self.pos)
            for i in range(cfg.layers):
                prog.matvec(w[f"{i}.qkv"], h, qkv, norm_weight=w[f"{i}.attn_norm"], eps=cfg.eps)
                prog.attention(qkv, self.k_cache[i], self.v_cache[i], att)
                prog.matvec(w[f"{i}.o"], att, h, residual=h, epilogue=FusedMatvec.EPI_ADD)
                prog.matvec(w[f"{i}.gate_up"], h, act, norm_weight=w[f"{i}.ffn_norm"], eps=cfg.eps,
                            epilogue=FusedMatvec.EPI_SWIGLU)
                prog.matvec(w[f"{i}.down"], act, h, residual=h, epilogue=FusedMatvec.EPI_ADD)
            prog.matvec(w["lm_head"], h, logits, norm_weight=w["out_norm"], eps=cfg.eps)
            try:
                self._program = prog.build()
            except capi.LhipError as e:
                if e.status != capi.LHIP_ERR_UNSUPPORTED:
                    raise

    def forward_decode(self, token_f32: torch.Tensor):
        """One token at position pos through the fused batch-1 path; returns the logits (vocab,)."""
        cfg, lib = self.cfg, self.lib
        self._room(1)
        if not self.fused_decode:
            return self.forward(token_f32, 1)
        if self._plans is None:
            self._build_plans()
        plans, head, h, qkv, att, act, logits = self._plans
        self._embed(token_f32, h, 1)
        if self._program is not None:
            self._program.run()
            return logits
        for i, (p_qkv, p_o, p_gu, p_down) in enumerate(plans):
            p_qkv.run(h)                                   # qkv = Wqkv norm(h)
            if self.merge_in_o_proj and self._can_merge_in_o_proj:
                self._attend_partial(i, qkv)
                w_o = self.w[f"{i}.o"]
                capi.check(lib.lhip_q8_0_matvec_attn_merge_f32(w_o.planar.data_ptr(), h.data_ptr(), w_o.n, w_o.k,
                                                               self._attn_ws.data_ptr(), self.pos.data_ptr(), cfg.q_heads,
                                                               cfg.kv_heads, cfg.head_dim, self.max_seq, h.data_ptr(), _s()),
                           "lhip_q8_0_matvec_attn_merge_f32")  # h += Wo merge(partial states)
            else:
                self._attend_one(i, qkv, att)
                p_o.run(att)                               # h += Wo att
            p_gu.run(h)                                    # act = up * swish(gate) of Wgu norm(h)
            p_down.run(act)                                # h += Wdown act
        head.run(h)                                        # logits = Wout norm(h)
        return logits

    def _attend_partial(self, i, qkv):
        """Rotary, cache append and attention over the key ranges for one new token of layer i; the ranges' partial
        states stay in the workspace."""
        cfg = self.cfg
        capi.check(self.lib.lhip_attention_decode_partial_f32(qkv.data_ptr(), self.k_cache[i].data_ptr(),
                                                              self.v_cache[i].data_ptr(), self.pos.data_ptr(), cfg.q_heads,
                                                              cfg.kv_heads, cfg.head_dim, self.max_seq, cfg.theta,
                                                              self._attn_ws.data_ptr(), _s()),
                   "lhip_attention_decode_partial_f32")

    def _attend_one(self, i, qkv, att):
        """Rotary, cache append and attention for one new token of layer i."""
        cfg, lib = self.cfg, self.lib
        if self._attn_ws is not None:
            capi.check(lib.lhip_attention_decode_f32(qkv.data_ptr(), self.k_cache[i].data_ptr(),
                                                     self.v_cache[i].data_ptr(), att.data_ptr(), self.pos.data_ptr(),
                                                     cfg.q_heads, cfg.kv_heads, cfg.head_dim, self.max_seq, cfg.theta,
                                                     self._attn_ws.data_ptr(), _s()), "lhip_attention_decode_f32")
            return
        capi.check(lib.lhip_rope_kv_append_f32(qkv.data_ptr(), self.k_cache[i].data_ptr(), self.v_cache[i].data_ptr(),
                                               self.pos.data_ptr(), 1, cfg.q_heads, cfg.kv_heads, cfg.head_dim,
                                               self.max_seq, cfg.theta, _s()), "rope")
        capi.check(lib.lhip_attention_f32(qkv.data_ptr(), self.k_cache[i].data_ptr(), self.v_cache[i].data_ptr(),
                                          att.data_ptr(), self.pos.data_ptr(), 1, cfg.q_heads, cfg.kv_heads,
                                          cfg.head_dim, self.max_seq, _s()), "attention")

    def _pick(self, logits, advance):
        capi.check(self.lib.lhip_argmax_f32(logits.data_ptr(), self.cfg.vocab, self.tok.data_ptr(),
                                            self.tok_i.data_ptr(), self.pos.data_ptr(), advance, _s()), "argmax")

    # ---- generation loop (examples/llama/src/main.rs:101-190) ----------------
    def prefill(self, tokens, bf16: bool = False):
        t = torch.as_tensor(np.asarray(tokens, dtype=np.float32)).to(self.dev)
        logits = self.forward(t, t.numel(), bf16=bf16)
        self._pick(logits, t.numel())
        self._pos_host += t.numel()
        return logits

    def decode_step(self):
        logits = self.forward_decode(self.tok)
        self._pick(logits, 1)
        self._pos_host += 1
        return logits

    def decode(self, steps: int, use_graph: bool = True):
        """Greedy decode of `steps` tokens after a prefill; returns the token ids (first = the prefill's pick)."""
        self._room(steps)
        out = torch.empty(steps, dtype=torch.int32, device=self.dev)
        # Capturing the graph runs two real steps first (a warm-up and the captured one), which append K/V rows at
        # pos and pos + 1 before the position is put back: with fewer than two free positions the steps that still
        # fit run eagerly instead.
        if use_graph and self._graph is None and self._pos_host + 2 > self.max_seq:
            use_graph = False
        if not use_graph:
            for i in range(steps):
                out[i:i + 1].copy_(self.tok_i)
                self.decode_step()
            self._check_program()
            return out
        if self._graph is None:
            pos0, tok0, toki0, host0 = self.pos.clone(), self.tok.clone(), self.tok_i.clone(), self._pos_host
            st = torch.cuda.Stream(device=self.dev)
            st.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(st):
                self.decode_step()  # warm-up outside capture (allocates the step's buffers)
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=st):
                    self.decode_step()
            torch.cuda.current_stream().wait_stream(st)
            self._graph = g
            # undo the two steps above: the cache rows they wrote are rewritten by the replays
            self.pos.copy_(pos0)
            self.tok.copy_(tok0)
            self.tok_i.copy_(toki0)
            self._pos_host = host0
        for i in range(steps):
            out[i:i + 1].copy_(self.tok_i)
            self._graph.replay()
        self._pos_host += steps
        self._check_program()
        return out

    def _check_program(self):
        """With the persistent decode program, a grid-wide wait that gave up leaves the step's results meaningless by
        design; ask (this synchronises the device) before the tokens are handed back."""
        if self._program is not None and self._program.timed_out():
            raise capi.LhipError(capi.LHIP_ERR_HIP, "LlamaQ8.decode",
                                 "the persistent decode program gave up a wait: the tokens of this call are not valid")


def fuse_rows(*raws: np.ndarray) -> np.ndarray:
    """Row-concatenate Q8_0 weights with the same K: their raw block streams simply follow each other."""
    return np.concatenate([np.ascontiguousarray(r, dtype=np.uint8).reshape(-1) for r in raws])


def interleave_rows(a: np.ndarray, b: np.ndarray, k: int) -> np.ndarray:
    """Raw Q8_0 block streams of two (n, k) weights -> the (2n, k) weight whose rows alternate a_0, b_0, a_1, ..."""
    row = k // 32 * 34
    a = np.ascontiguousarray(a, dtype=np.uint8).reshape(-1, row)
    b = np.ascontiguousarray(b, dtype=np.uint8).reshape(-1, row)
    return np.stack([a, b], axis=1).reshape(-1)


def random_weights(cfg: LlamaConfig, seed: int, device="cuda:0", scale_sigma: float | None = None) -> dict:
    """Random Q8_0 model built on the device (quants U{-127..127}; block scales |N(0, sigma)|/127 with sigma
    chosen so activations stay O(1): sigma ~ sqrt(3 / fan_in) / 0.8); norms 1 + small noise; embeddings N(0, 1)."""
    lib = capi.load_library()
    dev = torch.device(device)
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)

    def q8(n, k):
        nb = n * k // 32
        sigma = scale_sigma if scale_sigma is not None else float(np.sqrt(3.0 / k) / 0.8)
        qs = torch.randint(-127, 128, (nb, 32), dtype=torch.int8, device=dev, generator=gen)
        d = (torch.randn((nb, 1), device=dev, generator=gen).abs() * (sigma / 127.0)).to(torch.float16)
        raw = torch.empty((nb, 34), dtype=torch.uint8, device=dev)
        raw[:, :2] = d.view(torch.uint8)
        raw[:, 2:] = qs.view(torch.uint8)
        planar = torch.empty(lib.lhip_q8_0_planar_nbytes(n, k), dtype=torch.uint8, device=dev)
        capi.check(lib.lhip_q8_0_repack(raw.data_ptr(), planar.data_ptr(), n, k, _s()), "lhip_q8_0_repack")
        torch.cuda.synchronize()
        return Q8Weight(planar, n, k)

    def norm():
        return 1.0 + 0.05 * torch.randn(cfg.dim, device=dev, generator=gen)

    w = {"embed": torch.randn((cfg.vocab, cfg.dim), device=dev, generator=gen), "out_norm": norm(),
         "lm_head": q8(cfg.vocab, cfg.dim)}
    for i in range(cfg.layers):
        w[f"{i}.attn_norm"], w[f"{i}.ffn_norm"] = norm(), norm()
        w[f"{i}.qkv"] = q8(cfg.qkv_rows, cfg.dim)
        w[f"{i}.o"] = q8(cfg.dim, cfg.dim)
        w[f"{i}.gate_up"] = q8(2 * cfg.ffn, cfg.dim)
        w[f"{i}.down"] = q8(cfg.dim, cfg.ffn)
    return w
