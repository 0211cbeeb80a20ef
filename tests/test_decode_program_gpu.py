"""The persistent decode program (lhip_decode_program_*): a decode step as one launch.  Its operations share their
arithmetic and reduction orders with the per-kernel fused path (lhip_q8_0_matvec_fused_f32,
lhip_attention_decode_f32), so the bar is equality of bits with that path, which the other test files hold against
the oracle; a direct comparison with the numpy oracle is made as well."""
import ctypes as C

import numpy as np
import pytest

torch = pytest.importorskip("torch")

from conftest import rel_err  # noqa: E402
from luminal_amd import capi, synth  # noqa: E402
from luminal_amd.llama import LlamaConfig, LlamaQ8  # noqa: E402
from luminal_amd.quantized import DecodeProgram, FusedMatvec, Q8Weight  # noqa: E402
from oracle import llama_oracle as lo  # noqa: E402
from test_llama_gpu import build_model, empty_cache  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def bits(t):
    return t.view(torch.int32)


def weight(n, k, seed):
    qs, d = synth.q8_0_random(n, k, seed=seed, scale_sigma=float(np.sqrt(3.0 / k) / 0.8))
    return Q8Weight.from_raw(synth.q8_0_raw_blocks(qs, d), n, k, DEV)


# (n, k): step shapes 1x1 (k = 1024, 3072), 1x2, 1x4 / 2x4, 1x7 (k = 7168, 14336); fewer row groups than waves,
# odd n, a tall matrix that takes two rows per wave
@pytest.mark.parametrize("n,k", [(4096, 4096), (6144, 4096), (4096, 14336), (300, 1024), (1001, 3072), (5000, 2048),
                                 (37, 7168), (20000, 4096), (40000, 1024)])
@pytest.mark.parametrize("norm", [False, True])
def test_single_matvec_phase_equals_the_fused_matvec(n, k, norm):
    w = weight(n, k, n + k)
    torch.manual_seed(n)
    x = torch.randn(k, device=DEV)
    g = (1 + 0.1 * torch.randn(k, device=DEV)) if norm else None
    pos = torch.zeros(1, dtype=torch.int32, device=DEV)
    y_ref = torch.empty(n, device=DEV)
    FusedMatvec([w], [y_ref], norm_weight=g, eps=1e-5).run(x)
    y = torch.full((n,), float("nan"), device=DEV)
    prog = DecodeProgram(pos=pos).matvec(w, x, y, norm_weight=g, eps=1e-5).build()
    prog.run()
    torch.cuda.synchronize()
    assert not prog.timed_out()
    assert torch.equal(bits(y), bits(y_ref))


def test_chain_of_phases_with_every_epilogue_equals_the_fused_matvecs():
    """h -> (norm) gate|up + SwiGLU -> down + residual -> (norm) head, twice over, as 6 phases of one launch."""
    d, f, v = 2048, 3072, 1500
    w_gu, w_down, w_head = weight(2 * f, d, 1), weight(d, f, 2), weight(v, d, 3)
    torch.manual_seed(0)
    g1, g2 = 1 + 0.1 * torch.randn(d, device=DEV), 1 + 0.1 * torch.randn(d, device=DEV)
    h0 = torch.randn(d, device=DEV)
    pos = torch.zeros(1, dtype=torch.int32, device=DEV)

    def buffers():
        return h0.clone(), torch.empty(f, device=DEV), torch.empty(v, device=DEV), torch.empty(v, device=DEV)

    h, act, l1, l2 = buffers()
    for logits in (l1, l2):
        FusedMatvec([w_gu], [act], norm_weight=g1, eps=1e-5, epilogue=FusedMatvec.EPI_SWIGLU).run(h)
        FusedMatvec([w_down], [h], residual=h, epilogue=FusedMatvec.EPI_ADD).run(act)
        FusedMatvec([w_head], [logits], norm_weight=g2, eps=1e-5).run(h)
    hp, actp, l1p, l2p = buffers()
    prog = DecodeProgram(pos=pos)
    for logits in (l1p, l2p):
        prog.matvec(w_gu, hp, actp, norm_weight=g1, eps=1e-5, epilogue=FusedMatvec.EPI_SWIGLU)
        prog.matvec(w_down, actp, hp, residual=hp, epilogue=FusedMatvec.EPI_ADD)
        prog.matvec(w_head, hp, logits, norm_weight=g2, eps=1e-5)
    prog.build().run()
    torch.cuda.synchronize()
    assert not prog.timed_out()
    for got, want in ((hp, h), (actp, act), (l1p, l1), (l2p, l2)):
        assert torch.equal(bits(got), bits(want))
    # a second run starts from the h the first one left behind: the program holds no state of its own
    for logits in (l1, l2):
        FusedMatvec([w_gu], [act], norm_weight=g1, eps=1e-5, epilogue=FusedMatvec.EPI_SWIGLU).run(h)
        FusedMatvec([w_down], [h], residual=h, epilogue=FusedMatvec.EPI_ADD).run(act)
        FusedMatvec([w_head], [logits], norm_weight=g2, eps=1e-5).run(h)
    prog.run()
    torch.cuda.synchronize()
    assert torch.equal(bits(l2p), bits(l2)) and torch.equal(bits(hp), bits(h))


CONFIGS = [LlamaConfig(vocab=1000, dim=1024, layers=3, q_heads=8, kv_heads=2, ffn=2048),      # head_dim 128, G = 4
           LlamaConfig(vocab=700, dim=1024, layers=2, q_heads=16, kv_heads=2, ffn=1024),      # head_dim 64, G = 8
           LlamaConfig(vocab=515, dim=2048, layers=2, q_heads=16, kv_heads=16, ffn=7168)]     # G = 1, k = 7168


@pytest.mark.parametrize("cfg", CONFIGS, ids=["g4_hd128", "g8_hd64", "g1_hd128_k7168"])
def test_decode_steps_equal_the_per_kernel_path_bit_for_bit(oracle, cfg):
    eng, wf = build_model(oracle, cfg, seed=cfg.dim + cfg.ffn, max_seq=96)
    eng.persistent_decode = True
    ref = LlamaQ8(cfg, eng.w, 96, DEV)
    prompt = [int(t) for t in np.random.default_rng(1).integers(0, cfg.vocab, 70)]  # attention over > 1 tile of keys
    for e in (eng, ref):
        e.prefill(prompt)
    kc, vc = empty_cache(cfg), empty_cache(cfg)
    lo.forward(cfg, wf, prompt, kc, vc, 0)
    for step in range(5):
        tok = int(ref.tok_i.item())
        assert int(eng.tok_i.item()) == tok
        a, b = eng.decode_step(), ref.decode_step()
        assert eng._program is not None and ref._program is None
        assert torch.equal(bits(a), bits(b)), step
        want = lo.forward(cfg, wf, [tok], kc, vc, len(prompt) + step)[0]
        # logits after several layers and a 70-token context: the per-kernel path, whose bits these are, sits at
        # 2.3e-3 on the worst of these steps under the floor-1e-3-rms metric
        assert rel_err(a.cpu().numpy(), want) < 4e-3, step
    # the caches the two paths wrote agree as well
    for i in range(cfg.layers):
        assert torch.equal(bits(eng.k_cache[i]), bits(ref.k_cache[i])) and torch.equal(bits(eng.v_cache[i]), bits(ref.v_cache[i]))
    assert not eng._program.timed_out()


def test_llama3_8b_layer_dimensions_and_graph_replay(oracle):
    cfg = LlamaConfig(vocab=2048, dim=4096, layers=2, q_heads=32, kv_heads=8, ffn=14336)
    eng, _ = build_model(oracle, cfg, seed=31, max_seq=64)
    eng.persistent_decode = True
    ref = LlamaQ8(cfg, eng.w, 64, DEV)
    prompt = list(range(3, 23))
    for e in (eng, ref):
        e.prefill(prompt)
    for step in range(3):
        assert torch.equal(bits(eng.decode_step()), bits(ref.decode_step())), step
    assert eng._program is not None and not eng._program.timed_out()
    # replayed from a graph, with eager work and synchronisation between the replays
    eng.reset()
    eng.prefill(prompt)
    eager = eng.decode(8, use_graph=False).cpu().numpy()
    eng.reset()
    eng.prefill(prompt)
    graphed = eng.decode(8, use_graph=True).cpu().numpy()
    ref.reset()
    ref.prefill(prompt)
    assert np.array_equal(eager, graphed) and np.array_equal(eager, ref.decode(8, use_graph=False).cpu().numpy())
    assert not eng._program.timed_out()


def test_create_argument_errors():
    lib = capi.load_library()
    w = weight(64, 1024, 1)
    x, y = torch.zeros(1024, device=DEV), torch.zeros(64, device=DEV)
    pos = torch.zeros(1, dtype=torch.int32, device=DEV)
    handle = C.c_void_p()

    def create(op, heads=(0, 0, 0, 0)):
        arr = (capi.DecodeOp * 1)(op)
        return lib.lhip_decode_program_create(arr, 1, *heads, 0.0, pos.data_ptr(), C.byref(handle))

    def mv(**kw):
        base = dict(type=0, epilogue=0, planar=w.planar.data_ptr(), n=64, k=1024, x=x.data_ptr(), y=y.data_ptr(),
                    norm_weight=None, eps=0.0, residual=None, k_cache=None, v_cache=None)
        base.update(kw)
        return capi.DecodeOp(**base)

    assert create(mv(planar=None)) == capi.LHIP_ERR_NULL_PTR
    assert create(mv(k=1000)) == capi.LHIP_ERR_INVALID_SHAPE
    assert create(mv(k=512)) == capi.LHIP_ERR_UNSUPPORTED
    assert create(mv(k=15360)) == capi.LHIP_ERR_UNSUPPORTED
    assert create(mv(epilogue=1)) == capi.LHIP_ERR_NULL_PTR          # residual missing
    assert create(mv(epilogue=2, n=63)) == capi.LHIP_ERR_INVALID_SHAPE
    assert create(mv(epilogue=3)) == capi.LHIP_ERR_INVALID_SHAPE
    assert create(mv(x=x.data_ptr() + 4)) == capi.LHIP_ERR_MISALIGNED
    assert create(mv(type=7)) == capi.LHIP_ERR_INVALID_SHAPE
    att = capi.DecodeOp(1, 0, None, 0, 0, x.data_ptr(), y.data_ptr(), None, 0.0, None, x.data_ptr(), x.data_ptr())
    assert create(att, (6, 4, 128, 64)) == capi.LHIP_ERR_INVALID_SHAPE   # q heads not a multiple of kv heads
    assert create(att, (12, 4, 128, 64)) == capi.LHIP_ERR_UNSUPPORTED    # group of 3
    assert create(att, (8, 2, 96, 64)) == capi.LHIP_ERR_UNSUPPORTED      # head_dim
    assert handle.value is None
    assert lib.lhip_decode_program_run(None, None) == capi.LHIP_ERR_NULL_PTR
    assert lib.lhip_decode_program_destroy(None) == capi.LHIP_OK


@pytest.mark.parametrize("same_input", [False, True], ids=["independent_input", "input_is_the_residual"])
def test_residual_produced_by_a_phase_the_input_does_not_depend_on(same_input):
    """y1 = W1 x, then y2 = W2 z + y1 with z written before the launch (or z = y1): nothing orders phase 0 before the
    moment phase 1 requests its residual rows, so the residual has to travel as tagged words and be waited for like
    an input.  Small n: most workgroups have no row group and run ahead.  Bit-equal to the two fused launches, on
    several runs (each launch has tags of its own)."""
    d = 1024
    w1, w2 = weight(d, d, 41), weight(d, d, 42)
    torch.manual_seed(5)
    x, z = torch.randn(d, device=DEV), torch.randn(d, device=DEV)
    pos = torch.zeros(1, dtype=torch.int32, device=DEV)
    y1_ref, y2_ref = torch.empty(d, device=DEV), torch.empty(d, device=DEV)
    y1, y2 = torch.full((d,), float("nan"), device=DEV), torch.full((d,), float("nan"), device=DEV)
    prog = DecodeProgram(pos=pos).matvec(w1, x, y1)
    prog.matvec(w2, y1 if same_input else z, y2, residual=y1, epilogue=FusedMatvec.EPI_ADD).build()
    for run in range(4):
        x.normal_()
        FusedMatvec([w1], [y1_ref]).run(x)
        FusedMatvec([w2], [y2_ref], residual=y1_ref, epilogue=FusedMatvec.EPI_ADD).run(y1_ref if same_input else z)
        prog.run()
        torch.cuda.synchronize()
        assert not prog.timed_out()
        assert torch.equal(bits(y1), bits(y1_ref)) and torch.equal(bits(y2), bits(y2_ref)), run


def test_overwrite_is_refused_unless_its_readers_are_known_to_be_done():
    """A buffer may be overwritten by a phase only if every phase that read or wrote its old contents either is an
    ancestor of the overwriting phase's input or is followed, on that chain of inputs, by a phase that employs at
    least as many workgroups (a workgroup takes the phases in order): any other phase may still be running in some
    workgroup."""
    d = 1024
    w, w_tall = weight(d, d, 43), weight(4 * d, d, 44)
    pos = torch.zeros(1, dtype=torch.int32, device=DEV)
    a, c, e = (torch.zeros(d, device=DEV) for _ in range(3))
    b4 = torch.zeros(4 * d, device=DEV)
    # phase 0: a -> b4 on every workgroup of the grid; phase 1: a (before the launch) -> c on half of them; phase 2
    # reads c and overwrites b4.  The old writer, phase 0, is no ancestor of phase 2's input (c <- phase 1 <- a) and
    # phase 1 employs fewer workgroups than phase 0: some of phase 0's may still be storing.  Refused.
    prog = DecodeProgram(pos=pos).matvec(w_tall, a, b4).matvec(w, a, c).matvec(w_tall, c, b4)
    with pytest.raises(capi.LhipError) as err:
        prog.build()
    assert err.value.status == capi.LHIP_ERR_UNSUPPORTED
    # phase 0: a -> b; phase 1: b -> c; phase 2: c -> e; phase 3 reads e and overwrites b: reader (1) and writer (0)
    # of the old b are ancestors of phase 3's input.  Accepted, and equal to the fused launches.
    b = torch.zeros(d, device=DEV)
    torch.manual_seed(6)
    a.normal_()
    prog = DecodeProgram(pos=pos).matvec(w, a, b).matvec(w, b, c).matvec(w, c, e).matvec(w, e, b).build()
    prog.run()
    torch.cuda.synchronize()
    assert not prog.timed_out()
    rb, rc, re_, rb2 = (torch.empty(d, device=DEV) for _ in range(4))
    FusedMatvec([w], [rb]).run(a)
    FusedMatvec([w], [rc]).run(rb)
    FusedMatvec([w], [re_]).run(rc)
    FusedMatvec([w], [rb2]).run(re_)
    assert torch.equal(bits(b), bits(rb2)) and torch.equal(bits(c), bits(rc)) and torch.equal(bits(e), bits(re_))
