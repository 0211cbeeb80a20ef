#!/usr/bin/env python3
"""Benchmark of the Q8_0 decode hot path on one MI355X.

Workload ("llama3_8b_q8_0_decode_projection_set"): one step is one decode
token's worth of Q8_0 projections of Llama-3-8B at batch 1 — 32 layers x
{q, k, v, o, gate, up, down} plus lm_head, 225 matvecs over 7.97 GB of
distinct weights (so every launch streams from HBM, not from cache), f32
activations ~N(0,1), random weights: quants U{-127..127}, block scales
|N(0,0.02)|/127 in f16.  Inputs are resident in HBM before timing starts.
The sibling projections that read the same activations (q|k|v, gate|up) go
out as one grouped launch each, from their separate weight buffers into their
separate outputs, so a step is 129 launches; the 225-launch form is timed
beside it.

Prints ONE JSON line: whole-step GB/s of algorithmic bytes
(N*K*34/32 + 4K + 4N per matvec), per-shape GB/s, the roofline fraction of the
matvec kernel against 8 TB/s, and the CPU baseline (the oracle's restatement of
the reference's dequantise-then-f32-matmul path) timed on this host.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# HBM bytes per launch (FETCH_SIZE scaled by the copy-kernel factor 2.0, plus WRITE_SIZE) of each section's dominant
# kernel (for the MoE layer: of the layer's launches at T = 64), copied from the committed rocprofv3 counter
# summaries named beside them, where the figure is written with its digits in groups of three followed by " B";
# tests/test_bench_cli.py checks that each file still holds its figure, so a refreshed profile and this table cannot
# drift apart unnoticed.
TRAFFIC = {
    "gemv": (138310222, "profiles/q8_gemv_decode_projection_set.md"),
    "gemm": (725655654, "profiles/q8_gemm_prefill_set.md"),
    "moe_t64": (443523277, "profiles/mxfp4_moe_layer.md"),
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="decode_projection_set",
                    choices=["decode_projection_set", "prefill_gemm", "moe", "rows_f32", "issue_rates"],
                    help="decode_projection_set (default, the headline metric), prefill_gemm (the Q8_0 prefill GEMM set), "
                         "moe (the MXFP4 expert layer)")
    ap.add_argument("--layers", type=int, default=None, help="override the 32 layers (debug only; marks the line)")
    ap.add_argument("--cell", default=None, help="prefill_gemm only: one cell, NAME:M (e.g. gate/up:2048), for a counter "
                                                  "pass that must tell one call's launches apart; prints that cell only")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true", help="skip the end-to-end Llama-3-8B decode section")
    ap.add_argument("--no-sections", action="store_true", help="skip the prefill-GEMM and MoE sections of the default line")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    return ap.parse_args()


def make_weight(torch, lib, capi, n, k, gen, dev):
    """Random Q8_0 weight built on the device as raw GGUF blocks, then repacked
    by the library (the same path a loader takes)."""
    nb = n * k // 32
    qs = torch.randint(-127, 128, (nb, 32), dtype=torch.int8, device=dev, generator=gen)
    d = (torch.randn((nb, 1), device=dev, generator=gen).abs() * (0.02 / 127.0)).to(torch.float16)
    raw = torch.empty((nb, 34), dtype=torch.uint8, device=dev)
    raw[:, :2] = d.view(torch.uint8)
    raw[:, 2:] = qs.view(torch.uint8)
    planar = torch.empty(lib.lhip_q8_0_planar_nbytes(n, k), dtype=torch.uint8, device=dev)
    capi.check(lib.lhip_q8_0_repack(raw.data_ptr(), planar.data_ptr(), n, k,
                                    torch.cuda.current_stream().cuda_stream), "lhip_q8_0_repack")
    torch.cuda.synchronize()
    return planar


def cpu_baseline(seconds: float):
    """Dequantise once (untimed, as the reference's loader does), then time the
    f32 matvecs of ONE layer's seven projections, single-threaded like the
    reference's matrixmultiply configuration, for about `seconds`."""
    import numpy as np

    from luminal_amd import synth
    from oracle import cpu_oracle

    names = ["q", "k", "v", "o", "gate", "up", "down"]
    ws, xs, outs, q8_bytes = [], [], [], 0
    for i, nm in enumerate(names):
        n, k = synth.LLAMA3_8B_PROJ[nm]
        qs, d = synth.q8_0_random(n, k, seed=900 + i)
        w = cpu_oracle.q8_0_dequant(synth.q8_0_raw_blocks(qs, d), n * k).reshape(n, k)
        ws.append(w)
        xs.append(synth.activations(1, k, seed=950 + i))
        outs.append(np.empty((1, n), np.float32))
        q8_bytes += synth.q8_0_gemv_bytes(n, k)

    def one_pass(threads):
        for w, x, o in zip(ws, xs, outs):
            cpu_oracle.matmul_fast_f32(x, w, threads=threads, out=o)

    def timed(threads, budget):
        one_pass(threads)  # warm
        t0 = time.perf_counter()
        reps = 0
        while True:
            one_pass(threads)
            reps += 1
            if time.perf_counter() - t0 >= budget:
                break
        return (time.perf_counter() - t0) / reps, reps

    t1, reps1 = timed(1, seconds * 0.7)
    ncpu = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16))
    tn, repsn = timed(ncpu, seconds * 0.3)
    return {
        "value": round(q8_bytes / t1 / 1e9, 3),
        "unit": "GB/s",
        "cores": 1,
        "kind": "port",
        "sample": (f"one layer's 7 projections (q,k,v,o,gate,up,down; {q8_bytes} Q8_0-equivalent bytes, "
                   f"f32 weights after load-time dequant), {reps1} passes, {t1 * 1e3:.1f} ms/pass single-threaded"),
        "all_cores": {"value": round(q8_bytes / tn / 1e9, 3), "cores": ncpu, "passes": repsn,
                      "ms_per_pass": round(tn * 1e3, 2)},
    }


MFMA_BF16_PEAK_TFLOPS = 2500.0
MFMA_FP8_PEAK_TFLOPS = 5000.0
MFMA_FP4_PEAK_TFLOPS = 10100.0


def _event_us(torch, fn, reps, warm=1, repeats=1):
    """Average time of one call over `reps` back-to-back calls (HIP events on torch's current stream), after `warm`
    untimed calls; with `repeats` > 1 the best of that many such averages (the clocks of an idle GPU take a few
    milliseconds to come up, which a cell of a few short launches otherwise pays for)."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    best = None
    for _ in range(repeats):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / reps
        best = us if best is None or us < best else best
    return best


def bench_issue_rates(args):
    """Issue rates of the matrix instructions the GEMMs use and of the fp4 -> bf16 conversion: register-only loops
    (lhip_issue_rate_probe), one and two waves per SIMD; cycles per instruction from the kernel's own cycle counter,
    the shader clock from that counter against the 100 MHz wall clock, TFLOP/s from HIP events."""
    import torch

    from luminal_amd import capi

    lib = capi.load_library()
    dev = torch.device("cuda:0")
    capi.check(lib.lhip_init(0), "lhip_init")
    stream = torch.cuda.current_stream().cuda_stream
    kinds = [("v_mfma_f32_32x32x16_bf16", 0, 4, 2 * 32 * 32 * 16), ("v_mfma_f32_16x16x32_bf16", 1, 8, 2 * 16 * 16 * 32),
             ("v_mfma_scale_f32_16x16x128_f8f6f4 fp8 x fp8", 2, 8, 2 * 16 * 16 * 128),
             ("v_mfma_scale_f32_16x16x128_f8f6f4 fp8 x fp4", 3, 8, 2 * 16 * 16 * 128),
             ("v_mfma_scale_f32_16x16x128_f8f6f4 fp4 x fp4", 4, 8, 2 * 16 * 16 * 128),
             ("v_mfma_scale_f32_16x16x128_f8f6f4 fp6 x fp4", 5, 8, 2 * 16 * 16 * 128),
             ("v_cvt_scalef32_pk_bf16_fp4", 6, 8, 0)]
    iters = 20000
    rows = {}
    for name, kind, per_iter, flop in kinds:
        for wps in (1, 2):
            out = torch.zeros(2 * 1024 * wps, dtype=torch.int64, device=dev)

            def run():
                capi.check(lib.lhip_issue_rate_probe(kind, iters, wps, out.data_ptr(), stream), "lhip_issue_rate_probe")

            us = _event_us(torch, run, 3)
            torch.cuda.synchronize()
            o = out.view(-1, 2).double()
            cycles, ticks = float(o[:, 0].median()), float(o[:, 1].median())
            n_inst = iters * per_iter  # per wave
            clock_ghz = cycles / ticks * 0.1
            # a SIMD's instruction stream is the wps waves' together: the launch's duration in shader cycles over the
            # instructions the SIMD issued (the launch overhead of ~2 us in ~1 ms is inside the figure)
            row = {"cycles_per_instruction_per_simd": round(us * 1e3 * clock_ghz / (n_inst * wps), 2),
                   "one_wave_cycles_per_own_instruction": round(cycles / n_inst, 2),
                   "shader_clock_ghz": round(clock_ghz, 3), "launch_us": round(us, 1)}
            if flop:
                row["tflops"] = round(1024.0 * wps * n_inst * flop / us / 1e6, 1)
            rows[f"{name}, {wps} wave(s) per SIMD"] = row
    return {"metric": "issue rates of the matrix and conversion instructions (calibration)", "unit": "cycles per instruction per SIMD",
            "n_gpus": 1, "data": "synthetic", "config": {"workload": "issue_rates", "iters": iters,
                                                         "independent_instructions_per_iteration": 8},
            "rates": rows}


def bench_rows_f32(args):
    """The reference's own operator on a prompt: QuantizedMatmul<f32> (lhip_q8_0_matmul_f32) with M in
    {16, 128, 512} activation rows over the Llama-3-8B weight shapes, f32 in and out at f32 accuracy.  From six
    rows on the library runs it on the matrix cores (codes as exact bf16, x as three bf16 limbs: three products per
    step, the block scale applied to each block's f32 sum; weights streamed once per 64 rows); the one-matvec-per-
    row-group form the reference's launch corresponds to is timed beside it on the 128-row gate shape.  A step is one pass over all shapes at all three M."""
    import torch

    from luminal_amd import capi

    lib = capi.load_library()
    dev = torch.device("cuda:0")
    capi.check(lib.lhip_init(0), "lhip_init")
    gen = torch.Generator(device=dev)
    gen.manual_seed(0x5EED + 5)
    stream = torch.cuda.current_stream().cuda_stream
    shapes = {"q/o": (4096, 4096), "k/v": (1024, 4096), "gate/up": (14336, 4096), "down": (4096, 14336)}
    ms_list = (16, 128, 512)
    bufs = {nm: [make_weight(torch, lib, capi, n, k, gen, dev) for _ in range(4)] for nm, (n, k) in shapes.items()}
    xs = {(m, k): torch.randn((m, k), device=dev, generator=gen) for m in ms_list for k in (4096, 14336)}
    ys = {(m, n): torch.empty((m, n), device=dev) for m in ms_list for n in (4096, 1024, 14336)}

    def run(nm, m, b):
        n, k = shapes[nm]
        capi.check(lib.lhip_q8_0_matmul_f32(b.data_ptr(), xs[(m, k)].data_ptr(), ys[(m, n)].data_ptr(), m, n, k, stream),
                   "lhip_q8_0_matmul_f32")

    def step():
        for nm in shapes:
            for m in ms_list:
                run(nm, m, bufs[nm][0])

    flops_step = sum(2.0 * m * n * k for (n, k) in shapes.values() for m in ms_list)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = {}
    for nm, (n, k) in shapes.items():
        for m in ms_list:
            us = _event_us(torch, lambda: [run(nm, m, b) for b in bufs[nm]], 3, warm=1, repeats=3) / len(bufs[nm])
            passes = (m + 63) // 64
            per[f"{nm} M={m}"] = {"us": round(us, 1), "tflops": round(2.0 * m * n * k / us / 1e6, 1),
                                  "weight_gbs": round(passes * n * k * 34 / 32 / us / 1e3, 1)}
    # the matvec form (a launch shape given: never the matrix-core form) on gate at 128 rows
    n, k, m = 14336, 4096, 128
    b = bufs["gate/up"][0]
    mv_us = _event_us(torch, lambda: capi.check(lib.lhip_q8_0_matmul_f32_cfg(
        b.data_ptr(), xs[(m, k)].data_ptr(), ys[(m, n)].data_ptr(), m, n, k, 2, 4, 4, 4, stream), "cfg"), 3)
    g = per["gate/up M=128"]
    print(json.dumps({
        "metric": "Q8_0 f32 matmul operator with several activation rows (f32-exact on bf16 MFMA): TFLOP/s, 1 GPU",
        "value": round(flops_step / (wall / args.steps) / 1e12, 1), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall * 1e3 / args.steps, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 codes as bf16 x f32 activations as three bf16 limbs, three products per step, block scales and sums in f32, f32 out",
        "data": "synthetic", "config": {"workload": "llama3_8b_q8_0_f32_rows_set", "m": list(ms_list)},
        "per_shape": per, "matvec_form_gate_m128_us": round(mv_us, 1),
        "roofline": {"bound": "mfma", "kernel": "lhip::q8_gemm_skinny_kernel<4, *, 8, float> (gate/up, M=128: two passes of 64 rows in one launch)",
                     "achieved": round(3 * g["tflops"], 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(3 * g["tflops"] / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                     "note": "achieved counts the three bf16 products issued per useful multiply-add"}}))


def cpu_baseline_gemm(seconds: float):
    """The reference's CPU path for the prefill GEMM at M = 128 (the only M the plan of record times on the host):
    dequantise once, then the f32 matmul of the q/o shape (4096 x 4096), single-threaded like the reference's
    matrixmultiply configuration, and on all host cores."""
    import numpy as np

    from luminal_amd import synth
    from oracle import cpu_oracle

    n, k, m = 4096, 4096, 128
    qs, d = synth.q8_0_random(n, k, seed=910)
    w = cpu_oracle.q8_0_dequant(synth.q8_0_raw_blocks(qs, d), n * k).reshape(n, k)
    x = synth.activations(m, k, seed=911)
    out = np.empty((m, n), np.float32)

    def timed(threads, budget):
        cpu_oracle.matmul_fast_f32(x, w, threads=threads, out=out)
        t0 = time.perf_counter()
        reps = 0
        while True:
            cpu_oracle.matmul_fast_f32(x, w, threads=threads, out=out)
            reps += 1
            if time.perf_counter() - t0 >= budget:
                break
        return (time.perf_counter() - t0) / reps, reps

    fl = 2.0 * m * n * k
    t1, r1 = timed(1, seconds * 0.7)
    ncpu = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16))
    tn, rn = timed(ncpu, seconds * 0.3)
    return {"value": round(fl / t1 / 1e12, 5), "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"q/o shape 4096 x 4096 at M = 128, f32 weights after load-time dequant, {r1} passes, "
                      f"{t1 * 1e3:.1f} ms/pass single-threaded",
            "all_cores": {"value": round(fl / tn / 1e12, 5), "cores": ncpu, "passes": rn, "ms_per_pass": round(tn * 1e3, 2)}}


def bench_prefill_gemm(args, cpu_seconds=None):
    """Prefill GEMM set: the seven Llama-3-8B weight shapes in Q8_0 against bf16 activations,
    M in {128, 512, 2048}, f32 accumulation, bf16 output.  A step is one pass over all shapes at
    all three M; weights rotate over distinct buffers.  Returns the section (a dict)."""
    import torch

    from luminal_amd import capi, synth

    lib = capi.load_library()
    dev = torch.device("cuda:0")
    capi.check(lib.lhip_init(0), "lhip_init")
    gen = torch.Generator(device=dev)
    gen.manual_seed(0x5EED + 2)
    stream = torch.cuda.current_stream().cuda_stream
    shapes = {"q/o": (4096, 4096), "k/v": (1024, 4096), "gate/up": (14336, 4096), "down": (4096, 14336),
              "lm_head": (128256, 4096)}
    ms_list = (128, 512, 2048)
    if getattr(args, "cell", None):
        cell_name, cell_m = args.cell.rsplit(":", 1)
        shapes, ms_list = {cell_name: shapes[cell_name]}, (int(cell_m),)
    bufs, xs, ys = {}, {}, {}
    rotate_bytes = 512 << 20  # twice the 256 MB last-level cache: every launch of a rotation streams from HBM
    for nm, (n, k) in shapes.items():
        nbuf = max(1, -(-rotate_bytes // (n * k * 34 // 32)))
        bufs[nm] = [make_weight(torch, lib, capi, n, k, gen, dev) for _ in range(nbuf)]
    for m in ms_list:
        for k in (4096, 14336):
            xs[(m, k)] = torch.randn((m, k), device=dev, generator=gen).to(torch.bfloat16)
        for n in (4096, 1024, 14336, 128256):
            ys[(m, n)] = torch.empty((m, n), dtype=torch.bfloat16, device=dev)

    def run(nm, m, b):
        n, k = shapes[nm]
        st = lib.lhip_q8_0_matmul_bf16(b.data_ptr(), xs[(m, k)].data_ptr(), ys[(m, n)].data_ptr(), m, n, k, stream)
        if st:
            capi.check(st, "lhip_q8_0_matmul_bf16")

    def step():
        for nm in shapes:
            for m in ms_list:
                run(nm, m, bufs[nm][0])

    flops_step = sum(2.0 * m * n * k for (n, k) in shapes.values() for m in ms_list)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per = {}
    for nm, (n, k) in shapes.items():
        for m in ms_list:
            us = _event_us(torch, lambda: [run(nm, m, b) for b in bufs[nm]], 3, warm=1, repeats=3) / len(bufs[nm])
            fl = 2.0 * m * n * k
            by = n * k * 34 // 32 + 2 * m * k + 2 * m * n
            per[f"{nm} M={m}"] = {"us": round(us, 1), "tflops": round(fl / us / 1e6, 1),
                                  "frac_mfma_bf16": round(fl / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
                                  "gbs": round(by / us / 1e3, 1), "frac_hbm": round(by / us / 1e3 / HBM_PEAK_GBS, 4)}
    if getattr(args, "cell", None):
        return {"metric": "Q8_0 prefill GEMM TFLOP/s (MFMA utilisation), 1 GPU", "config": {"cell": args.cell},
                "per_shape": per}
    # dominant kernel: q8_gemm_bf16_kernel<256, 128, 4, 2, 4, __bf16> on the M = 2048 gate/up shape (time and traffic of
    # the whole call: the kernel's two launches and the reduction between the K slices of the second)
    n, k, m = 14336, 4096, 2048
    us = _event_us(torch, lambda: [run("gate/up", m, b) for b in bufs["gate/up"]], 5, warm=1, repeats=3) / len(bufs["gate/up"])
    ach = 2.0 * m * n * k / us / 1e6
    value = flops_step / (wall / args.steps) / 1e12
    g128 = per["gate/up M=128"]
    out = {
        "metric": "Q8_0 prefill GEMM TFLOP/s (MFMA utilisation), 1 GPU", "value": round(value, 1), "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall * 1e3 / args.steps, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 codes as exact bf16 x bf16 activations on the matrix cores, block scales and sums in f32, bf16 out",
        "data": "synthetic",
        "config": {"workload": "llama3_8b_q8_0_prefill_gemm_set", "m": list(ms_list),
                   "weight_rotation": "every cell is timed over distinct weight buffers of at least 512 MB in all "
                                      f"({', '.join(f'{nm}: {len(b)}' for nm, b in bufs.items())} buffers)"},
        "per_shape": per,
        "roofline": {"bound": "mfma", "kernel": "lhip::q8_gemm_bf16_kernel<256, 128, 4, 2, 4, __bf16> (gate/up, M=2048: the call, "
                                                   "i.e. this kernel over three whole rounds of column tiles, the same kernel over two K "
                                                   "slices of the rest, and their sum)",
                     "achieved": round(ach, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(ach / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": TRAFFIC["gemm"][0],
                     "traffic_source": TRAFFIC["gemm"][1], "avg_launch_us": round(us, 1)},
        "roofline_m128": {"bound": "hbm", "kernel": "lhip::q8_gemm_skinny_kernel<8, *, 8, __bf16> (gate/up, M=128)",
                          "achieved": g128["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": g128["frac_hbm"],
                          "traffic": None}}
    if cpu_seconds:
        out["cpu_baseline"] = cpu_baseline_gemm(cpu_seconds)
    del bufs, xs, ys
    torch.cuda.empty_cache()
    return out


def cpu_baseline_moe(seconds: float):
    """The oracle's expert layer (exact dequantisation, then f32-input matmuls accumulated in f64) at T = 1 and on a
    sample of the T = 64 batch, one thread and all host cores (tokens dealt out over threads).  Eight experts are
    built (the work per token does not depend on which experts it is routed to)."""
    from concurrent.futures import ThreadPoolExecutor

    import numpy as np

    from luminal_amd import synth
    from oracle import cpu_oracle

    e, h, i, topk = 8, synth.MOE_HIDDEN, synth.MOE_INTER, synth.MOE_TOPK
    gu_c, gu_s = synth.mxfp4_random(e * 2 * i, h, seed=920)
    dn_c, dn_s = synth.mxfp4_random(e * h, i, seed=921)
    w_gu = cpu_oracle.mxfp4_dequant(synth.mxfp4_raw_blocks(gu_c, gu_s), gu_c.size).reshape(e, 2 * i, h)
    w_dn = cpu_oracle.mxfp4_dequant(synth.mxfp4_raw_blocks(dn_c, dn_s), dn_c.size).reshape(e, h, i)
    del gu_c, gu_s, dn_c, dn_s
    rng = np.random.default_rng(922)
    ncpu = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16") or 16))
    t_sample = ncpu  # tokens of the T = 64 batch that are run: one per thread in the all-cores leg
    x = cpu_oracle.bf16_bits_to_f32(cpu_oracle.f32_to_bf16_bits(rng.standard_normal((t_sample, h)).astype(np.float32)))
    sel, wts = cpu_oracle.moe_route(rng.standard_normal((t_sample, e)).astype(np.float32), topk)

    def run(rows, threads):
        if threads == 1:
            cpu_oracle.moe_forward(x[rows], w_gu, w_dn, sel[rows], wts[rows], act_bf16=True)
            return
        with ThreadPoolExecutor(threads) as ex:
            list(ex.map(lambda r: cpu_oracle.moe_forward(x[r:r + 1], w_gu, w_dn, sel[r:r + 1], wts[r:r + 1], act_bf16=True), rows))

    def timed(rows, threads, budget):
        t0 = time.perf_counter()
        reps = 0
        while True:
            run(rows, threads)
            reps += 1
            if time.perf_counter() - t0 >= budget:
                break
        return (time.perf_counter() - t0) / reps

    fl_tok = 199065600.0
    one = timed(np.arange(1), 1, seconds * 0.4)                  # T = 1, one thread
    allc = timed(np.arange(t_sample), ncpu, seconds * 0.6)       # t_sample tokens, one per thread
    return {"value": round(fl_tok / one / 1e12, 6), "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"T = 1: one token through its 4 experts, {one * 1e3:.0f} ms single-threaded (f64 accumulation); "
                      f"T = 64: {t_sample} of the 64 tokens, one per thread",
            "t1_us": round(one * 1e6, 0),
            "t64_all_cores": {"value": round(t_sample * fl_tok / allc / 1e12, 6), "cores": ncpu,
                              "us_for_64_tokens_extrapolated": round(allc * 64 / t_sample * 1e6, 0)}}


def bench_moe(args, cpu_seconds=None):
    """MoE workload: gpt-oss-style MXFP4 expert layer, H = I = 2880, 32 experts, top-4,
    T in {1, 64, 1024}; a step is one layer pass at each T (routing rotates so T = 1 streams
    different experts from HBM every pass).  Returns the section (a dict)."""
    import torch

    from luminal_amd import capi, synth
    from luminal_amd.moe import Mxfp4Weight, MoEExperts, route_topk

    lib = capi.load_library()
    dev = torch.device("cuda:0")
    capi.check(lib.lhip_init(0), "lhip_init")
    gen = torch.Generator(device=dev)
    gen.manual_seed(0x5EED + 3)
    E, H, I, K4 = synth.MOE_EXPERTS, synth.MOE_HIDDEN, synth.MOE_INTER, synth.MOE_TOPK

    def weight(n, k):  # random e2m1 codes, e8m0 exponents uniform in [-8, 0], built raw then repacked by the library
        nb = n * k // 32
        raw = torch.empty((nb, 17), dtype=torch.uint8, device=dev)
        raw[:, :16] = torch.randint(0, 256, (nb, 16), dtype=torch.uint8, device=dev, generator=gen)
        raw[:, 16] = torch.randint(119, 128, (nb,), dtype=torch.uint8, device=dev, generator=gen)
        planar = torch.empty(lib.lhip_mxfp4_planar_nbytes(n, k), dtype=torch.uint8, device=dev)
        capi.check(lib.lhip_mxfp4_repack(raw.data_ptr(), planar.data_ptr(), n, k,
                                         torch.cuda.current_stream().cuda_stream), "lhip_mxfp4_repack")
        torch.cuda.synchronize()
        return Mxfp4Weight(planar, n, k)

    layer = MoEExperts(weight(E * 2 * I, H), weight(E * H, I), E, H, I)
    cases = {}
    for T in (1, 64, 1024):
        x = torch.randn((T, H), device=dev, generator=gen).to(torch.bfloat16)
        routes = []
        for r in range(8):
            logits = torch.randn((T, E), device=dev, generator=gen)
            if T == 1:
                logits[0, 4 * r:4 * r + 4] += 100.0
            routes.append(route_topk(logits, K4))
        cases[T] = (x, routes)
    it = [0]
    modes = {"exact": capi.LHIP_MOE_EXACT, "fast": capi.LHIP_MOE_FAST}

    def run(T, mode=capi.LHIP_MOE_EXACT):
        x, routes = cases[T]
        sel, wts = routes[it[0] % 8]
        it[0] += 1
        layer.process(x, sel, wts, mode)

    def step():
        for T in cases:
            run(T)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    errors = _moe_strict_errors(torch, layer, cases, modes)
    per = {}
    flops_step = 0.0
    for T in cases:
        touched = E if T >= 64 else K4
        by = touched * 13219200 + 2 * 2 * T * H
        fl = T * 199065600.0
        flops_step += fl
        for name, mode in modes.items():
            us = _event_us(torch, lambda: run(T, mode), 16, warm=4, repeats=3)
            row = {"us": round(us, 1), "gbs": round(by / us / 1e3, 1), "frac_hbm": round(by / us / 1e3 / HBM_PEAK_GBS, 4),
                   "tflops": round(fl / us / 1e6, 1), "strict_err": errors[(T, name)]}
            if name == "exact":  # one bf16 x bf16 product per multiply-add
                row["frac_mfma_bf16"] = round(fl / us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 5)
            else:                # two fp8 x fp4 products per multiply-add
                row["frac_mfma_fp4"] = round(fl / us / 1e6 / MFMA_FP4_PEAK_TFLOPS, 5)
                row["frac_mfma_fp8_two_pass"] = round(2 * fl / us / 1e6 / MFMA_FP8_PEAK_TFLOPS, 5)
            per[f"T={T} {name}"] = row
    t64, t1024, f1024 = per["T=64 exact"], per["T=1024 exact"], per["T=1024 fast"]
    out = {
        "metric": "MXFP4 MoE expert layer (H=I=2880, 32 experts, top-4): GB/s and TFLOP/s, 1 GPU",
        "value": round(flops_step / (wall / args.steps) / 1e12, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall * 1e3 / args.steps, 3), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None,
        "dtype": "default (exact): fp4 (e2m1, e8m0 block scales) weights expanded exactly to bf16 x bf16 activations, f32 "
                 "accumulate on v_mfma_f32_16x16x32_bf16, bf16 out; fast: raw fp4 x two fp8 halves of each activation on "
                 "v_mfma_scale_f32_16x16x128_f8f6f4",
        "data": "synthetic", "config": {"workload": "gpt_oss_style_mxfp4_moe_layer", "tokens": [1, 64, 1024],
                                        "modes": "value and roofline are the default (exact) mode; per_tokens has both"},
        "per_tokens": per,
        "strict_err_legend": "max |y-t| / max(|t|, 1e-3 rms(t)) against f64 on sampled tokens: act = SwiGLU activations "
                             "(bf16) vs f64 of x; down = f32 down rows vs f64 of the activations the GPU produced; "
                             "y_given_act = layer output vs f64 down projection + weighted sum of those activations; "
                             "y_independent = layer output vs f64 with the intermediate rounded to bf16 on its own "
                             "(differs wherever an activation lies within rounding error of a bf16 boundary)",
        "roofline": {"bound": "hbm", "kernel": "whole layer at T=64, exact mode (plan, 2 grouped GEMMs, combine)",
                     "achieved": t64["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": t64["frac_hbm"],
                     "traffic": TRAFFIC["moe_t64"][0], "traffic_source": TRAFFIC["moe_t64"][1]},
        "roofline_t1024_mfma": {"bound": "mfma", "kernel": "whole layer at T=1024, exact mode (bf16 matrix instruction)",
                                "achieved": t1024["tflops"], "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                                "frac": t1024["frac_mfma_bf16"], "traffic": None},
        "roofline_t1024_mfma_fast": {"bound": "mfma", "kernel": "whole layer at T=1024, fast mode (block-scaled fp8 x fp4)",
                                     "achieved": f1024["tflops"], "peak": MFMA_FP4_PEAK_TFLOPS, "unit": "TFLOP/s",
                                     "frac": f1024["frac_mfma_fp4"], "frac_of_fp8_two_pass": f1024["frac_mfma_fp8_two_pass"],
                                     "traffic": None}}
    if cpu_seconds:
        out["cpu_baseline"] = cpu_baseline_moe(cpu_seconds)
    del layer, cases
    torch.cuda.empty_cache()
    return out


def _moe_strict_errors(torch, layer, cases, modes, n_tokens=3):
    """The layer's strict element-wise error per T and mode, each matmul against f64 arithmetic of its own inputs
    (torch on the device; weights through lhip_mxfp4_dequant_f32, whose values are tested bit-exact) on a few tokens."""
    e, h, i = layer.e, layer.h, layer.i
    w_gu = layer.gu.dequantize().view(e, 2 * i, h)
    w_dn = layer.dn.dequantize().view(e, h, i)

    def rel(y, t):
        y, t = y.double().reshape(-1), t.double().reshape(-1)
        floor = 1e-3 * float(t.pow(2).mean().sqrt()) + 1e-300
        return float(((y - t).abs() / t.abs().clamp_min(floor)).max())

    out = {}
    for T, (x, routes) in cases.items():
        sel, wts = routes[0]
        topk = sel.shape[1]
        toks = sorted({0, T - 1, T // 2})[:n_tokens]
        for name, mode in modes.items():
            y = layer.process(x, sel, wts, mode)
            act_g, down_g = layer.intermediates()
            want_act, got_act, want_down, got_down, y_given, y_indep = [], [], [], [], [], []
            for t in toks:
                yg = torch.zeros(h, dtype=torch.float64, device=x.device)
                yi = torch.zeros(h, dtype=torch.float64, device=x.device)
                for s_ in range(topk):
                    ex = int(sel[t, s_])
                    r = t * topk + s_
                    gu = w_gu[ex].double() @ x[t].double()
                    g, u = gu[:i], gu[i:]
                    a = u * (g / (1.0 + torch.exp(-g)))
                    want_act.append(a)
                    got_act.append(act_g[r])
                    wd = w_dn[ex].double()
                    d_own = wd @ act_g[r].double()
                    want_down.append(d_own)
                    got_down.append(down_g[r])
                    yg += float(wts[t, s_]) * d_own
                    yi += float(wts[t, s_]) * (wd @ a.float().to(torch.bfloat16).double())
                y_given.append(yg)
                y_indep.append(yi)
            yt = torch.stack([y[t] for t in toks])
            out[(T, name)] = {"act": float(f"{rel(torch.stack(got_act), torch.stack(want_act)):.3g}"),
                              "down": float(f"{rel(torch.stack(got_down), torch.stack(want_down)):.3g}"),
                              "y_given_act": float(f"{rel(yt, torch.stack(y_given)):.3g}"),
                              "y_independent": float(f"{rel(yt, torch.stack(y_indep)):.3g}")}
    del w_gu, w_dn
    torch.cuda.empty_cache()
    return out


def llama_decode(torch):
    """End-to-end workload: random-weight Llama-3-8B, all linears Q8_0, norms and embeddings f32;
    512-token prefill (bf16 GEMM path), then 256 greedy batch-1 decode steps (f32 matvec path,
    one captured HIP graph per step, token and position stay on the device)."""
    import numpy as np

    from luminal_amd.llama import LLAMA3_8B, LlamaQ8, random_weights

    cfg = LLAMA3_8B
    w = random_weights(cfg, seed=4, device="cuda:0")
    eng = LlamaQ8(cfg, w, max_seq=1024)
    prompt = np.random.default_rng(0).integers(0, cfg.vocab, 512)
    eng.prefill(prompt, bf16=True)          # warm-up (allocates buffers)
    eager = eng.decode(8, use_graph=False).tolist()
    eng.reset()
    eng.prefill(prompt, bf16=True)
    replayed = eng.decode(8, use_graph=True).tolist()   # captures the decode graph
    if eager != replayed:
        raise SystemExit(f"bench.py: graph replay picked {replayed}, eager stepping {eager}")
    eng.reset()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eng.prefill(prompt, bf16=True)
    torch.cuda.synchronize()
    t_prefill = time.perf_counter() - t0
    t0 = time.perf_counter()
    toks = eng.decode(256, use_graph=True)
    torch.cuda.synchronize()
    t_decode = time.perf_counter() - t0
    weight_bytes = cfg.layers * sum(synth_bytes(n, k) for n, k in
                                    [(cfg.qkv_rows, cfg.dim), (cfg.dim, cfg.dim), (2 * cfg.ffn, cfg.dim),
                                     (cfg.dim, cfg.ffn)]) + synth_bytes(cfg.vocab, cfg.dim)
    ms = t_decode / 256 * 1e3
    # The same steps as one persistent launch each (lhip_decode_program_*): a measured alternative, not the default.
    alt = LlamaQ8(cfg, w, max_seq=1024)
    alt.persistent_decode = True
    alt.prefill(prompt, bf16=True)
    alt_first = alt.decode(8, use_graph=True).tolist()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    alt.decode(64, use_graph=True)
    torch.cuda.synchronize()
    t_alt = time.perf_counter() - t0
    program = {"tok_s": round(64 / t_alt, 1), "ms_per_token": round(t_alt / 64 * 1e3, 3), "decode_steps": 64,
               "first_8_tokens_equal": alt_first == eager,
               "timed_out": bool(alt._program.timed_out()) if alt._program is not None else None}
    if alt._program is not None:
        # where the time goes inside the one kernel: workgroup 0's clock per phase (wait for the phase's input
        # included), averaged over 8 eager steps and over the layers
        ticks = alt._program.trace(True)
        acc = None
        for _ in range(8):
            alt.decode_step()
            torch.cuda.synchronize()
            t = ticks.cpu().numpy().astype(np.float64)
            d = (t[1::2] - t[0::2]) / 100.0
            acc = d if acc is None else acc + d
        acc /= 8
        names = ["qkv", "attention", "merge", "o", "gate_up", "down"]
        program["phase_us_workgroup0"] = {nm: round(float(acc[i:6 * cfg.layers:6].mean()), 2) for i, nm in enumerate(names)}
        program["phase_us_workgroup0"]["lm_head"] = round(float(acc[-1]), 2)
        alt._program.trace(False)
    del alt
    # The output projection that merges the attention's key ranges itself (one launch fewer per layer): a measured
    # alternative as well.
    alt = LlamaQ8(cfg, w, max_seq=1024)
    alt.merge_in_o_proj = True
    alt.prefill(prompt, bf16=True)
    alt.decode(8, use_graph=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    alt.decode(64, use_graph=True)
    torch.cuda.synchronize()
    t_alt = time.perf_counter() - t0
    folded = {"tok_s": round(64 / t_alt, 1), "ms_per_token": round(t_alt / 64 * 1e3, 3), "decode_steps": 64}
    del alt
    return {"tok_s": round(256 / t_decode, 1), "ms_per_token": round(ms, 3), "persistent_program": program,
            "merge_in_o_proj": folded,
            "prefill_tokens": 512, "prefill_ms": round(t_prefill * 1e3, 2),
            "prefill_tok_s": round(512 / t_prefill, 1), "decode_steps": 256,
            "q8_0_weight_bytes_per_token": weight_bytes,
            "weight_stream_gbs": round(weight_bytes / (t_decode / 256) / 1e9, 1),
            "frac_hbm_peak": round(weight_bytes / (t_decode / 256) / 1e9 / HBM_PEAK_GBS, 4),
            "first_tokens": [int(t) for t in toks[:8].tolist()],
            "graph_replay_equals_eager_first_8": toks[:8].tolist() == eager}


def synth_bytes(n, k):
    return n * k * 34 // 32


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py: this build measures ONE GPU's share of the path (no collectives, no sharding); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.workload == "prefill_gemm":
        return print(json.dumps(bench_prefill_gemm(args, None if args.no_cpu_baseline else args.cpu_seconds)))
    if args.workload == "moe":
        return print(json.dumps(bench_moe(args, None if args.no_cpu_baseline else args.cpu_seconds)))
    if args.workload == "rows_f32":
        return bench_rows_f32(args)
    if args.workload == "issue_rates":
        return print(json.dumps(bench_issue_rates(args)))

    import torch

    from luminal_amd import capi, synth

    lib = capi.load_library()  # no fallback: raises if the HIP library is missing
    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    capi.check(lib.lhip_init(0), "lhip_init")
    gen = torch.Generator(device=dev)
    gen.manual_seed(0x5EED)

    layers = args.layers or synth.LLAMA3_8B_LAYERS
    layer_names = ["q", "k", "v", "o", "gate", "up", "down"]
    shapes = synth.LLAMA3_8B_PROJ

    weights = {nm: [] for nm in layer_names}
    for _ in range(layers):
        for nm in layer_names:
            n, k = shapes[nm]
            weights[nm].append(make_weight(torch, lib, capi, n, k, gen, dev))
    weights["lm_head"] = [make_weight(torch, lib, capi, *shapes["lm_head"], gen, dev)]

    x = {4096: torch.randn(4096, device=dev, generator=gen), 14336: torch.randn(14336, device=dev, generator=gen)}
    y = {nm: torch.empty(shapes[nm][0], device=dev) for nm in shapes}
    stream = torch.cuda.current_stream().cuda_stream

    def gemv(nm, wbuf):
        n, k = shapes[nm]
        st = lib.lhip_q8_0_matmul_f32(wbuf.data_ptr(), x[k].data_ptr(), y[nm].data_ptr(), 1, n, k, stream)
        if st:
            capi.check(st, "lhip_q8_0_matmul_f32")

    import ctypes as C

    def group(names, wbufs):
        """Argument block of one grouped launch: weights `names` (same K), each into its own output."""
        cnt = len(names)
        k = shapes[names[0]][1]
        return ((C.c_void_p * cnt)(*[b.data_ptr() for b in wbufs]),
                (C.c_void_p * cnt)(*[y[nm].data_ptr() for nm in names]),
                (C.c_int64 * cnt)(*[shapes[nm][0] for nm in names]), cnt, x[k].data_ptr(), k)

    def run_group(g):
        st = lib.lhip_q8_0_matvec_fused_f32(g[0], g[1], g[2], g[3], g[4], g[5], None, 0.0, None, 0, stream)
        if st:
            capi.check(st, "lhip_q8_0_matvec_fused_f32")

    plan = []  # per layer: (q|k|v), o, (gate|up), down
    for l in range(layers):
        plan.append((group(["q", "k", "v"], [weights["q"][l], weights["k"][l], weights["v"][l]]),
                     group(["o"], [weights["o"][l]]),
                     group(["gate", "up"], [weights["gate"][l], weights["up"][l]]),
                     group(["down"], [weights["down"][l]])))
    head = group(["lm_head"], [weights["lm_head"][0]])

    def step():
        for groups in plan:
            for g in groups:
                run_group(g)
        run_group(head)

    def step_ungrouped():
        for l in range(layers):
            for nm in layer_names:
                gemv(nm, weights[nm][l])
        gemv("lm_head", weights["lm_head"][0])

    launches = layers * 4 + 1
    step_bytes = layers * sum(synth.q8_0_gemv_bytes(*shapes[nm]) for nm in layer_names) \
        + synth.q8_0_gemv_bytes(*shapes["lm_head"])

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    gpu_ms = ev0.elapsed_time(ev1)
    ms_per_step = wall * 1e3 / args.steps
    value = step_bytes / (wall / args.steps) / 1e9

    # The same bytes as 225 separate matvec launches (one per weight).
    step_ungrouped()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_ungrouped()
    torch.cuda.synchronize()
    ungrouped = {"launches_per_step": layers * len(layer_names) + 1,
                 "gbs": round(step_bytes / ((time.perf_counter() - t0) / args.steps) / 1e9, 1)}

    # Per-shape rates: back-to-back launches rotating over that shape's distinct
    # weight buffers (lm_head alone is 558 MB, larger than the 256 MB last-level
    # cache), HIP events on the launch stream.
    per_shape = {}
    for nm in list(layer_names) + ["lm_head"]:
        bufs = weights[nm]
        reps = 20 if nm == "lm_head" else max(1, 128 // len(bufs))
        for b in bufs[:2]:
            gemv(nm, b)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            for b in bufs:
                gemv(nm, b)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (reps * len(bufs))
        nbytes = synth.q8_0_gemv_bytes(*shapes[nm])
        per_shape[nm] = {"n": shapes[nm][0], "k": shapes[nm][1], "us": round(us, 2),
                         "gbs": round(nbytes / us / 1e3, 1), "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
        if nm != "lm_head":
            # The same launch over ONE weight buffer again and again: it stays in the 256 MB last-level cache, so
            # this is the cache-resident rate, not an HBM figure.
            gemv(nm, bufs[0])
            torch.cuda.synchronize()
            e0.record()
            for _ in range(64):
                gemv(nm, bufs[0])
            e1.record()
            torch.cuda.synchronize()
            per_shape[nm]["cache_resident_us"] = round(e0.elapsed_time(e1) * 1e3 / 64, 2)

    for label, idx, names in (("q|k|v grouped", 0, ["q", "k", "v"]), ("gate|up grouped", 2, ["gate", "up"])):
        for groups in plan[:2]:
            run_group(groups[idx])
        torch.cuda.synchronize()
        reps = max(1, 128 // layers)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            for groups in plan:
                run_group(groups[idx])
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / (reps * layers)
        nbytes = sum(synth.q8_0_gemv_bytes(*shapes[nm]) for nm in names)
        per_shape[label] = {"n": [shapes[nm][0] for nm in names], "k": shapes[names[0]][1], "us": round(us, 2),
                            "gbs": round(nbytes / us / 1e3, 1), "frac_hbm": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}

    # Calibration: plain copy and read-only kernels of known size (1 GiB), for
    # scaling hardware byte counters and as the streaming rate of this part.
    cal_n = 1 << 30
    cal_src = torch.empty(cal_n, dtype=torch.uint8, device=dev).random_(0, 256, generator=gen)
    cal_dst = torch.empty(cal_n, dtype=torch.uint8, device=dev)
    cal_out = torch.zeros(1024, dtype=torch.int32, device=dev)
    calibration = {}
    for label, fn, moved in (
            ("copy_1GiB", lambda: lib.lhip_copy_bytes(cal_dst.data_ptr(), cal_src.data_ptr(), cal_n, stream), 2 * cal_n),
            ("read_1GiB", lambda: lib.lhip_read_bytes(cal_src.data_ptr(), cal_n, cal_out.data_ptr(), stream), cal_n)):
        fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(5):
            fn()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / 5
        calibration[label] = {"us": round(us, 1), "gbs": round(moved / us / 1e3, 1)}
    del cal_src, cal_dst

    # Roofline of the dominant kernel.  The gate|up grouped launches and lm_head run one kernel symbol,
    # q8_gemv_fused_kernel<2, 4, 4, false, 0> (2 rows x 4 slices of 1024 quants per step, 4 waves per workgroup,
    # one workgroup per CU, no prologue or epilogue): 33 of the step's 129 launches, 4.55 of its 7.98 GB and
    # about half of its time.  Its launches are replayed alone, in step order over the same distinct weights,
    # between two HIP events on the launch stream.
    dom_launches = layers + 1
    dom_bytes = layers * sum(synth.q8_0_gemv_bytes(*shapes[nm]) for nm in ("gate", "up")) \
        + synth.q8_0_gemv_bytes(*shapes["lm_head"])

    def dom_pass():
        for groups in plan:
            run_group(groups[2])
        run_group(head)

    dom_pass()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        dom_pass()
    e1.record()
    torch.cuda.synchronize()
    dom_us = e0.elapsed_time(e1) * 1e3 / (args.steps * dom_launches)
    achieved = (dom_bytes / dom_launches) / dom_us / 1e3  # GB/s
    roofline = {
        "bound": "hbm",
        "kernel": "lhip::q8_gemv_fused_kernel<2, 4, 4, false, 0>",
        "achieved": round(achieved, 1),
        "peak": HBM_PEAK_GBS,
        "unit": "GB/s",
        "frac": round(achieved / HBM_PEAK_GBS, 4),
        # HBM bytes per launch from rocprofv3 FETCH_SIZE + WRITE_SIZE (see profiles/): within 1 % of algorithmic
        "traffic": TRAFFIC["gemv"][0] if layers == 32 else None,
        "traffic_source": TRAFFIC["gemv"][1],
        "launches_per_step": dom_launches,
        "bytes_per_launch": round(dom_bytes / dom_launches),
        "avg_launch_us": round(dom_us, 3),
        "whole_step": {"achieved": round(step_bytes / (gpu_ms / args.steps) / 1e6, 1), "launches": launches,
                       "avg_launch_us": round(gpu_ms * 1e3 / (args.steps * launches), 3)},
    }

    out = {
        "metric": "Q8_0 GEMV HBM GB/s (% of peak) + Llama-3-8B Q8_0 decode tok/s, 1 GPU",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 weights x f32 activations, f32 accumulate",
        "data": "synthetic",
        "config": {
            "workload": "llama3_8b_q8_0_decode_projection_set" + ("" if layers == 32 else f"_DEBUG_{layers}_layers"),
            "batch": 1,
            "launches_per_step": launches,
            "bytes_per_step": step_bytes,
            "projection_tokens_per_s": round(args.steps / wall, 1),
        },
        "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "per_shape": per_shape,
        "one_launch_per_weight": ungrouped,
        "calibration": calibration,
        "roofline": roofline,
    }
    del weights
    torch.cuda.empty_cache()
    if not args.no_decode and layers == 32:
        out["llama3_8b_q8_0_decode"] = llama_decode(torch)
        torch.cuda.empty_cache()
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(args.cpu_seconds)
    if not args.no_sections and layers == 32:
        # configs 2 and 3 of the benchmark plan ride in the same line, each with its own roofline and CPU baseline
        sec = argparse.Namespace(steps=max(2, args.steps // 4), warmup=1)
        cpu_s = None if args.no_cpu_baseline else min(args.cpu_seconds, 8.0)
        out["prefill_gemm"] = bench_prefill_gemm(sec, cpu_s)
        out["moe"] = bench_moe(sec, cpu_s)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
