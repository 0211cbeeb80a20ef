// Q8_0 matrix-vector product for batch-1 decode:  y[n] = sum_k x[k] * W[n][k].
//
// Replaces the CUDA matvec of the reference
// (crates/luminal_cuda/src/quantized.rs:42-109): same arithmetic — quants
// converted to f32, multiplied with f32 activations, a partial sum per block
// scaled by float(d), f32 accumulation — on a layout and launch shape chosen
// for gfx950.
//
// The kernel is HBM-bound: 34/32 bytes per weight are read exactly once.
//   * Planar weights: every lane issues aligned 16-byte loads
//     (global_load_dwordx4) and one wave instruction covers 1 KiB of a row.
//   * One wavefront owns R consecutive rows.  Lane l owns quants
//     [16 l, 16 l + 16) of every 1024-wide slice of K, i.e. half a block, so
//     its scale is block (slice*32 + l/2).  The 16 activations of the slice
//     are loaded once and reused for all R rows.
//   * All loads of an unrolled step are issued before the first use, so a
//     wave keeps R*U 16-byte loads in flight per lane.
//   * Rows are reduced across the 64 lanes with DPP adds inside each row of
//     16 lanes and four readlanes; there are no atomics and the result does
//     not depend on the launch shape of other rows.
#include <hip/hip_fp16.h>
#include <limits.h>
#include <stdio.h>

#include "common.h"

namespace lhip {
// q8_gemm_skinny.hip: the matrix-core form with f32-accurate (head + tail bf16) operands for several activation rows.
bool q8_gemm_split_supports(int n, int k, const void *x, const void *y, bool f16);
lhip_status q8_gemm_split_launch(const int8_t *qs, const __half *ds, const void *x, void *y, int64_t m, int n, int k,
                                 bool f16, int splits, hipStream_t s, bool own_workspace = false, float *ws = nullptr,
                                 size_t ws_floats = 0);
size_t q8_gemm_split_workspace_floats(int64_t m, int n, int k);
// From this many activation rows on the plain operators take that form where the shape allows it: the weights are
// then streamed once per 64 rows instead of once per row.  The matrix-core form has a fixed cost (its launch, a
// reduce launch where K is sliced, staging) that a matvec pass over a small matrix stays under.  Measured, matvec
// against matrix cores, us: 1024 x 4096 at five rows 6.0 / 10.7; 4096 x 4096 at three rows 12.4 / 12.7, at four
// 15.8 / 12.4; 14336 x 4096 at two rows 20.6 / 21.5, at three 31.7 / 22.0; 128256 x 4096 at two rows 168 / 130.
static int split_min_rows(int64_t n, int64_t k) {
    const int64_t codes = n * k;
    return codes >= (int64_t{256} << 20) ? 2 : codes >= (int64_t{32} << 20) ? 3 : codes >= (int64_t{8} << 20) ? 4 : 6;
}


}  // namespace lhip

#include "q8_gemv_device.h"
#include "attention_decode_device.h"

namespace lhip {

// ---------------------------------------------------------------------------
// Fused decode variant of the pipelined kernel (batch 1):
//   * up to four weights that read the same activations run as one launch
//     (sibling projections q|k|v, gate|up): one launch overhead, one staging
//     of x per workgroup, and the short problems fill the tail of the long one;
//   * optional RMS-norm prologue: y = W (x * g) / sqrt(mean(x^2) + eps), the
//     sum of squares recomputed by every workgroup while it stages x, which
//     removes the norm launch and its round trip through HBM;
//   * epilogues: none, y = residual + W x, or SwiGLU on interleaved rows
//     (row 2j = gate_j, row 2j+1 = up_j, y[j] = up * gate * sigmoid(gate)).
// The per-row arithmetic is that of the plain kernel, so results agree with
// it bit for bit when no prologue or epilogue is selected.
// ---------------------------------------------------------------------------

constexpr int kMaxGroup = 4;

struct GemvGroup {
    const int8_t *qs[kMaxGroup];
    const unsigned short *ds[kMaxGroup];
    float *y[kMaxGroup];
    int n[kMaxGroup];
    int group_end[kMaxGroup];  // running total of row groups; unused entries hold INT_MAX
};

struct GemvFuse {
    const float *norm_w;    // PRO_NORM: gain of the RMS norm, K floats
    float eps;
    const float *residual;  // EPI_ADD: N floats (single weight only)
    // PRO_MERGE: the activations are the output of decode attention, formed here from the partial states its key
    // ranges left in the attention workspace (lhip_attention_decode_partial_f32) instead of being read from x
    const float *ws_ml;
    const float4 *ws_acc;
    const int *pos;
    int hkv, g, c4, n_splits, max_seq;  // KV heads, query heads per KV head, head_dim / 4, ranges of the workspace
};

enum { EPI_NONE = 0, EPI_ADD = 1, EPI_SWIGLU = 2 };
enum { PRO_NONE = 0, PRO_NORM = 1, PRO_MERGE = 2 };

// PRO_MERGE: float4 `src` of the attention output (head = src / c4, column src % c4) from the partial states, with
// the arithmetic and the order of additions of attention_merge_body: its SG = 256 / c4 sub-groups take the ranges
// sg, sg + SG, ... in a chain of fused multiply-adds each, and their sums are added in sub-group order (a sub-group
// without ranges adds zeros).  Up to eight ranges - every context of at most 2048 keys - are requested at once and
// cost one trip to memory; more than eight take a loop of dependent trips, which is correct and slow: callers that
// serve longer contexts keep the merge launch.
__device__ __forceinline__ float4 merged_attention_piece(const GemvFuse &f, int src, int n_active) {
    const int head = src / f.c4, c = src - head * f.c4;
    const int kvh = head / f.g, gq = head - kvh * f.g;
    const size_t base = static_cast<size_t>(kvh) * f.n_splits;
    auto slot_of = [&](int s) { return (base + min(s, n_active - 1)) * f.g + gq; };  // ranges past the last re-read it
    float4 a[8];
    float2 ml[8];
#pragma unroll
    for (int s = 0; s < 8; ++s) {  // every request before the first use
        const size_t slot = slot_of(s);
        ml[s] = *reinterpret_cast<const float2 *>(f.ws_ml + slot * 2);
        a[s] = f.ws_acc[slot * f.c4 + c];
    }
    float mx = -INFINITY;
#pragma unroll
    for (int s = 0; s < 8; ++s)
        if (s < n_active) mx = fmaxf(mx, ml[s].x);
    for (int s = 8; s < n_active; ++s) mx = fmaxf(mx, f.ws_ml[slot_of(s) * 2]);
    float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
    float den = 0.f;
    const int sgn = kDecThreads / f.c4;  // the merge kernel's sub-groups: 8 (head_dim 128) or 16 (head_dim 64)
#pragma unroll
    for (int sg = 0; sg < 8; ++sg) {
        const float w = sg < n_active ? dec_merge_weight(ml[sg].x, mx) : 0.f;
        float4 p = make_float4(fmaf(a[sg].x, w, 0.f), fmaf(a[sg].y, w, 0.f), fmaf(a[sg].z, w, 0.f), fmaf(a[sg].w, w, 0.f));
        float d = fmaf(ml[sg].y, w, 0.f);
        if (sgn == 8) {  // this sub-group's further ranges sg + 8, sg + 16, ... continue its chain
            for (int s = sg + 8; s < n_active; s += 8) {
                const size_t slot = slot_of(s);
                const float2 m2 = *reinterpret_cast<const float2 *>(f.ws_ml + slot * 2);
                const float4 a2 = f.ws_acc[slot * f.c4 + c];
                const float w2 = dec_merge_weight(m2.x, mx);
                d = fmaf(m2.y, w2, d);
                p.x = fmaf(a2.x, w2, p.x); p.y = fmaf(a2.y, w2, p.y); p.z = fmaf(a2.z, w2, p.z); p.w = fmaf(a2.w, w2, p.w);
            }
        }
        if (sg == 0) {
            num = p;
            den = d;
        } else {
            num.x += p.x; num.y += p.y; num.z += p.z; num.w += p.w;
            den += d;
        }
    }
    if (sgn == 16) {  // sub-groups 8..15 hold one range each
        for (int s = 8; s < 16; ++s) {
            float4 p = make_float4(0.f, 0.f, 0.f, 0.f);
            float d = 0.f;
            if (s < n_active) {
                const size_t slot = slot_of(s);
                const float2 m2 = *reinterpret_cast<const float2 *>(f.ws_ml + slot * 2);
                const float4 a2 = f.ws_acc[slot * f.c4 + c];
                const float w2 = dec_merge_weight(m2.x, mx);
                d = fmaf(m2.y, w2, 0.f);
                p = make_float4(fmaf(a2.x, w2, 0.f), fmaf(a2.y, w2, 0.f), fmaf(a2.z, w2, 0.f), fmaf(a2.w, w2, 0.f));
            }
            num.x += p.x; num.y += p.y; num.z += p.z; num.w += p.w;
            den += d;
        }
    }
    const float inv = 1.0f / den;
    return make_float4(num.x * inv, num.y * inv, num.z * inv, num.w * inv);
}

struct Located {
    const int8_t *qs;
    const unsigned short *ds;
    float *y;
    int n;
    int row0;
};

// Row group -> (weight, first row).  All operands are wave-uniform.
template <int R>
__device__ __forceinline__ Located locate(const GemvGroup &p, int gg) {
    // Two dependent reads of the argument buffer: the three boundaries at once, then the entries of the weight they
    // select (written as a chain of comparisons, this compiled to a branch and a one-word read per boundary).
    const int e0 = p.group_end[0], e1 = p.group_end[1], e2 = p.group_end[2];
    const int w = (gg >= e0) + (gg >= e1) + (gg >= e2);  // boundaries ascend; unused ones are INT_MAX
    const int before = w == 0 ? 0 : (w == 1 ? e0 : (w == 2 ? e1 : e2));
    return Located{p.qs[w], p.ds[w], p.y[w], p.n[w], (gg - before) * R};
}

template <int R, int S, int W, int PRO, int EPI>
__global__ __launch_bounds__(W * 64) void q8_gemv_fused_kernel(const int8_t *qs0, const unsigned short *ds0,
                                                               const float *__restrict__ x, const float *aux, int n0,
                                                               int end0, int k, int n_groups, int grid_blocks, float eps,
                                                               const GemvGroup p, const GemvFuse f) {
    // The scalar arguments in front (the first weight of the group, the activations and the sizes) reach the wave in
    // registers; the two structs are read from the argument buffer by the wave itself.  A wave whose first row group
    // lies in the first weight - every wave of a single-weight launch - requests its first weights without waiting
    // for that read, nor does the staging of the activations (grid_blocks is gridDim.x, which otherwise comes out of
    // the same buffer; eps repeats f.eps; aux is f.norm_w for a kernel with the norm prologue, else f.residual).
    // Fourteen dwords: what the hardware preloads.
    const float *norm_w = PRO == PRO_NORM ? aux : f.norm_w;
    const float *residual = PRO == PRO_NORM ? f.residual : aux;
    static_assert(EPI != EPI_SWIGLU || R % 2 == 0, "SwiGLU pairs live in one wave");
    constexpr bool NORM = PRO == PRO_NORM;
    extern __shared__ float4 xs4[];
    __shared__ float red[W];
    const unsigned lane = threadIdx.x & 63u;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wave_global = blockIdx.x * W + wave;
    const int total_waves = grid_blocks * W;

    const int chunks = k / (S * 1024);
    const int my_groups = wave_global < n_groups ? (n_groups - wave_global + total_waves - 1) / total_waves : 0;
    const int T = my_groups * chunks;

    // EPI_ADD: the residual of a row group is requested together with the group's first weight step, i.e. ahead
    // of loads the pipeline waits for anyway.  Read at the group's end instead, it would be the youngest load in
    // flight and waiting for it would drain the prefetched next step every time (wait counts retire in order).
    auto residual_of = [&](const Located &l, bool live) -> float {
        const int row = l.row0 + static_cast<int>(lane);
        return (EPI == EPI_ADD && live && lane < static_cast<unsigned>(R) && row < l.n) ? residual[row] : 0.f;
    };
    float res_cur = 0.f, res_next = 0.f;

    StepBuf<R, S> a, b;
    {
        const int g0 = wave_global < n_groups ? wave_global : 0;
        if (g0 < end0) {  // wave-uniform
            load_step(a, qs0, ds0, g0 * R, n0, k, 0, lane, T > 0);
            asm volatile("" ::: "memory");  // keeps the two arms apart: merged, the loads would wait for the structs
        } else {
            const Located l = locate<R>(p, g0);
            load_step(a, l.qs, l.ds, l.row0, l.n, k, 0, lane, T > 0);
        }
        res_cur = residual_of(locate<R>(p, g0), T > 0);
    }

    // The norm's scalar factor commutes with the matrix product, so x * g is staged at once and the row sums
    // are multiplied by 1/sqrt(mean(x^2) + eps) at the end: the sum of squares rides on the staging loads and
    // is published by the staging barrier.
    {
        const float4 *x4 = reinterpret_cast<const float4 *>(x);
        const float4 *g4 = reinterpret_cast<const float4 *>(norm_w);
        const int k4 = k >> 2;
        float ss = 0.f;
        int n_active = 0;
        if (PRO == PRO_MERGE) {  // the key ranges the attention launch cut this position's context into
            const int n_keys = min(*f.pos + 1, f.max_seq);
            const int eff = dec_active_splits(n_keys, f.n_splits, true);
            const int chunk = (n_keys + eff - 1) / eff;
            n_active = (n_keys + chunk - 1) / chunk;
        }
#pragma unroll 4
        for (int i = threadIdx.x; i < k4; i += W * 64) {
            const int src = (i & ~255) | ((i & 63) << 2) | ((i >> 6) & 3);
            float4 v;
            if (PRO == PRO_MERGE)
                v = merged_attention_piece(f, src, n_active);
            else
                v = x4[src];
            if (NORM) {
                const float4 g = g4[src];
                // spelled out, so that every kernel that takes this sum rounds it the same way
                ss = fmaf(v.x, v.x, ss);
                ss = fmaf(v.y, v.y, ss);
                ss = fmaf(v.z, v.z, ss);
                ss = fmaf(v.w, v.w, ss);
                v = make_float4(v.x * g.x, v.y * g.y, v.z * g.z, v.w * g.w);
            }
            xs4[i] = v;
        }
        if (NORM) {
            ss = wave_sum(ss);
            if (lane == 0) red[wave] = ss;
        }
    }
    // The structs are read here, behind the first weight loads and the staging loads: left to their first use inside
    // the pipeline loop, the read would stall the second step of every wave.
    asm volatile("" ::"s"(p.group_end[1]), "s"(p.group_end[2]), "s"(p.n[1]));
    __syncthreads();
    if (T == 0) return;
    float scale = 1.f;
    if (NORM) {
        float total = 0.f;
#pragma unroll
        for (int w = 0; w < W; ++w) total += red[w];
        scale = 1.0f / sqrtf(total / static_cast<float>(k) + eps);
    }

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;

    int t = 0, g = wave_global, c = 0;
    auto next = [&](int &gg, int &cc) {
        if (++cc == chunks) {
            cc = 0;
            gg += total_waves;
        }
    };
    auto issue = [&](StepBuf<R, S> &buf, int gg, int cc, bool live) {
        const Located l = locate<R>(p, live ? gg : 0);
        if (EPI == EPI_ADD && cc == 0) res_next = residual_of(l, live);
        load_step(buf, l.qs, l.ds, l.row0, l.n, k, cc * S, lane, live);
    };
    auto finish_group = [&](int gg) {
        const Located l = locate<R>(p, gg);
        float sum[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            sum[r] = wave_sum(acc[r]);
            if (NORM) sum[r] *= scale;
            acc[r] = 0.f;
        }
        if (EPI == EPI_SWIGLU) {
            float out = 0.f;
#pragma unroll
            for (int j = 0; j < R / 2; ++j) {
                const float gate = sum[2 * j], up = sum[2 * j + 1];
                const float v = up * (gate * (1.0f / (1.0f + expf(-gate))));
                if (lane == static_cast<unsigned>(j)) out = v;
            }
            const int pair = l.row0 / 2 + static_cast<int>(lane);
            if (lane < static_cast<unsigned>(R / 2) && 2 * pair + 1 < l.n) l.y[pair] = out;
        } else {
            float out = 0.f;
#pragma unroll
            for (int r = 0; r < R; ++r)
                if (lane == static_cast<unsigned>(r)) out = sum[r];
            const int row = l.row0 + static_cast<int>(lane);
            if (lane < static_cast<unsigned>(R) && row < l.n) {
                if (EPI == EPI_ADD) out += res_cur;
                l.y[row] = out;
            }
            if (EPI == EPI_ADD) res_cur = res_next;
        }
    };

    while (true) {
        int g1 = g, c1 = c;
        next(g1, c1);
        issue(b, g1, c1, t + 1 < T);
        __builtin_amdgcn_sched_barrier(0);
        compute_step(a, xs4, c * S, lane, acc);
        if (c == chunks - 1) finish_group(g);
        if (++t >= T) break;
        g = g1;
        c = c1;
        next(g1, c1);
        issue(a, g1, c1, t + 1 < T);
        __builtin_amdgcn_sched_barrier(0);
        compute_step(b, xs4, c * S, lane, acc);
        if (c == chunks - 1) finish_group(g);
        if (++t >= T) break;
        g = g1;
        c = c1;
    }
}

constexpr int kNumCUs = 256;
constexpr int64_t kMaxGridRows = 65535;  // grid y
constexpr int kMaxLdsK = 16384;  // 64 KiB of staged activations

template <int R, int W, int U, typename T>
static lhip_status launch_oneshot(const int8_t *qs, const __half *ds, const T *x, T *y, int m, int n, int k,
                                  hipStream_t s) {
    const unsigned tiles = static_cast<unsigned>((n + R * W - 1) / (R * W));
    hipLaunchKernelGGL((q8_gemv_f32_kernel<R, W, U, T>), dim3(tiles, static_cast<unsigned>(m)), dim3(W * 64), 0, s, qs,
                       ds, x, y, n, k);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

// Workgroups of the persistent kernel: one wave per row group, capped at blocks_per_cu resident workgroups per CU.
static int pipe_grid(int n, int r, int w, int blocks_per_cu) {
    const int n_groups = (n + r - 1) / r;
    const int grid = (n_groups + w - 1) / w, cap = kNumCUs * blocks_per_cu;
    return grid > cap ? cap : grid;
}

template <int R, int S, int W, typename T>
static lhip_status launch_pipe(const int8_t *qs, const __half *ds, const T *x, T *y, int m, int n, int k,
                               int blocks_per_cu, hipStream_t s) {
    if (k % (S * 1024) != 0 || k > kMaxLdsK) return LHIP_ERR_UNSUPPORTED;
    const int grid = pipe_grid(n, R, W, blocks_per_cu);
    hipLaunchKernelGGL((q8_gemv_f32_pipe_kernel<R, S, W, T>), dim3(static_cast<unsigned>(grid), static_cast<unsigned>(m)),
                       dim3(W * 64), static_cast<size_t>(k) * sizeof(float), s, qs,
                       reinterpret_cast<const unsigned short *>(ds), x, y, n, k);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

// Launch-shape table.  blocks_per_cu == 0 selects the one-shot kernel
// (rows_per_wave in {1,2,4,8}, k_unroll in {1,2,4}); otherwise the pipelined
// kernel (rows_per_wave in {1,2,4}, k_unroll = slices per step in {1,2,4},
// waves_per_block in {4,8,16}).
static lhip_status dispatch(int rows_per_wave, int k_unroll, int blocks_per_cu, int waves_per_block, const int8_t *qs,
                            const __half *ds, const float *x, float *y, int m, int n, int k, hipStream_t s) {
    if (blocks_per_cu < 0 || blocks_per_cu > 16) return LHIP_ERR_UNSUPPORTED;
    if (blocks_per_cu == 0) {
#define LHIP_CASE(R, U) \
    if (rows_per_wave == R && k_unroll == U) return launch_oneshot<R, 4, U>(qs, ds, x, y, m, n, k, s);
        LHIP_CASE(1, 1) LHIP_CASE(1, 2) LHIP_CASE(1, 4)
        LHIP_CASE(2, 1) LHIP_CASE(2, 2) LHIP_CASE(2, 4)
        LHIP_CASE(4, 1) LHIP_CASE(4, 2) LHIP_CASE(4, 4)
        LHIP_CASE(8, 1) LHIP_CASE(8, 2)
#undef LHIP_CASE
        return LHIP_ERR_UNSUPPORTED;
    }
#define LHIP_CASE(R, S)                                                                                          \
    if (rows_per_wave == R && k_unroll == S) {                                                                   \
        if (waves_per_block == 4) return launch_pipe<R, S, 4>(qs, ds, x, y, m, n, k, blocks_per_cu, s);          \
        if (waves_per_block == 8) return launch_pipe<R, S, 8>(qs, ds, x, y, m, n, k, blocks_per_cu, s);          \
        if constexpr (R * S <= 8)                                                                                \
            if (waves_per_block == 16) return launch_pipe<R, S, 16>(qs, ds, x, y, m, n, k, blocks_per_cu, s);    \
        return LHIP_ERR_UNSUPPORTED;                                                                             \
    }
    LHIP_CASE(1, 1) LHIP_CASE(1, 2) LHIP_CASE(1, 4)
    LHIP_CASE(2, 1) LHIP_CASE(2, 2) LHIP_CASE(2, 4)
    LHIP_CASE(4, 1) LHIP_CASE(4, 2) LHIP_CASE(4, 4)
#undef LHIP_CASE
    return LHIP_ERR_UNSUPPORTED;
}

// The f16 activation type runs the launch shapes choose() picks, nothing else.
static lhip_status dispatch_f16(int rows_per_wave, int k_unroll, int blocks_per_cu, int waves_per_block, const int8_t *qs,
                                const __half *ds, const __half *x, __half *y, int m, int n, int k, hipStream_t s) {
    if (blocks_per_cu == 0) {
        if (rows_per_wave == 1) return launch_oneshot<1, 4, 1>(qs, ds, x, y, m, n, k, s);
        if (rows_per_wave == 2) return launch_oneshot<2, 4, 1>(qs, ds, x, y, m, n, k, s);
        return launch_oneshot<4, 4, 1>(qs, ds, x, y, m, n, k, s);
    }
    if (rows_per_wave == 2) return launch_pipe<2, 4, 4>(qs, ds, x, y, m, n, k, blocks_per_cu, s);
    if (waves_per_block == 16)
        return k_unroll == 2 ? launch_pipe<1, 2, 16>(qs, ds, x, y, m, n, k, blocks_per_cu, s)
                             : launch_pipe<1, 1, 16>(qs, ds, x, y, m, n, k, blocks_per_cu, s);
    return k_unroll == 2 ? launch_pipe<1, 2, 4>(qs, ds, x, y, m, n, k, blocks_per_cu, s)
                         : launch_pipe<1, 1, 4>(qs, ds, x, y, m, n, k, blocks_per_cu, s);
}

// Default launch shape per problem size.
static void choose(int n, int k, int *rows_per_wave, int *k_unroll, int *blocks_per_cu, int *waves_per_block) {
    *waves_per_block = 4;
    int slices = 0;  // slices per pipeline step that divide K, 0 if none
    if (k <= kMaxLdsK) {
        if (k % 4096 == 0) slices = 4;
        else if (k % 2048 == 0) slices = 2;
        else if (k % 1024 == 0) slices = 1;
    }
    if (slices == 0) {  // ragged or very long K: one-shot kernel
        *rows_per_wave = n >= 8192 ? 4 : (n >= 4096 ? 2 : 1);
        *k_unroll = 1;
        *blocks_per_cu = 0;
        return;
    }
    // Measured on MI355X: very tall matrices run best with one fat wave per
    // SIMD (2 rows x 4 slices, double-buffered); everything else with one row
    // x 2 slices per step and as many resident workgroups as the LDS stage of
    // the activations allows, up to 3 per CU.
    if (n >= 32768 && slices == 4) {
        *rows_per_wave = 2;
        *k_unroll = 4;
        *blocks_per_cu = 1;
        return;
    }
    *rows_per_wave = 1;
    *k_unroll = slices >= 2 ? 2 : 1;
    const int fit = (160 * 1024) / (k * 4);  // workgroups whose staged activations fit the CU's LDS
    if (fit >= 3) {
        *blocks_per_cu = 3;
    } else {  // long K: one workgroup of 16 waves per CU shares a single staged copy
        *blocks_per_cu = 1;
        *waves_per_block = 16;
    }
}

template <int R, int S, int W, int PRO, int EPI>
static lhip_status launch_fused(const GemvGroup &p, const GemvFuse &f, const float *x, int k, int n_groups,
                                int blocks_per_cu, hipStream_t s) {
    int grid = (n_groups + W - 1) / W;
    const int cap = kNumCUs * blocks_per_cu;
    if (grid > cap) grid = cap;
    const size_t lds_bytes = static_cast<size_t>(k) * sizeof(float);
    static LdsOptIn opt;  // with the static reduction array: beyond the default limit (K = 16384)
    if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(q8_gemv_fused_kernel<R, S, W, PRO, EPI>), lds_bytes,
                                    lds_bytes + W * sizeof(float) > 64 * 1024))
        return st;
    hipLaunchKernelGGL((q8_gemv_fused_kernel<R, S, W, PRO, EPI>), dim3(static_cast<unsigned>(grid)), dim3(W * 64),
                       lds_bytes, s, p.qs[0], p.ds[0], x, PRO == PRO_NORM ? f.norm_w : f.residual, p.n[0], p.group_end[0], k, n_groups,
                       grid, f.eps, p, f);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

template <int R, int S, int W>
static lhip_status launch_fused_variant(bool norm, int epi, const GemvGroup &p, const GemvFuse &f, const float *x, int k,
                                        int n_groups, int blocks_per_cu, hipStream_t s) {
    if (epi == EPI_SWIGLU) {
        if constexpr (R % 2 == 0) {
            return norm ? launch_fused<R, S, W, PRO_NORM, EPI_SWIGLU>(p, f, x, k, n_groups, blocks_per_cu, s)
                        : launch_fused<R, S, W, PRO_NONE, EPI_SWIGLU>(p, f, x, k, n_groups, blocks_per_cu, s);
        } else {
            return LHIP_ERR_UNSUPPORTED;
        }
    }
    if (epi == EPI_ADD)
        return norm ? launch_fused<R, S, W, PRO_NORM, EPI_ADD>(p, f, x, k, n_groups, blocks_per_cu, s)
                    : launch_fused<R, S, W, PRO_NONE, EPI_ADD>(p, f, x, k, n_groups, blocks_per_cu, s);
    return norm ? launch_fused<R, S, W, PRO_NORM, EPI_NONE>(p, f, x, k, n_groups, blocks_per_cu, s)
                : launch_fused<R, S, W, PRO_NONE, EPI_NONE>(p, f, x, k, n_groups, blocks_per_cu, s);
}

// Launch shapes of the fused kernel: (rows per wave, slices per step, waves per workgroup, workgroups per CU).
static lhip_status dispatch_fused(int r, int sl, int w, int bpc, bool norm, int epi, const GemvGroup &p,
                                  const GemvFuse &f, const float *x, int k, int n_groups, hipStream_t s) {
#define LHIP_CASE(R, S, W) \
    if (r == R && sl == S && w == W) return launch_fused_variant<R, S, W>(norm, epi, p, f, x, k, n_groups, bpc, s);
    LHIP_CASE(2, 4, 4) LHIP_CASE(1, 2, 4) LHIP_CASE(2, 2, 4) LHIP_CASE(1, 1, 4) LHIP_CASE(2, 1, 4)
    LHIP_CASE(1, 2, 16) LHIP_CASE(2, 2, 8) LHIP_CASE(1, 1, 16) LHIP_CASE(2, 1, 8)
#undef LHIP_CASE
    return LHIP_ERR_UNSUPPORTED;
}

// Default launch shape of the fused kernel for n_total rows (all weights together).
static void choose_fused(int64_t n_total, int k, int pro, int epi, int *r, int *sl, int *w, int *bpc) {
    const int slices = k % 4096 == 0 ? 4 : (k % 2048 == 0 ? 2 : 1);
    const int fit = (160 * 1024) / (k * 4);
    if (n_total >= 16384 && slices == 4 && fit >= 1) {
        *r = 2, *sl = 4, *w = 4, *bpc = 1;
        return;
    }
    const bool pairs = epi == EPI_SWIGLU;
    *sl = slices >= 2 ? 2 : 1;
    if (fit >= 3) {
        // (measured, q|k|v = 6144 rows at K = 4096: four workgroups per CU 7.25 us against 7.55 with three when nothing
        // precedes the products; with the norm prologue, which every workgroup pays for, three or two: decode 481 tok/s
        // against 474 with four; the 4096 rows of o: 6.15 with three, 6.25 with four)
        *r = pairs ? 2 : 1, *w = 4, *bpc = pairs ? 2 : (pro == PRO_NONE && n_total > 4096 ? 4 : 3);
    } else {
        *r = pairs ? 2 : 1, *w = pairs ? 8 : 16, *bpc = 1;
    }
}

static lhip_status check_args(const void *planar, const float *x, float *y, int64_t m, int64_t n, int64_t k) {
    if (!planar || !x || !y) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (m <= 0 || m > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(planar, 256) || !aligned(x, 16) || !aligned(y, 4)) return LHIP_ERR_MISALIGNED;
    // Rows of x start at multiples of K floats; K % 32 == 0 keeps them 16-byte aligned.
    return LHIP_OK;
}

}  // namespace lhip

using namespace lhip;

extern "C" {

lhip_status lhip_q8_0_matmul_f32_gemm(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                      int64_t k, void *stream);
lhip_status lhip_q8_0_matmul_f16_gemm(const void *planar_dev, const void *x_f16_dev, void *y_f16_dev, int64_t m,
                                      int64_t n, int64_t k, void *stream);

lhip_status lhip_q8_0_matmul_f32_cfg(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                     int64_t k, int rows_per_wave, int k_unroll, int blocks_per_cu,
                                     int waves_per_block, void *stream) {
    if (lhip_status s = check_args(planar_dev, x_dev, y_dev, m, n, k)) return s;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    // the activation rows are the grid's y dimension: passes of at most kMaxGridRows
    for (int64_t m0 = 0; m0 < m; m0 += kMaxGridRows) {
        const int mc = static_cast<int>(m - m0 < kMaxGridRows ? m - m0 : kMaxGridRows);
        if (lhip_status st = dispatch(rows_per_wave, k_unroll, blocks_per_cu, waves_per_block,
                                      reinterpret_cast<const int8_t *>(base),
                                      reinterpret_cast<const __half *>(base + q8_scale_offset(n, k)), x_dev + m0 * k,
                                      y_dev + m0 * n, mc, static_cast<int>(n), static_cast<int>(k), as_stream(stream)))
            return st;
    }
    return LHIP_OK;
}

lhip_status lhip_q8_0_matmul_f32(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                 int64_t k, void *stream) {
    if (lhip_status s = check_args(planar_dev, x_dev, y_dev, m, n, k)) return s;
    if (m >= split_min_rows(n, k) && q8_gemm_split_supports(static_cast<int>(n), static_cast<int>(k), x_dev, y_dev, false))
        return lhip_q8_0_matmul_f32_gemm(planar_dev, x_dev, y_dev, m, n, k, stream);
    int r, u, b, w;
    choose(static_cast<int>(n), static_cast<int>(k), &r, &u, &b, &w);
    return lhip_q8_0_matmul_f32_cfg(planar_dev, x_dev, y_dev, m, n, k, r, u, b, w, stream);
}

lhip_status lhip_q8_0_gemv_kernel_plan(int64_t n, int64_t k, int f16, char *kernel_name, size_t kernel_name_cap,
                                       uint32_t grid[3], uint32_t block[3], uint32_t *lds_bytes) {
    if (!kernel_name || !grid || !block || !lds_bytes) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    int r, u, b, w;
    choose(static_cast<int>(n), static_cast<int>(k), &r, &u, &b, &w);
    const char *t = f16 ? "f16" : "f32";
    int len;
    if (b == 0) {  // launch_oneshot<R, 4, 1>
        len = snprintf(kernel_name, kernel_name_cap, "lhip_kernel_q8_0_gemv_%s_oneshot_r%d", t, r);
        grid[0] = static_cast<uint32_t>((n + r * 4 - 1) / (r * 4));
        block[0] = 256;
        *lds_bytes = 0;
    } else {  // launch_pipe<R, S, W>
        len = snprintf(kernel_name, kernel_name_cap, "lhip_kernel_q8_0_gemv_%s_pipe_r%ds%dw%d", t, r, u, w);
        grid[0] = static_cast<uint32_t>(pipe_grid(static_cast<int>(n), r, w, b));
        block[0] = static_cast<uint32_t>(w) * 64;
        *lds_bytes = static_cast<uint32_t>(k) * 4;
    }
    grid[1] = grid[2] = block[1] = block[2] = 1;
    return len > 0 && static_cast<size_t>(len) < kernel_name_cap ? LHIP_OK : LHIP_ERR_INVALID_SHAPE;
}

lhip_status lhip_q8_0_matmul_f16(const void *planar_dev, const void *x_f16_dev, void *y_f16_dev, int64_t m, int64_t n,
                                 int64_t k, void *stream) {
    if (!planar_dev || !x_f16_dev || !y_f16_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (m <= 0 || m > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
    // Rows of x start at multiples of K halves; K % 32 == 0 keeps them 8-byte aligned.
    if (!aligned(planar_dev, 256) || !aligned(x_f16_dev, 8) || !aligned(y_f16_dev, 2)) return LHIP_ERR_MISALIGNED;
    if (m >= split_min_rows(n, k) && q8_gemm_split_supports(static_cast<int>(n), static_cast<int>(k), x_f16_dev, y_f16_dev, true))
        return lhip_q8_0_matmul_f16_gemm(planar_dev, x_f16_dev, y_f16_dev, m, n, k, stream);
    auto *base = static_cast<const uint8_t *>(planar_dev);
    int r, u, b, w;
    choose(static_cast<int>(n), static_cast<int>(k), &r, &u, &b, &w);
    for (int64_t m0 = 0; m0 < m; m0 += kMaxGridRows) {
        const int mc = static_cast<int>(m - m0 < kMaxGridRows ? m - m0 : kMaxGridRows);
        if (lhip_status st = dispatch_f16(r, u, b, w, reinterpret_cast<const int8_t *>(base),
                                          reinterpret_cast<const __half *>(base + q8_scale_offset(n, k)),
                                          static_cast<const __half *>(x_f16_dev) + m0 * k,
                                          static_cast<__half *>(y_f16_dev) + m0 * n, mc, static_cast<int>(n),
                                          static_cast<int>(k), as_stream(stream)))
            return st;
    }
    return LHIP_OK;
}

lhip_status lhip_q8_0_matmul_f32_gemm(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                      int64_t k, void *stream) {
    if (lhip_status s = check_args(planar_dev, x_dev, y_dev, m, n, k)) return s;
    if (!q8_gemm_split_supports(static_cast<int>(n), static_cast<int>(k), x_dev, y_dev, false)) return LHIP_ERR_UNSUPPORTED;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    return q8_gemm_split_launch(reinterpret_cast<const int8_t *>(base),
                                reinterpret_cast<const __half *>(base + q8_scale_offset(n, k)), x_dev, y_dev, m,
                                static_cast<int>(n), static_cast<int>(k), false, 0, as_stream(stream));
}

lhip_status lhip_q8_0_matmul_f16_gemm(const void *planar_dev, const void *x_f16_dev, void *y_f16_dev, int64_t m,
                                      int64_t n, int64_t k, void *stream) {
    if (!planar_dev || !x_f16_dev || !y_f16_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (m <= 0 || m > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(planar_dev, 256) || !aligned(x_f16_dev, 8) || !aligned(y_f16_dev, 2)) return LHIP_ERR_MISALIGNED;
    if (!q8_gemm_split_supports(static_cast<int>(n), static_cast<int>(k), x_f16_dev, y_f16_dev, true))
        return LHIP_ERR_UNSUPPORTED;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    return q8_gemm_split_launch(reinterpret_cast<const int8_t *>(base),
                                reinterpret_cast<const __half *>(base + q8_scale_offset(n, k)), x_f16_dev, y_f16_dev, m,
                                static_cast<int>(n), static_cast<int>(k), true, 0, as_stream(stream));
}

size_t lhip_q8_0_matmul_workspace_nbytes(int64_t m, int64_t n, int64_t k) {
    if (check_q8_shape(n, k) != LHIP_OK || m <= 0 || m > kMaxDim) return 0;
    if (m < split_min_rows(n, k) || k % 512 != 0 || n % 4 != 0) return 0;  // the matvec kernels keep nothing outside their outputs
    return q8_gemm_split_workspace_floats(m, static_cast<int>(n), static_cast<int>(k)) * sizeof(float);
}

lhip_status lhip_q8_0_matmul_f32_ws(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                    int64_t k, void *workspace_dev, size_t workspace_nbytes, void *stream) {
    if (lhip_status s = check_args(planar_dev, x_dev, y_dev, m, n, k)) return s;
    if (workspace_dev && !aligned(workspace_dev, 256)) return LHIP_ERR_MISALIGNED;
    if (m >= split_min_rows(n, k) && q8_gemm_split_supports(static_cast<int>(n), static_cast<int>(k), x_dev, y_dev, false)) {
        auto *base = static_cast<const uint8_t *>(planar_dev);
        return q8_gemm_split_launch(reinterpret_cast<const int8_t *>(base),
                                    reinterpret_cast<const __half *>(base + q8_scale_offset(n, k)), x_dev, y_dev, m,
                                    static_cast<int>(n), static_cast<int>(k), false, 0, as_stream(stream), true,
                                    static_cast<float *>(workspace_dev), workspace_dev ? workspace_nbytes / sizeof(float) : 0);
    }
    return lhip_q8_0_matmul_f32(planar_dev, x_dev, y_dev, m, n, k, stream);  // matvec kernels: no shared state
}

lhip_status lhip_q8_0_matmul_f16_ws(const void *planar_dev, const void *x_f16_dev, void *y_f16_dev, int64_t m, int64_t n,
                                    int64_t k, void *workspace_dev, size_t workspace_nbytes, void *stream) {
    if (!planar_dev || !x_f16_dev || !y_f16_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (m <= 0 || m > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(planar_dev, 256) || !aligned(x_f16_dev, 8) || !aligned(y_f16_dev, 2)) return LHIP_ERR_MISALIGNED;
    if (workspace_dev && !aligned(workspace_dev, 256)) return LHIP_ERR_MISALIGNED;
    if (m >= split_min_rows(n, k) && q8_gemm_split_supports(static_cast<int>(n), static_cast<int>(k), x_f16_dev, y_f16_dev, true)) {
        auto *base = static_cast<const uint8_t *>(planar_dev);
        return q8_gemm_split_launch(reinterpret_cast<const int8_t *>(base),
                                    reinterpret_cast<const __half *>(base + q8_scale_offset(n, k)), x_f16_dev, y_f16_dev, m,
                                    static_cast<int>(n), static_cast<int>(k), true, 0, as_stream(stream), true,
                                    static_cast<float *>(workspace_dev), workspace_dev ? workspace_nbytes / sizeof(float) : 0);
    }
    return lhip_q8_0_matmul_f16(planar_dev, x_f16_dev, y_f16_dev, m, n, k, stream);
}

lhip_status lhip_q8_0_matvec_fused_f32_cfg(const void *const *planar_dev, float *const *y_dev, const int64_t *n,
                                           int count, const float *x_dev, int64_t k, const float *norm_weight_dev,
                                           float eps, const float *residual_dev, int epilogue, int rows_per_wave,
                                           int k_unroll, int waves_per_block, int blocks_per_cu, void *stream) {
    if (!planar_dev || !y_dev || !n || !x_dev) return LHIP_ERR_NULL_PTR;
    if (count < 1 || count > kMaxGroup) return LHIP_ERR_INVALID_SHAPE;
    if (epilogue != EPI_NONE && epilogue != EPI_ADD && epilogue != EPI_SWIGLU) return LHIP_ERR_UNSUPPORTED;
    if (epilogue == EPI_ADD && (!residual_dev || count != 1)) return residual_dev ? LHIP_ERR_UNSUPPORTED : LHIP_ERR_NULL_PTR;
    if (!aligned(x_dev, 16) || (norm_weight_dev && !aligned(norm_weight_dev, 16))) return LHIP_ERR_MISALIGNED;
    if (k <= 0 || k % 1024 != 0 || k > kMaxLdsK) return k > 0 && k % 32 == 0 ? LHIP_ERR_UNSUPPORTED : LHIP_ERR_INVALID_SHAPE;
    if (rows_per_wave < 1 || k_unroll < 1 || blocks_per_cu < 1 || blocks_per_cu > 16 || k % (k_unroll * 1024) != 0)
        return LHIP_ERR_UNSUPPORTED;
    GemvGroup p;
    int64_t groups = 0;
    for (int i = 0; i < kMaxGroup; ++i) {
        if (i < count) {
            if (!planar_dev[i] || !y_dev[i]) return LHIP_ERR_NULL_PTR;
            if (lhip_status st = check_q8_shape(n[i], k)) return st;
            if (epilogue == EPI_SWIGLU && n[i] % 2 != 0) return LHIP_ERR_INVALID_SHAPE;
            if (!aligned(planar_dev[i], 256) || !aligned(y_dev[i], 4)) return LHIP_ERR_MISALIGNED;
            auto *base = static_cast<const uint8_t *>(planar_dev[i]);
            p.qs[i] = reinterpret_cast<const int8_t *>(base);
            p.ds[i] = reinterpret_cast<const unsigned short *>(base + q8_scale_offset(n[i], k));
            p.y[i] = y_dev[i];
            p.n[i] = static_cast<int>(n[i]);
            groups += (n[i] + rows_per_wave - 1) / rows_per_wave;
            if (groups > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
            p.group_end[i] = static_cast<int>(groups);
        } else {
            p.qs[i] = p.qs[0], p.ds[i] = p.ds[0], p.y[i] = p.y[0], p.n[i] = p.n[0];
            p.group_end[i] = INT_MAX;
        }
    }
    GemvFuse f{};
    f.norm_w = norm_weight_dev;
    f.eps = eps;
    f.residual = residual_dev;
    return dispatch_fused(rows_per_wave, k_unroll, waves_per_block, blocks_per_cu, norm_weight_dev != nullptr, epilogue,
                          p, f, x_dev, static_cast<int>(k), static_cast<int>(groups), as_stream(stream));
}

lhip_status lhip_q8_0_matvec_attn_merge_f32(const void *planar_dev, float *y_dev, int64_t n, int64_t k,
                                            const void *attn_workspace_dev, const int32_t *pos_dev, int64_t q_heads,
                                            int64_t kv_heads, int64_t head_dim, int64_t max_seq, const float *residual_dev,
                                            void *stream) {
    if (!planar_dev || !y_dev || !attn_workspace_dev || !pos_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status st = check_q8_shape(n, k)) return st;
    if (q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || max_seq <= 0 || q_heads % kv_heads != 0 || max_seq > kMaxDim ||
        kv_heads > 65535 || k != q_heads * head_dim)
        return LHIP_ERR_INVALID_SHAPE;
    const int64_t gq = q_heads / kv_heads;
    if (!(gq == 1 || gq == 2 || gq == 4 || gq == 8) || !(head_dim == 64 || head_dim == 128)) return LHIP_ERR_UNSUPPORTED;
    // one 16-wave workgroup per CU shares a single merged copy of the activations; slices of 2048
    if (k % 2048 != 0 || k > kMaxLdsK) return LHIP_ERR_UNSUPPORTED;
    if (!aligned(planar_dev, 256) || !aligned(y_dev, 4) || !aligned(attn_workspace_dev, 256) ||
        (residual_dev && !aligned(residual_dev, 4)))
        return LHIP_ERR_MISALIGNED;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    GemvGroup p;
    for (int i = 0; i < kMaxGroup; ++i) {
        p.qs[i] = reinterpret_cast<const int8_t *>(base);
        p.ds[i] = reinterpret_cast<const unsigned short *>(base + q8_scale_offset(n, k));
        p.y[i] = y_dev;
        p.n[i] = static_cast<int>(n);
        p.group_end[i] = i == 0 ? static_cast<int>(n) : INT_MAX;
    }
    const int splits = dec_splits(kv_heads);
    auto *ws = static_cast<const uint8_t *>(attn_workspace_dev);
    GemvFuse f{};
    f.residual = residual_dev;
    f.ws_ml = reinterpret_cast<const float *>(ws);
    f.ws_acc = reinterpret_cast<const float4 *>(ws + dec_ml_bytes(kv_heads, splits, gq));
    f.pos = pos_dev;
    f.hkv = static_cast<int>(kv_heads);
    f.g = static_cast<int>(gq);
    f.c4 = static_cast<int>(head_dim / 4);
    f.n_splits = splits;
    f.max_seq = static_cast<int>(max_seq);
    hipStream_t s = as_stream(stream);
    const int ki = static_cast<int>(k), groups = static_cast<int>(n);
    return residual_dev ? launch_fused<1, 2, 16, PRO_MERGE, EPI_ADD>(p, f, nullptr, ki, groups, 1, s)
                        : launch_fused<1, 2, 16, PRO_MERGE, EPI_NONE>(p, f, nullptr, ki, groups, 1, s);
}

lhip_status lhip_q8_0_matvec_fused_f32(const void *const *planar_dev, float *const *y_dev, const int64_t *n, int count,
                                       const float *x_dev, int64_t k, const float *norm_weight_dev, float eps,
                                       const float *residual_dev, int epilogue, void *stream) {
    if (!n) return LHIP_ERR_NULL_PTR;
    if (count < 1 || count > kMaxGroup) return LHIP_ERR_INVALID_SHAPE;
    if (k <= 0 || k % 1024 != 0 || k > kMaxLdsK) return k > 0 && k % 32 == 0 ? LHIP_ERR_UNSUPPORTED : LHIP_ERR_INVALID_SHAPE;
    int64_t total = 0;
    for (int i = 0; i < count; ++i) total += n[i] > 0 ? n[i] : 0;
    int r, sl, w, bpc;
    choose_fused(total, static_cast<int>(k), norm_weight_dev ? PRO_NORM : PRO_NONE, epilogue, &r, &sl, &w, &bpc);
    return lhip_q8_0_matvec_fused_f32_cfg(planar_dev, y_dev, n, count, x_dev, k, norm_weight_dev, eps, residual_dev,
                                          epilogue, r, sl, w, bpc, stream);
}

}  // extern "C"
