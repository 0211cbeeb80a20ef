// Persistent decode program: a whole batch-1 decode step (every layer's matvecs and attention, then the
// vocabulary projection) as ONE launch.
//
// Why.  Launched one by one, the kernels of a Llama-3-8B step each stream their weights at close to the HBM
// rate once they are going, but every launch pays ~7 us around that: ~3 us between the end of one kernel and
// the first wave of the next, ~2.5 us until the first weights and the staged activations have arrived, ~1.3 us
// while the slowest waves finish.  With 6 launches per layer that is 40 us of a 65 us layer.  Here the grid
// (one workgroup of 8 wavefronts per compute unit) stays resident and walks a list of phases, and the weight
// stream does not stop between them: weights do not depend on the previous phase, so every wave requests the
// first two pipeline steps of the next matvec while it finishes the current one and holds them in registers.
//
// Phases.  MATVEC: the fused Q8_0 matvec of q8_gemv.hip (optional RMS-norm prologue; epilogues none / residual
// add / SwiGLU) with the same per-row arithmetic and the same reduction orders, so results equal the per-kernel
// path bit for bit where that path runs four-wave workgroups.  ATTENTION and MERGE: the bodies of
// attention_decode_device.h, one (KV head, key range) piece or one KV head per workgroup.
//
// Synchronisation is carried by the data.  A vector produced in one phase and consumed in a later one
// (activations, attention partials) lives in a shadow array of 64-bit words (value, tag), the tag naming the
// launch and the producing phase.  Producers write each word with one agent-coherent store; a consumer reads
// the words it needs with agent-coherent loads and repeats until all of them carry the tag it expects.  There
// is no barrier, no fence and no cache write-back: a consumer starts one memory round trip after the last
// producer's store (measured: 1.8 us per hop for 256 workgroups exchanging 4096 values, against 2.6 us for a
// counter barrier plus 3 us for the loads that can only start behind it), and workgroups that have nothing to
// wait for run ahead.  An array may be overwritten two phases after it was written: a workgroup that writes in
// phase p + 2 has read all of phase p + 1's output, so every workgroup has finished phase p + 1 and with it
// its reads of phase p's output.  The program is checked for this when it is created.  Weights, norm gains and
// the KV caches of earlier positions are read-only within a launch and use ordinary (non-temporal) loads.
//
// Termination.  Every wait is bounded: a thread that repeats its loads kTagSpinLimit times raises a flag, every
// other waiter that sees the flag stops waiting, and the kernel runs to its end (with meaningless results).
// The flag is sticky and reported by lhip_decode_program_status.  All workgroups must be resident at once:
// the grid is one workgroup per compute unit, which the register and LDS budget of the kernel guarantees.
#include <hip/hip_fp16.h>
#include <limits.h>
#include <algorithm>

#include <new>
#include <vector>

#include "attention_decode_device.h"
#include "common.h"
#include "q8_gemv_device.h"

namespace lhip {

constexpr int kProgWaves = 8;
constexpr int kProgThreads = kProgWaves * 64;
constexpr int kProgSlots = 8;            // 16-byte weight loads per lane and pipeline step
constexpr int kProgMaxK = 14336;         // activations staged in LDS as f32: 56 KiB
constexpr int kSyncWords = 64;           // [0] launch counter, [32] abort flag of the running launch, [48] sticky flag
constexpr unsigned kTagsPerLaunch = 8192;  // tag = launch * kTagsPerLaunch + phase + 1; never 0

enum { PHASE_MATVEC = 0, PHASE_ATTENTION = 1, PHASE_MERGE = 2 };
enum { EPI_NONE = 0, EPI_ADD = 1, EPI_SWIGLU = 2 };

typedef unsigned long long tagged_t;  // (tag << 32) | float bits

struct ProgOp {
    int type;
    int r, s;          // MATVEC: rows per wave and 1024-quant slices per pipeline step, r * s <= kProgSlots
    int n, k, n_groups, chunks;
    int epi, norm;
    float eps;
    int next_matvec;   // index of the next MATVEC phase, -1 if none
    int x_phase;       // phase that produces x (its tag is expected), -1: x is there before the launch
    const int8_t *qs;
    const unsigned short *ds;
    const float *x;    // MATVEC: activations (K);  ATTENTION: fused qkv row.  Read when x_phase < 0 ...
    const tagged_t *x_t;  // ... otherwise this shadow
    float *y;          // MATVEC: output;  MERGE: attention output rows (written besides the shadow)
    tagged_t *y_t;
    const float *norm_w;
    const float *residual;     // EPI_ADD: read when res_t is null
    const tagged_t *res_t;     // shadow of the residual when an earlier phase of the launch wrote it
    int res_phase;             // ... and that phase (its tag is expected on the shadow's words)
    float *k_cache, *v_cache;
};

struct AttnParams {
    int hkv, max_seq, splits;
    float theta;
    tagged_t *ws_ml;   // shadows of the partial softmax states
    tagged_t *ws_acc;
};

struct Buf8 {
    u32x4 q[kProgSlots];
    unsigned d[kProgSlots];  // f16 scale code, zero-extended
    float res;               // EPI_ADD: residual of the step's row (lane < r)
    unsigned res_tag;        // ... and the tag its word carried when it was fetched (see matvec_phase)
};

// One pipeline step of weights: slot i = slice (i / r), row (i % r).  Every step issues the same number of loads
// (the wait counts the compiler derives stay exact on every path): slots past r * s, and steps past a wave's
// last, read the first bytes of the planes with ordinary loads, which the compute unit's own cache serves once
// one wave has fetched the line; live slots stream past that cache.
__device__ __forceinline__ void load8(Buf8 &b, const int8_t *__restrict__ qs, const unsigned short *__restrict__ ds,
                                      int row0, int n, int k, int slice0, int r, int s, unsigned lane, bool live) {
    const int nblk = k >> 5;
    const unsigned qoff = lane * 16u, doff = (lane >> 1) * 2u;
    const int used = live ? r * s : 0;
#pragma unroll
    for (int i = 0; i < kProgSlots; ++i) {
        if (i < used) {  // wave-uniform
            const int sl = r == 2 ? (i >> 1) : i, rr = r == 2 ? (i & 1) : 0;
            const int row = min(row0 + rr, n - 1);  // rows past the end re-read the last row
            const unsigned kb = static_cast<unsigned>(slice0 + sl) * 1024u;
            const char *qrow = reinterpret_cast<const char *>(qs) + static_cast<size_t>(row) * k + kb;
            const char *drow = reinterpret_cast<const char *>(ds) + (static_cast<size_t>(row) * nblk + (kb >> 5)) * 2;
            b.q[i] = __builtin_nontemporal_load(as_global(reinterpret_cast<const u32x4 *>(qrow + qoff)));
            b.d[i] = __builtin_nontemporal_load(as_global(reinterpret_cast<const unsigned short *>(drow + doff)));
        } else {
            b.q[i] = *as_global(reinterpret_cast<const u32x4 *>(qs));
            b.d[i] = *as_global(ds);
        }
    }
    asm volatile("" ::"v"(qoff), "v"(doff));
}

// Arithmetic of compute_step (q8_gemv_device.h) on the slot layout of load8, with r and s wave-uniform run-time
// values: one code path for every step shape.  Per row the slices are taken in increasing order, each as
// acc = fma(dot16(q, x), float(d), acc), which is the order of the per-kernel matvec.
__device__ __forceinline__ void compute8(Buf8 &b, const float4 *xs4, int slice0, int r, int s, unsigned lane,
                                         float &acc0, float &acc1) {
    const int used = r * s;
    float4 xv[4];
#pragma unroll
    for (int i = 0; i < kProgSlots; ++i) {
        if (i < used) {  // wave-uniform
            if (r == 1 || (i & 1) == 0) {
                const float4 *xp = xs4 + (slice0 + (r == 2 ? (i >> 1) : i)) * 256 + lane;
#pragma unroll
                for (int j = 0; j < 4; ++j) xv[j] = xp[j * 64];
            }
            asm volatile("" : "+v"(b.q[i]), "+v"(b.d[i]));
            const float dot = dot16(b.q[i], xv);
            const float d = __half2float(__ushort_as_half(static_cast<unsigned short>(b.d[i])));
            if (r == 2 && (i & 1)) acc1 = fmaf(dot, d, acc1);
            else acc0 = fmaf(dot, d, acc0);
        }
    }
}

struct WaveCtx {
    int wave_global, total_waves;
    unsigned lane;
    int tid;
};

// What a wave needs of a matvec phase to request its steps.
struct StepGeom {
    const int8_t *qs;
    const unsigned short *ds;
    int n, k, r, s, n_groups, chunks;
};
__device__ __forceinline__ StepGeom geom_of(const ProgOp &o) {
    return StepGeom{o.qs, o.ds, o.n, o.k, o.r, o.s, o.n_groups, o.chunks};
}

// Steps 0 and 1 of a wave in the matvec phase described by `o` (dead loads when !valid or there is no such step).
__device__ __forceinline__ void load_phase_step(Buf8 &buf, const StepGeom &o, bool valid, int j, const WaveCtx &w) {
    const int my_groups = w.wave_global < o.n_groups ? (o.n_groups - w.wave_global + w.total_waves - 1) / w.total_waves : 0;
    const bool live = valid && j < my_groups * o.chunks;
    const int g = w.wave_global + ((j == 1 && o.chunks == 1) ? w.total_waves : 0);
    const int c = (j == 1 && o.chunks > 1) ? 1 : 0;
    load8(buf, o.qs, o.ds, g * o.r, o.n, o.k, c * o.s, o.r, o.s, w.lane, live);
}

// One MATVEC phase.  On entry a / b hold this wave's steps 0 / 1 of the phase; on return its steps 0 / 1 of the
// next MATVEC phase.
__device__ __forceinline__ void matvec_phase(const ProgOp *__restrict__ ops, int p, unsigned tag_base, unsigned *flags,
                                             Buf8 &a, Buf8 &b, float4 *xs4, float *red, const WaveCtx &w) {
    const ProgOp op = ops[p];
    const int R = op.r, S = op.s;
    const int k = op.k, chunks = op.chunks, n_groups = op.n_groups, n = op.n;
    const int epi = op.epi;
    const bool norm = op.norm != 0;
    const unsigned lane = w.lane;
    const int my_groups = w.wave_global < n_groups ? (n_groups - w.wave_global + w.total_waves - 1) / w.total_waves : 0;
    const int T = my_groups * chunks;
    TaggedIO io{tag_base + static_cast<unsigned>(op.x_phase) + 1u, tag_base + static_cast<unsigned>(p) + 1u, flags,
                flags + 16};
    // The next matvec phase's geometry is fetched now: by the time this phase's last steps ask for it, it is there.
    const int nx = op.next_matvec;
    const StepGeom nxt = geom_of(ops[nx >= 0 ? nx : p]);

    // Residuals of the first two steps' rows: requested now, together with the staging loads, and those of later
    // steps with their weights.  A residual written by an earlier phase of this launch comes as a tagged word like
    // every other hand-over.  Its writer need not have finished when the request goes out - nothing orders a phase
    // that this phase's input does not depend on before it - so the tag travels with the value and is looked at
    // where the value is used (settle_residual): in the usual case, the writer being the producer of an earlier
    // input of this workgroup, it is there and the check costs a compare.
    const unsigned res_tag_want = tag_base + static_cast<unsigned>(op.res_phase) + 1u;
    auto residual_row = [&](int g) -> int {
        return min(g * R + static_cast<int>(lane < static_cast<unsigned>(R) ? lane : 0u), n - 1);
    };
    auto load_residual = [&](Buf8 &buf, int g) {
        const int row = residual_row(g);
        if (op.res_t != nullptr) {
            const tagged_t raw = __hip_atomic_load(as_global(op.res_t) + row, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            buf.res = __uint_as_float(static_cast<unsigned>(raw));
            buf.res_tag = static_cast<unsigned>(raw >> 32);
        } else {
            buf.res = as_global(op.residual)[row];
            buf.res_tag = res_tag_want;
        }
    };
    // The residual of row group g as fetched into buf, or - when its word did not carry the writer's tag yet -
    // fetched again until it does (bounded like every wait of the program).
    auto settle_residual = [&](const Buf8 &buf, int g) -> float {
        float v = buf.res;
        if (op.res_t == nullptr) return v;
        bool ok = buf.res_tag == res_tag_want;
        while (io.again(__all(ok))) {
            const tagged_t raw = __hip_atomic_load(as_global(op.res_t) + residual_row(g), __ATOMIC_RELAXED,
                                                   __HIP_MEMORY_SCOPE_AGENT);
            v = __uint_as_float(static_cast<unsigned>(raw));
            ok = static_cast<unsigned>(raw >> 32) == res_tag_want;
        }
        return v;
    };
    if (epi == EPI_ADD) {
        load_residual(a, T > 0 ? w.wave_global : 0);
        load_residual(b, T > 1 ? w.wave_global + (chunks == 1 ? w.total_waves : 0) : 0);
    }

    // ---- activations to LDS: float4 index slice*256 + j*64 + lane holds x[slice*1024 + lane*16 + j*4 .. +3].
    // A thread fetches up to 7 float4 per round and, when they come from an earlier phase, repeats the round
    // until every word carries that phase's tag.  With the norm, x * gain is staged and the sum of squares is
    // taken on the way by the first 256 threads in increasing index, the order of a four-wave workgroup.
    // A workgroup none of whose waves has a row group in this phase stages nothing: it is then no reader of the
    // phase's input at all, which the host's rule for overwriting a buffer relies on (lhip_decode_program_create).
    if (static_cast<int>(blockIdx.x) * kProgWaves < n_groups) {
        constexpr int kBatch = 7;  // K = 14336 over 512 threads in one round
        const float4 *x4 = reinterpret_cast<const float4 *>(op.x);
        const float4 *g4 = reinterpret_cast<const float4 *>(op.norm_w);
        const bool tagged = op.x_phase >= 0;
        const int k4 = k >> 2;
        const int workers = norm ? 256 : kProgThreads;
        float ss = 0.f;
        if (w.tid < workers) {
            for (int i0 = w.tid; i0 < k4; i0 += kBatch * workers) {
                float4 v[kBatch];
                if (!tagged) {
#pragma unroll
                    for (int u = 0; u < kBatch; ++u) {
                        const int i = min(i0 + u * workers, k4 - 1);
                        v[u] = ldg4(x4 + ((i & ~255) | ((i & 63) << 2) | ((i >> 6) & 3)));
                    }
                } else {
                    // A round requests every word still missing before it looks at any of them, so it costs one
                    // memory round trip; words that have arrived are not requested again.
                    tagged_t raw[kBatch][4];
                    unsigned have = 0u;  // bit u: v[u] is complete
                    bool ok;
                    do {
#pragma unroll
                        for (int u = 0; u < kBatch; ++u) {
                            if ((have >> u) & 1u) continue;
                            const int i = min(i0 + u * workers, k4 - 1);
                            const int src = (i & ~255) | ((i & 63) << 2) | ((i >> 6) & 3);
#pragma unroll
                            for (int c = 0; c < 4; ++c)
                                raw[u][c] = __hip_atomic_load(as_global(op.x_t) + 4 * src + c, __ATOMIC_RELAXED,
                                                              __HIP_MEMORY_SCOPE_AGENT);
                        }
                        ok = true;
#pragma unroll
                        for (int u = 0; u < kBatch; ++u) {
                            if ((have >> u) & 1u) continue;
                            bool mine = true;
#pragma unroll
                            for (int c = 0; c < 4; ++c) mine = mine && static_cast<unsigned>(raw[u][c] >> 32) == io.in_tag;
                            if (mine) {
                                have |= 1u << u;
                                v[u] = make_float4(__uint_as_float(static_cast<unsigned>(raw[u][0])),
                                                   __uint_as_float(static_cast<unsigned>(raw[u][1])),
                                                   __uint_as_float(static_cast<unsigned>(raw[u][2])),
                                                   __uint_as_float(static_cast<unsigned>(raw[u][3])));
                            } else {
                                ok = false;
                            }
                        }
                    } while (io.again(ok));
                }
#pragma unroll
                for (int u = 0; u < kBatch; ++u) {
                    const int i = i0 + u * workers;
                    if (i < k4) {
                        if (norm) {
                            const int src = (i & ~255) | ((i & 63) << 2) | ((i >> 6) & 3);
                            const float4 g = ldg4(g4 + src);
                            ss = fmaf(v[u].x, v[u].x, ss);
                            ss = fmaf(v[u].y, v[u].y, ss);
                            ss = fmaf(v[u].z, v[u].z, ss);
                            ss = fmaf(v[u].w, v[u].w, ss);
                            xs4[i] = make_float4(v[u].x * g.x, v[u].y * g.y, v[u].z * g.z, v[u].w * g.w);
                        } else {
                            xs4[i] = v[u];
                        }
                    }
                }
            }
            if (norm) {
                ss = wave_sum(ss);
                if (lane == 0) red[w.tid >> 6] = ss;
            }
        }
    }
    __syncthreads();
    // Stores of earlier phases have been acknowledged before this phase issues its own (see the header): they
    // were issued at least one exchange ago, and the loads this also waits for are needed now anyway.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    float scale = 1.f;
    if (norm) {
        float total = 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) total += red[i];
        scale = 1.0f / sqrtf(total / static_cast<float>(k) + op.eps);
    }

    float acc0 = 0.f, acc1 = 0.f;

    auto next = [&](int &gg, int &cc) {
        if (++cc == chunks) {
            cc = 0;
            gg += w.total_waves;
        }
    };
    int g = w.wave_global, c = 0;         // step being computed
    int g2 = g, c2 = c;                   // step t + 2
    next(g2, c2);
    next(g2, c2);

    auto finish_group = [&](int gg, float res) {
        float sum0 = wave_sum(acc0), sum1 = 0.f;
        if (R == 2) sum1 = wave_sum(acc1);
        if (norm) {
            sum0 *= scale;
            sum1 *= scale;
        }
        acc0 = acc1 = 0.f;
        const int row0 = gg * R;
        if (epi == EPI_SWIGLU) {  // R == 2: rows (gate, up) of one output
            const float v = sum1 * (sum0 * (1.0f / (1.0f + expf(-sum0))));
            const int pair = row0 / 2;
            if (lane == 0 && 2 * pair + 1 < n) {
                if (op.y_t != nullptr) io.st1(reinterpret_cast<float *>(op.y_t), pair, v);
                as_global(op.y)[pair] = v;
            }
        } else {
            const float out = lane == 1 ? sum1 : sum0;
            const int row = row0 + static_cast<int>(lane);
            if (lane < static_cast<unsigned>(R) && row < n) {
                const float v = epi == EPI_ADD ? out + res : out;
                if (op.y_t != nullptr) io.st1(reinterpret_cast<float *>(op.y_t), row, v);
                as_global(op.y)[row] = v;
            }
        }
    };
    auto compute = [&](Buf8 &cur) {
        compute8(cur, xs4, c * S, R, S, lane, acc0, acc1);
        if (c == chunks - 1) finish_group(g, epi == EPI_ADD ? settle_residual(cur, g) : 0.f);
        next(g, c);
    };
    auto refill = [&](Buf8 &cur, bool live) {  // with the step (g2, c2) of this phase
        __builtin_amdgcn_sched_barrier(0);
        if (epi == EPI_ADD) load_residual(cur, live ? g2 : 0);
        load8(cur, op.qs, op.ds, g2 * R, n, k, c2 * S, R, S, lane, live);
        next(g2, c2);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto load_next = [&](Buf8 &cur, int j) {
        __builtin_amdgcn_sched_barrier(0);
        load_phase_step(cur, nxt, nx >= 0, j, w);
        __builtin_amdgcn_sched_barrier(0);
    };

    // The steps are taken in pairs (a, then b), so that a and b end the phase in the roles they started it in;
    // an odd count is padded with a dead step, which is loaded (from a cached line) but not computed.  The
    // buffer just consumed is refilled from this phase, in the last pair from the next matvec phase.
    const int Te = (T + 1) & ~1;
    int t = 0;
    for (; t + 2 < Te; t += 2) {
        compute(a);
        refill(a, t + 2 < T);
        compute(b);
        refill(b, t + 3 < T);
    }
    if (Te > 0) {
        compute(a);
        load_next(a, 0);
        if (t + 1 < T) compute(b);
        load_next(b, 1);
    } else {
        load_next(a, 0);
        load_next(b, 1);
    }
}

template <int G, int HD>
union ProgShared {
    AttnShared<G, HD> attn;
    MergeShared merge;
};

template <int G, int HD>
__global__ __launch_bounds__(kProgThreads) void decode_program_kernel(const ProgOp *__restrict__ ops, int n_ops,
                                                                      int first_matvec,
                                                                      const int *__restrict__ pos_dev,
                                                                      const AttnParams ap, unsigned *sync,
                                                                      unsigned long long *trace) {
    // dynamic LDS: staged activations or attention / merge scratch (never live together)
    extern __shared__ float4 lds4[];
    __shared__ float red[4];
    auto &sh = *reinterpret_cast<ProgShared<G, HD> *>(lds4);

    WaveCtx w;
    w.tid = threadIdx.x;
    w.lane = threadIdx.x & 63u;
    w.wave_global = blockIdx.x * kProgWaves + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    w.total_waves = gridDim.x * kProgWaves;
    const int pos = *pos_dev;
    const unsigned tag_base = sync[0] * kTagsPerLaunch;  // the launch counter was advanced by the kernel before this one
    unsigned *flags = sync + 32;                         // [0] abort flag of this launch, [16] sticky flag

    Buf8 a, b;
    a.res = b.res = 0.f;
    if (first_matvec >= 0) {
        const StepGeom first = geom_of(ops[first_matvec]);
        load_phase_step(a, first, true, 0, w);
        load_phase_step(b, first, true, 1, w);
    }

    const bool tracing = trace != nullptr && blockIdx.x == 0 && threadIdx.x == 0;
    for (int p = 0; p < n_ops; ++p) {
        if (tracing) trace[2 * p] = wall_clock64();
        const ProgOp &op = ops[p];
        // LDS changes hands: the slowest wave of the workgroup has finished the previous phase's reads of it
        __syncthreads();
        if (op.type == PHASE_MATVEC) {
            matvec_phase(ops, p, tag_base, flags, a, b, lds4, red, w);
        } else {
            TaggedIO io{tag_base + static_cast<unsigned>(op.x_phase) + 1u, tag_base + static_cast<unsigned>(p) + 1u, flags,
                        flags + 16};
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // earlier phases' stores acknowledged
            if (op.type == PHASE_ATTENTION) {
                const int items = ap.hkv * ap.splits;
                for (int item = blockIdx.x; item < items; item += gridDim.x) {
                    attention_decode_body<G, HD, kProgThreads>(io, sh.attn, item / ap.splits, item % ap.splits,
                                                               reinterpret_cast<const float *>(op.x_t), op.k_cache,
                                                               op.v_cache, pos, ap.hkv, ap.max_seq, ap.theta, ap.splits,
                                                               reinterpret_cast<float *>(ap.ws_ml),
                                                               reinterpret_cast<float4 *>(ap.ws_acc));
                    __syncthreads();
                }
            } else {
                for (int item = blockIdx.x; item < ap.hkv * G; item += gridDim.x) {
                    attention_merge_body<G, HD, kProgThreads>(io, sh.merge, item, reinterpret_cast<float *>(op.y_t), pos,
                                                              ap.max_seq, ap.splits,
                                                              reinterpret_cast<const float *>(ap.ws_ml),
                                                              reinterpret_cast<const float4 *>(ap.ws_acc), op.y);
                    __syncthreads();
                }
            }
        }
        if (tracing) trace[2 * p + 1] = wall_clock64();
    }
}

// Runs before the program kernel: next launch number (the tags of the previous launch become stale), abort flag off.
__global__ void decode_program_begin_kernel(unsigned *sync) {
    if (threadIdx.x == 0) {
        sync[0] += 1u;
        sync[32] = 0u;
    }
}

struct Program {
    int device = 0;
    int n_phases = 0, first_matvec = -1;
    int g = 0, hd = 0;          // 0: no attention phase
    int grid = 0;
    size_t lds_bytes = 0;
    AttnParams ap{};
    const int32_t *pos = nullptr;
    ProgOp *ops_dev = nullptr;
    unsigned *sync_dev = nullptr;  // kSyncWords
    void *shadow_dev = nullptr;    // every shadow array, one allocation
    unsigned long long *trace_dev = nullptr;  // caller's buffer, or null
};

template <int G, int HD>
static lhip_status launch_program(const Program &pr, hipStream_t s) {
    auto kernel = decode_program_kernel<G, HD>;
    static LdsOptIn opt;
    if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(kernel), pr.lds_bytes, pr.lds_bytes > 48 * 1024)) return st;
    hipLaunchKernelGGL(decode_program_begin_kernel, dim3(1), dim3(64), 0, s, pr.sync_dev);
    LHIP_CHECK_LAUNCH();
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(pr.grid)), dim3(kProgThreads), pr.lds_bytes, s, pr.ops_dev,
                       pr.n_phases, pr.first_matvec, pr.pos, pr.ap, pr.sync_dev, pr.trace_dev);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

template <int G, int HD>
static size_t shared_bytes() {
    return sizeof(ProgShared<G, HD>);
}

static bool prog_attention_supported(int64_t g, int64_t hd) {
    return (g == 1 || g == 2 || g == 4 || g == 8) && (hd == 64 || hd == 128);
}

// What the host knows about a caller's buffer while it lays the phases out.
struct BufferState {
    const void *base;
    size_t shadow_offset;      // in words, into the shadow allocation
    int writer;                // phase that wrote the current contents, -1: the caller
    std::vector<int> readers;  // phases that read the current contents
};

}  // namespace lhip

using namespace lhip;

extern "C" {

lhip_status lhip_decode_program_create(const lhip_decode_op *ops, int n_ops, int64_t q_heads, int64_t kv_heads,
                                       int64_t head_dim, int64_t max_seq, float theta, const int32_t *pos_dev,
                                       void **program) {
    if (!ops || !program) return LHIP_ERR_NULL_PTR;
    *program = nullptr;
    if (n_ops <= 0 || n_ops > 2048) return LHIP_ERR_INVALID_SHAPE;
    if (!pos_dev) return LHIP_ERR_NULL_PTR;  // the kernel reads it in any case
    int device = 0;
    LHIP_HIP_TRY(hipGetDevice(&device));
    hipDeviceProp_t prop;
    LHIP_HIP_TRY(hipGetDeviceProperties(&prop, device));
    const int grid = prop.multiProcessorCount;
    if (grid < 1) return LHIP_ERR_UNSUPPORTED;
    const int total_waves = grid * kProgWaves;

    bool has_attention = false;
    for (int i = 0; i < n_ops; ++i) has_attention |= ops[i].type == LHIP_DECODE_ATTENTION;
    int g = 0, splits = 0;
    if (has_attention) {
        if (q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || max_seq <= 0 || q_heads % kv_heads != 0 ||
            max_seq > kMaxDim || kv_heads > 65535)
            return LHIP_ERR_INVALID_SHAPE;
        if (!prog_attention_supported(q_heads / kv_heads, head_dim)) return LHIP_ERR_UNSUPPORTED;
        g = static_cast<int>(q_heads / kv_heads);
        splits = dec_splits(kv_heads);
    }

    // Buffers the operations name, by base address.  A buffer written by a phase gets a shadow array of tagged
    // words that later phases read instead of it.
    std::vector<BufferState> buffers;
    size_t shadow_words = 0;
    auto find = [&](const void *base) -> BufferState * {
        for (auto &b : buffers)
            if (b.base == base) return &b;
        return nullptr;
    };
    // A read of `base` by phase `reader`: the phase whose tag to expect (-1: plain read) and the shadow's offset.
    // own = the in-place residual, which the writing thread reads itself before it writes: no hazard, not noted.
    auto note_read = [&](const void *base, int reader, bool own, size_t *offset) -> int {
        BufferState *b = find(base);
        if (!b) {
            buffers.push_back(BufferState{base, SIZE_MAX, -1, {}});
            if (!own) buffers.back().readers.push_back(reader);
            return -1;
        }
        if (!own) b->readers.push_back(reader);
        *offset = b->shadow_offset;
        return b->writer;
    };
    // A write of `words` values to `base` by phase `writer` whose own input comes from phase `input_phase`.
    // A workgroup that writes has seen the whole output of `input_phase`, so every workgroup that works in that
    // phase has finished reading its input, has finished every earlier phase it works in (a workgroup takes the
    // phases in order) and (a wave waits for its stores to be acknowledged before it stores for a later phase)
    // has seen every store it issued up to then land; the same holds, step by step, for the phase that produced
    // that input, and so on back along the chain of inputs.  The workgroups that work in a phase are the first
    // workers[phase] of the grid, and one that does not work in a phase does not read its input either.  So a
    // phase r that read or wrote the old contents is known to be done with them if it lies on that chain, or if
    // some later phase on the chain employs at least as many workgroups as r does; anything else (a phase the
    // writer's input does not depend on may still be running somewhere) is refused.
    std::vector<ProgOp> phases;
    std::vector<int> workers;
    auto settled = [&](int phase, int from) -> bool {
        for (int q = from; q >= phase; q = phases[static_cast<size_t>(q)].x_phase) {
            if (q == phase) return true;
            // every one of a matvec's or a merge's first workers[q] workgroups does work in it; of an attention
            // phase's only those whose key range holds keys at the current position
            if (phases[static_cast<size_t>(q)].type != PHASE_ATTENTION &&
                workers[static_cast<size_t>(q)] >= workers[static_cast<size_t>(phase)])
                return true;
        }
        return false;
    };
    auto note_write = [&](const void *base, size_t words, int writer, int input_phase, size_t *offset) -> bool {
        BufferState *b = find(base);
        if (!b) {
            buffers.push_back(BufferState{base, SIZE_MAX, -1, {}});
            b = &buffers.back();
        }
        if (b->writer >= 0 && !settled(b->writer, input_phase)) return false;
        for (int r : b->readers)
            if (r != writer && !settled(r, input_phase)) return false;
        if (b->shadow_offset == SIZE_MAX) {
            b->shadow_offset = shadow_words;
            shadow_words += (words + 31) & ~size_t{31};
        }
        b->writer = writer;
        b->readers.clear();
        *offset = b->shadow_offset;
        return true;
    };

    struct Pending {  // offsets are turned into pointers once the shadow allocation exists
        size_t x = SIZE_MAX, y = SIZE_MAX, res = SIZE_MAX;
    };
    std::vector<Pending> pend;
    size_t max_k = 0;
    size_t ws_ml_off = SIZE_MAX, ws_acc_off = SIZE_MAX;
    int ws_last_reader = -1;  // latest merge phase that reads the partial states
    if (has_attention) {
        ws_ml_off = shadow_words;
        shadow_words += dec_ml_bytes(kv_heads, splits, g) / sizeof(float);
        ws_acc_off = shadow_words;
        shadow_words += static_cast<size_t>(kv_heads) * splits * g * static_cast<size_t>(head_dim);
    }
    for (int i = 0; i < n_ops; ++i) {
        const lhip_decode_op &o = ops[i];
        const int p = static_cast<int>(phases.size());
        ProgOp ph{};
        Pending pe;
        ph.next_matvec = -1;
        ph.x_phase = -1;
        if (o.type == LHIP_DECODE_MATVEC) {
            if (!o.planar || !o.x || !o.y) return LHIP_ERR_NULL_PTR;
            if (lhip_status st = check_q8_shape(o.n, o.k)) return st;
            if (o.k % 1024 != 0 || o.k > kProgMaxK) return LHIP_ERR_UNSUPPORTED;
            if (o.epilogue < LHIP_FUSE_NONE || o.epilogue > LHIP_FUSE_SWIGLU) return LHIP_ERR_INVALID_SHAPE;
            if (o.epilogue == LHIP_FUSE_ADD && !o.residual) return LHIP_ERR_NULL_PTR;
            if (o.epilogue == LHIP_FUSE_SWIGLU && o.n % 2 != 0) return LHIP_ERR_INVALID_SHAPE;
            if (!aligned(o.planar, 256) || !aligned(o.x, 16) || !aligned(o.y, 4) ||
                (o.norm_weight && !aligned(o.norm_weight, 16)) || (o.residual && !aligned(o.residual, 4)))
                return LHIP_ERR_MISALIGNED;
            if (o.x == o.y) return LHIP_ERR_INVALID_SHAPE;
            const int slices = static_cast<int>(o.k / 1024);
            ph.type = PHASE_MATVEC;
            ph.s = slices % 4 == 0 ? 4 : slices % 7 == 0 ? 7 : slices % 2 == 0 ? 2 : 1;
            // two rows per wave where SwiGLU pairs need it, or where that still leaves every wave two row groups
            ph.r = (ph.s <= 4 && (o.epilogue == LHIP_FUSE_SWIGLU || o.n / 2 >= 2 * static_cast<int64_t>(total_waves))) ? 2 : 1;
            if (o.epilogue == LHIP_FUSE_SWIGLU && ph.r != 2) return LHIP_ERR_UNSUPPORTED;
            ph.n = static_cast<int>(o.n);
            ph.k = static_cast<int>(o.k);
            ph.n_groups = (ph.n + ph.r - 1) / ph.r;
            ph.chunks = slices / ph.s;
            ph.epi = o.epilogue;
            ph.norm = o.norm_weight != nullptr;
            ph.eps = o.eps;
            auto *base = static_cast<const uint8_t *>(o.planar);
            ph.qs = reinterpret_cast<const int8_t *>(base);
            ph.ds = reinterpret_cast<const unsigned short *>(base + q8_scale_offset(o.n, o.k));
            ph.x = o.x;
            ph.y = o.y;
            ph.norm_w = o.norm_weight;
            ph.residual = o.epilogue == LHIP_FUSE_ADD ? o.residual : nullptr;
            ph.x_phase = note_read(o.x, p, false, &pe.x);
            ph.res_phase = ph.residual ? note_read(ph.residual, p, ph.residual == o.y, &pe.res) : -1;
            if (ph.res_phase < 0) pe.res = SIZE_MAX;
            const size_t out_words = static_cast<size_t>(o.epilogue == LHIP_FUSE_SWIGLU ? o.n / 2 : o.n);
            if (!note_write(o.y, out_words, p, ph.x_phase, &pe.y)) return LHIP_ERR_UNSUPPORTED;
            max_k = o.k > static_cast<int64_t>(max_k) ? static_cast<size_t>(o.k) : max_k;
            phases.push_back(ph);
            workers.push_back(std::min(grid, (ph.n_groups + kProgWaves - 1) / kProgWaves));
            pend.push_back(pe);
        } else if (o.type == LHIP_DECODE_ATTENTION) {
            if (!o.x || !o.y || !o.k_cache || !o.v_cache) return LHIP_ERR_NULL_PTR;
            if (!aligned(o.x, 16) || !aligned(o.y, 16) || !aligned(o.k_cache, 16) || !aligned(o.v_cache, 16))
                return LHIP_ERR_MISALIGNED;
            if (o.x == o.y) return LHIP_ERR_INVALID_SHAPE;
            ph.type = PHASE_ATTENTION;
            ph.x = o.x;
            ph.k_cache = o.k_cache;
            ph.v_cache = o.v_cache;
            ph.x_phase = note_read(o.x, p, false, &pe.x);
            // the body reads its input through the tagged accessors: it must come from a phase of this program
            if (ph.x_phase < 0) return LHIP_ERR_UNSUPPORTED;
            if (ws_last_reader >= 0 && !settled(ws_last_reader, ph.x_phase)) return LHIP_ERR_UNSUPPORTED;  // the previous merge may still be reading
            phases.push_back(ph);
            workers.push_back(std::min(grid, static_cast<int>(kv_heads) * splits));
            pend.push_back(pe);
            ProgOp m{};
            Pending pm;
            m.next_matvec = -1;
            m.type = PHASE_MERGE;
            m.x_phase = p;  // the partial states of the attention phase
            m.y = o.y;
            ws_last_reader = p + 1;
            if (!note_write(o.y, static_cast<size_t>(q_heads * head_dim), p + 1, p, &pm.y)) return LHIP_ERR_UNSUPPORTED;
            phases.push_back(m);
            workers.push_back(std::min(grid, static_cast<int>(q_heads)));
            pend.push_back(pm);
        } else {
            return LHIP_ERR_INVALID_SHAPE;
        }
    }
    int next = -1, first = -1;
    for (int i = static_cast<int>(phases.size()) - 1; i >= 0; --i) {
        phases[i].next_matvec = next;
        if (phases[i].type == PHASE_MATVEC) next = first = i;
    }

    auto *pr = new (std::nothrow) Program();
    if (!pr) return LHIP_ERR_HIP;
    pr->device = device;
    pr->n_phases = static_cast<int>(phases.size());
    pr->first_matvec = first;
    pr->grid = grid;
    pr->pos = pos_dev;
    pr->g = g;
    pr->hd = static_cast<int>(head_dim);
    size_t scratch = 0;
    if (has_attention) {
#define LHIP_CASE(G, HD) \
    if (g == G && head_dim == HD) scratch = shared_bytes<G, HD>();
        LHIP_CASE(1, 64) LHIP_CASE(2, 64) LHIP_CASE(4, 64) LHIP_CASE(8, 64)
        LHIP_CASE(1, 128) LHIP_CASE(2, 128) LHIP_CASE(4, 128) LHIP_CASE(8, 128)
#undef LHIP_CASE
    }
    pr->lds_bytes = max_k * 4 > scratch ? max_k * 4 : scratch;
    if (pr->lds_bytes < 16) pr->lds_bytes = 16;

    auto fail = [&](lhip_status s) {
        lhip_decode_program_destroy(pr);
        return s;
    };
    const size_t shadow_bytes = (shadow_words ? shadow_words : 1) * sizeof(tagged_t);
    if (hipMalloc(&pr->ops_dev, phases.size() * sizeof(ProgOp)) != hipSuccess) return fail(LHIP_ERR_HIP);
    if (hipMalloc(&pr->sync_dev, kSyncWords * sizeof(unsigned)) != hipSuccess) return fail(LHIP_ERR_HIP);
    if (hipMemset(pr->sync_dev, 0, kSyncWords * sizeof(unsigned)) != hipSuccess) return fail(LHIP_ERR_HIP);
    if (hipMalloc(&pr->shadow_dev, shadow_bytes) != hipSuccess) return fail(LHIP_ERR_HIP);
    if (hipMemset(pr->shadow_dev, 0, shadow_bytes) != hipSuccess) return fail(LHIP_ERR_HIP);  // tag 0: never valid
    auto *shadow = static_cast<tagged_t *>(pr->shadow_dev);
    for (size_t i = 0; i < phases.size(); ++i) {
        if (pend[i].x != SIZE_MAX && phases[i].x_phase >= 0) phases[i].x_t = shadow + pend[i].x;
        if (pend[i].y != SIZE_MAX) phases[i].y_t = shadow + pend[i].y;
        if (pend[i].res != SIZE_MAX) phases[i].res_t = shadow + pend[i].res;
    }
    if (has_attention) {
        pr->ap.hkv = static_cast<int>(kv_heads);
        pr->ap.max_seq = static_cast<int>(max_seq);
        pr->ap.splits = splits;
        pr->ap.theta = theta;
        pr->ap.ws_ml = shadow + ws_ml_off;
        pr->ap.ws_acc = shadow + ws_acc_off;
    }
    if (hipMemcpy(pr->ops_dev, phases.data(), phases.size() * sizeof(ProgOp), hipMemcpyHostToDevice) != hipSuccess)
        return fail(LHIP_ERR_HIP);
    *program = pr;
    return LHIP_OK;
}

lhip_status lhip_decode_program_run(void *program, void *stream) {
    if (!program) return LHIP_ERR_NULL_PTR;
    const Program &pr = *static_cast<const Program *>(program);
    hipStream_t s = as_stream(stream);
    if (pr.g == 0) return launch_program<1, 64>(pr, s);  // no attention phase: any instantiation serves
#define LHIP_CASE(G, HD) \
    if (pr.g == G && pr.hd == HD) return launch_program<G, HD>(pr, s);
    LHIP_CASE(1, 64) LHIP_CASE(2, 64) LHIP_CASE(4, 64) LHIP_CASE(8, 64)
    LHIP_CASE(1, 128) LHIP_CASE(2, 128) LHIP_CASE(4, 128) LHIP_CASE(8, 128)
#undef LHIP_CASE
    return LHIP_ERR_UNSUPPORTED;
}

lhip_status lhip_decode_program_trace(void *program, uint64_t *ticks_dev, int32_t *n_phases) {
    if (!program) return LHIP_ERR_NULL_PTR;
    auto *pr = static_cast<Program *>(program);
    if (ticks_dev && !aligned(ticks_dev, 8)) return LHIP_ERR_MISALIGNED;
    pr->trace_dev = reinterpret_cast<unsigned long long *>(ticks_dev);
    if (n_phases) *n_phases = pr->n_phases;
    return LHIP_OK;
}

lhip_status lhip_decode_program_status(void *program, int32_t *timed_out) {
    if (!program || !timed_out) return LHIP_ERR_NULL_PTR;
    const Program &pr = *static_cast<const Program *>(program);
    unsigned flag = 0;
    LHIP_HIP_TRY(hipMemcpy(&flag, pr.sync_dev + 48, sizeof(flag), hipMemcpyDeviceToHost));
    *timed_out = flag != 0;
    return LHIP_OK;
}

lhip_status lhip_decode_program_destroy(void *program) {
    if (!program) return LHIP_OK;
    auto *pr = static_cast<Program *>(program);
    if (pr->ops_dev) (void)hipFree(pr->ops_dev);
    if (pr->sync_dev) (void)hipFree(pr->sync_dev);
    if (pr->shadow_dev) (void)hipFree(pr->shadow_dev);
    delete pr;
    return LHIP_OK;
}

}  // extern "C"
