// Persistent decode program: a whole batch-1 decode step (every layer's matvecs and attention, then the
// vocabulary projection) as ONE launch.
//
// Why.  Launched one by one, the kernels of a Llama-3-8B step each stream their weights at close to the HBM
// rate once they are going, but every launch pays ~7 us around that: ~3 us between the end of one kernel and
// the first wave of the next, ~2.5 us until the first weights and the staged activations have arrived, ~1.3 us
// while the slowest waves finish.  With 6 launches per layer that is 40 us of a 65 us layer.  Here the grid
// (one workgroup of 8 wavefronts per compute unit) stays resident and walks a list of phases; consecutive
// phases are separated by a grid-wide barrier (~2.6 us), and the weight stream does not stop there: weights do
// not depend on the previous phase, so every wave requests the first two pipeline steps of the next matvec
// before it arrives at the barrier and holds them in registers across it.
//
// Phases.  MATVEC: the fused Q8_0 matvec of q8_gemv.hip (optional RMS-norm prologue; epilogues none / residual
// add / SwiGLU) with the same per-row arithmetic and the same reduction orders, so results equal the per-kernel
// path bit for bit where that path runs four-wave workgroups.  ATTENTION and MERGE: the bodies of
// attention_decode_device.h, one (KV head, key range) piece or one KV head per workgroup.
//
// Coherence.  Data produced in one phase and consumed in a later one (activation vectors, attention partials)
// crosses between workgroups of one launch, so it is written and read with agent-coherent accesses; no cache
// write-back or invalidate is needed at the barrier, which is what makes it cheap.  A wave waits for its own
// stores to be acknowledged, the workgroup meets, one thread adds to one of 8 arrival counters and the first
// wave polls all 8 with one load.  Weights, norm gains and the KV caches of earlier positions are read-only
// within a launch and use plain (non-temporal) loads.
//
// Termination.  Every wait is bounded: a workgroup that polls kSpinLimit times without seeing the others raises
// a flag, everyone who sees the flag stops waiting, and the kernel runs to its end (with meaningless results).
// The flag is sticky and reported by lhip_decode_program_status.  All workgroups must be resident at once:
// the grid is one workgroup per compute unit, which the register and LDS budget of the kernel guarantees.
#include <hip/hip_fp16.h>
#include <limits.h>

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
constexpr unsigned kSpinLimit = 1u << 20;
constexpr int kSyncGroups = 8;           // arrival counters
constexpr int kSyncStride = 32;          // unsigned words between counters (128 B)
constexpr int kSyncWords = kSyncGroups * kSyncStride + kSyncStride;  // counters, then the abort flag

enum { PHASE_MATVEC = 0, PHASE_ATTENTION = 1, PHASE_MERGE = 2 };
enum { EPI_NONE = 0, EPI_ADD = 1, EPI_SWIGLU = 2 };

struct ProgOp {
    int type;
    int r, s;          // MATVEC: rows per wave and 1024-quant slices per pipeline step, r * s <= kProgSlots
    int n, k, n_groups, chunks;
    int epi, norm;
    float eps;
    int next_matvec;   // index of the next MATVEC phase, -1 if none
    const int8_t *qs;
    const unsigned short *ds;
    const float *x;    // MATVEC: activations (K);  ATTENTION: fused qkv row
    float *y;          // MATVEC: output;  MERGE: attention output rows
    const float *norm_w;
    const float *residual;
    float *k_cache, *v_cache;
};

struct AttnParams {
    int hkv, max_seq, splits;
    float theta;
    float *ws_ml;
    float4 *ws_acc;
};

struct Buf8 {
    u32x4 q[kProgSlots];
    unsigned d[kProgSlots];  // f16 scale code, zero-extended
    float res;               // EPI_ADD: residual of the step's row (lane < r)
};

// One pipeline step of weights: slot i = slice (i / r), row (i % r); slots past r * s and dead steps aim at the
// first bytes of the planes (one cached line), so every step issues the same number of loads.
__device__ __forceinline__ void load8(Buf8 &b, const int8_t *__restrict__ qs, const unsigned short *__restrict__ ds,
                                      int row0, int n, int k, int slice0, int r, int s, unsigned lane, bool live) {
    const int nblk = k >> 5;
    const unsigned qoff = lane * 16u, doff = (lane >> 1) * 2u;
    const int used = live ? r * s : 0;
#pragma unroll
    for (int i = 0; i < kProgSlots; ++i) {
        const bool on = i < used;
        const int sl = r == 2 ? (i >> 1) : i, rr = r == 2 ? (i & 1) : 0;
        const int row = on ? min(row0 + rr, n - 1) : 0;  // rows past the end re-read the last row
        const unsigned kb = on ? static_cast<unsigned>(slice0 + sl) * 1024u : 0u;
        const char *qrow = reinterpret_cast<const char *>(qs) + static_cast<size_t>(row) * k + kb;
        const char *drow = reinterpret_cast<const char *>(ds) + (static_cast<size_t>(row) * nblk + (kb >> 5)) * 2;
        b.q[i] = __builtin_nontemporal_load(as_global(reinterpret_cast<const u32x4 *>(qrow + (on ? qoff : 0u))));
        b.d[i] = __builtin_nontemporal_load(as_global(reinterpret_cast<const unsigned short *>(drow + (on ? doff : 0u))));
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

// Grid-wide barrier number `phase` (1, 2, ...).  `aborted` is workgroup-uniform on return.
__device__ __forceinline__ void grid_barrier(unsigned *sync, unsigned phase, unsigned *sticky, bool &aborted,
                                             unsigned *flag_lds) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's stores have been acknowledged
    __syncthreads();
    if (threadIdx.x < 64) {
        unsigned *abort_flag = sync + kSyncGroups * kSyncStride;
        if (threadIdx.x == 0)
            __hip_atomic_fetch_add(sync + (blockIdx.x % kSyncGroups) * kSyncStride, 1u, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        const unsigned lane = threadIdx.x;
        // workgroups that add to counter `lane`
        const unsigned members = lane < kSyncGroups ? (gridDim.x - lane + kSyncGroups - 1) / kSyncGroups : 0u;
        const unsigned want = phase * members;
        bool stop = aborted;
        unsigned spins = 0;
        while (!stop) {
            unsigned v = want;
            if (lane < kSyncGroups)
                v = __hip_atomic_load(sync + lane * kSyncStride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            else if (lane == kSyncGroups)
                stop = __hip_atomic_load(abort_flag, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u;
            if (__builtin_amdgcn_ballot_w64(v >= want) == ~0ull) break;
            if (++spins > kSpinLimit) {
                if (lane == 0) {
                    __hip_atomic_store(abort_flag, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    __hip_atomic_store(sticky, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
                stop = true;
            }
            stop = __builtin_amdgcn_ballot_w64(stop) != 0ull;
        }
        if (lane == 0) *flag_lds = stop ? 1u : 0u;
    }
    __syncthreads();
    aborted = *flag_lds != 0u;
}

struct WaveCtx {
    int wave_global, total_waves;
    unsigned lane;
    int tid;
};

// Steps 0 and 1 of a wave in matvec phase `idx` (dead loads when there is no such phase or step).
__device__ __forceinline__ void load_phase_step(Buf8 &buf, const ProgOp *__restrict__ ops, int idx, int fallback, int j,
                                                const WaveCtx &w) {
    const ProgOp &o = ops[idx >= 0 ? idx : fallback];
    const int my_groups = w.wave_global < o.n_groups ? (o.n_groups - w.wave_global + w.total_waves - 1) / w.total_waves : 0;
    const bool live = idx >= 0 && j < my_groups * o.chunks;
    const int g = w.wave_global + ((j == 1 && o.chunks == 1) ? w.total_waves : 0);
    const int c = (j == 1 && o.chunks > 1) ? 1 : 0;
    load8(buf, o.qs, o.ds, g * o.r, o.n, o.k, c * o.s, o.r, o.s, w.lane, live);
}

// One MATVEC phase.  On entry a / b hold this wave's steps 0 / 1 of the phase; on return its steps 0 / 1 of the
// next MATVEC phase.
__device__ __forceinline__ void matvec_phase(const ProgOp *__restrict__ ops, int p, Buf8 &a, Buf8 &b, float4 *xs4,
                                             float *red, const WaveCtx &w) {
    const ProgOp &op = ops[p];
    const int R = op.r, S = op.s;
    const int k = op.k, chunks = op.chunks, n_groups = op.n_groups, n = op.n;
    const int epi = op.epi;
    const bool norm = op.norm != 0;
    const unsigned lane = w.lane;
    const int my_groups = w.wave_global < n_groups ? (n_groups - w.wave_global + w.total_waves - 1) / w.total_waves : 0;
    const int T = my_groups * chunks;

    // Residuals of the first two steps' rows: requested now, together with the staging loads.
    auto residual_of = [&](int g) -> float {
        const int row = min(g * R + static_cast<int>(lane < static_cast<unsigned>(R) ? lane : 0u), n - 1);
        return ld_agent(op.residual + row);
    };
    if (epi == EPI_ADD) {
        a.res = residual_of(T > 0 ? w.wave_global : 0);
        b.res = residual_of(T > 1 ? w.wave_global + (chunks == 1 ? w.total_waves : 0) : 0);
    }

    // ---- activations to LDS: float4 index slice*256 + j*64 + lane holds x[slice*1024 + lane*16 + j*4 .. +3].
    // With the norm, x * gain is staged and the sum of squares rides on the loads; the first 256 threads do it,
    // which keeps the order of that sum the one of a four-wave workgroup.
    {
        const float4 *x4 = reinterpret_cast<const float4 *>(op.x);
        const int k4 = k >> 2;
        if (norm) {
            const float4 *g4 = reinterpret_cast<const float4 *>(op.norm_w);
            float ss = 0.f;
            if (w.tid < 256) {
#pragma unroll 4
                for (int i = w.tid; i < k4; i += 256) {
                    const int src = (i & ~255) | ((i & 63) << 2) | ((i >> 6) & 3);
                    float4 v = ld_agent4(x4 + src);
                    const float4 g = ldg4(g4 + src);
                    ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
                    xs4[i] = make_float4(v.x * g.x, v.y * g.y, v.z * g.z, v.w * g.w);
                }
                ss = wave_sum(ss);
                if (lane == 0) red[w.tid >> 6] = ss;
            }
        } else {
#pragma unroll 4
            for (int i = w.tid; i < k4; i += kProgThreads) {
                const int src = (i & ~255) | ((i & 63) << 2) | ((i >> 6) & 3);
                xs4[i] = ld_agent4(x4 + src);
            }
        }
    }
    __syncthreads();
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
            if (lane == 0 && 2 * pair + 1 < n) st_agent(op.y + pair, v);
        } else {
            const float out = lane == 1 ? sum1 : sum0;
            const int row = row0 + static_cast<int>(lane);
            if (lane < static_cast<unsigned>(R) && row < n) st_agent(op.y + row, epi == EPI_ADD ? out + res : out);
        }
    };
    auto compute = [&](Buf8 &cur) {
        compute8(cur, xs4, c * S, R, S, lane, acc0, acc1);
        if (c == chunks - 1) finish_group(g, cur.res);
        next(g, c);
    };
    auto refill = [&](Buf8 &cur, bool live) {  // with the step (g2, c2) of this phase
        __builtin_amdgcn_sched_barrier(0);
        if (epi == EPI_ADD) cur.res = residual_of(live ? g2 : 0);
        load8(cur, op.qs, op.ds, g2 * R, n, k, c2 * S, R, S, lane, live);
        next(g2, c2);
        __builtin_amdgcn_sched_barrier(0);
    };
    const int nx = op.next_matvec;
    auto load_next = [&](Buf8 &cur, int j) {
        __builtin_amdgcn_sched_barrier(0);
        load_phase_step(cur, ops, nx, p, j, w);
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
    MergeShared<G> merge;
};

template <int G, int HD>
__global__ __launch_bounds__(kProgThreads) void decode_program_kernel(const ProgOp *__restrict__ ops, int n_ops,
                                                                      int first_matvec,
                                                                      const int *__restrict__ pos_dev,
                                                                      const AttnParams ap, unsigned *sync,
                                                                      unsigned *sticky) {
    // dynamic LDS: [staged activations | attention / merge scratch] (never live together), then red[4], flag
    extern __shared__ float4 lds4[];
    __shared__ float red[4];
    __shared__ unsigned flag_lds;
    auto &sh = *reinterpret_cast<ProgShared<G, HD> *>(lds4);

    WaveCtx w;
    w.tid = threadIdx.x;
    w.lane = threadIdx.x & 63u;
    w.wave_global = blockIdx.x * kProgWaves + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    w.total_waves = gridDim.x * kProgWaves;
    const int pos = *pos_dev;
    bool aborted = false;

    Buf8 a, b;
    a.res = b.res = 0.f;
    if (first_matvec >= 0) {
        load_phase_step(a, ops, first_matvec, first_matvec, 0, w);
        load_phase_step(b, ops, first_matvec, first_matvec, 1, w);
    }

    for (int p = 0; p < n_ops; ++p) {
        if (p > 0) grid_barrier(sync, static_cast<unsigned>(p), sticky, aborted, &flag_lds);
        const ProgOp &op = ops[p];
        if (op.type == PHASE_MATVEC) {
            matvec_phase(ops, p, a, b, lds4, red, w);
        } else if (op.type == PHASE_ATTENTION) {
            const int items = ap.hkv * ap.splits;
            for (int item = blockIdx.x; item < items; item += gridDim.x) {
                attention_decode_body<G, HD, kProgThreads, true>(sh.attn, item / ap.splits, item % ap.splits, op.x,
                                                                 op.k_cache, op.v_cache, pos, ap.hkv, ap.max_seq,
                                                                 ap.theta, ap.splits, ap.ws_ml, ap.ws_acc);
                __syncthreads();
            }
        } else {
            for (int item = blockIdx.x; item < ap.hkv; item += gridDim.x) {
                attention_merge_body<G, HD, kProgThreads, true>(sh.merge, item, op.y, pos, ap.max_seq, ap.splits,
                                                                ap.ws_ml, ap.ws_acc);
                __syncthreads();
            }
        }
    }
}

__global__ void decode_program_clear_kernel(unsigned *sync) {
    for (int i = threadIdx.x; i < kSyncWords; i += blockDim.x) sync[i] = 0u;
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
    unsigned *sync_dev = nullptr;  // kSyncWords, then the sticky flag
    void *ws_dev = nullptr;
};

template <int G, int HD>
static lhip_status launch_program(const Program &pr, hipStream_t s) {
    auto kernel = decode_program_kernel<G, HD>;
    if (pr.lds_bytes > 48 * 1024)
        LHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                         static_cast<int>(pr.lds_bytes)));
    hipLaunchKernelGGL(decode_program_clear_kernel, dim3(1), dim3(256), 0, s, pr.sync_dev);
    LHIP_CHECK_LAUNCH();
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(pr.grid)), dim3(kProgThreads), pr.lds_bytes, s, pr.ops_dev,
                       pr.n_phases, pr.first_matvec, pr.pos, pr.ap, pr.sync_dev, pr.sync_dev + kSyncWords);
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

}  // namespace lhip

using namespace lhip;

extern "C" {

lhip_status lhip_decode_program_create(const lhip_decode_op *ops, int n_ops, int64_t q_heads, int64_t kv_heads,
                                       int64_t head_dim, int64_t max_seq, float theta, const int32_t *pos_dev,
                                       void **program) {
    if (!ops || !program) return LHIP_ERR_NULL_PTR;
    *program = nullptr;
    if (n_ops <= 0 || n_ops > 4096) return LHIP_ERR_INVALID_SHAPE;
    int device = 0;
    LHIP_HIP_TRY(hipGetDevice(&device));
    hipDeviceProp_t prop;
    LHIP_HIP_TRY(hipGetDeviceProperties(&prop, device));
    const int grid = prop.multiProcessorCount;
    if (grid < kSyncGroups) return LHIP_ERR_UNSUPPORTED;
    const int total_waves = grid * kProgWaves;

    bool has_attention = false;
    for (int i = 0; i < n_ops; ++i) has_attention |= ops[i].type == LHIP_DECODE_ATTENTION;
    int g = 0;
    if (has_attention) {
        if (!pos_dev) return LHIP_ERR_NULL_PTR;
        if (q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || max_seq <= 0 || q_heads % kv_heads != 0 ||
            max_seq > kMaxDim || kv_heads > 65535)
            return LHIP_ERR_INVALID_SHAPE;
        if (!prog_attention_supported(q_heads / kv_heads, head_dim)) return LHIP_ERR_UNSUPPORTED;
        g = static_cast<int>(q_heads / kv_heads);
    } else if (!pos_dev) {
        return LHIP_ERR_NULL_PTR;  // the kernel reads it in any case
    }

    std::vector<ProgOp> phases;
    size_t max_k = 0;
    for (int i = 0; i < n_ops; ++i) {
        const lhip_decode_op &o = ops[i];
        ProgOp p{};
        p.next_matvec = -1;
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
            const int slices = static_cast<int>(o.k / 1024);
            p.type = PHASE_MATVEC;
            p.s = slices % 4 == 0 ? 4 : slices % 7 == 0 ? 7 : slices % 2 == 0 ? 2 : 1;
            // two rows per wave where SwiGLU pairs need it, or where that still leaves every wave two row groups
            p.r = (p.s <= 4 && (o.epilogue == LHIP_FUSE_SWIGLU || o.n / 2 >= 2 * static_cast<int64_t>(total_waves))) ? 2 : 1;
            if (o.epilogue == LHIP_FUSE_SWIGLU && p.r != 2) return LHIP_ERR_UNSUPPORTED;
            p.n = static_cast<int>(o.n);
            p.k = static_cast<int>(o.k);
            p.n_groups = (p.n + p.r - 1) / p.r;
            p.chunks = slices / p.s;
            p.epi = o.epilogue;
            p.norm = o.norm_weight != nullptr;
            p.eps = o.eps;
            auto *base = static_cast<const uint8_t *>(o.planar);
            p.qs = reinterpret_cast<const int8_t *>(base);
            p.ds = reinterpret_cast<const unsigned short *>(base + q8_scale_offset(o.n, o.k));
            p.x = o.x;
            p.y = o.y;
            p.norm_w = o.norm_weight;
            p.residual = o.residual;
            max_k = o.k > static_cast<int64_t>(max_k) ? static_cast<size_t>(o.k) : max_k;
            phases.push_back(p);
        } else if (o.type == LHIP_DECODE_ATTENTION) {
            if (!o.x || !o.y || !o.k_cache || !o.v_cache) return LHIP_ERR_NULL_PTR;
            if (!aligned(o.x, 16) || !aligned(o.y, 16) || !aligned(o.k_cache, 16) || !aligned(o.v_cache, 16))
                return LHIP_ERR_MISALIGNED;
            p.type = PHASE_ATTENTION;
            p.x = o.x;
            p.k_cache = o.k_cache;
            p.v_cache = o.v_cache;
            phases.push_back(p);
            ProgOp m{};
            m.next_matvec = -1;
            m.type = PHASE_MERGE;
            m.y = o.y;
            phases.push_back(m);
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

    lhip_status st = LHIP_OK;
    auto fail = [&](lhip_status s) {
        lhip_decode_program_destroy(pr);
        return s;
    };
    if (hipMalloc(&pr->ops_dev, phases.size() * sizeof(ProgOp)) != hipSuccess) return fail(LHIP_ERR_HIP);
    if (hipMalloc(&pr->sync_dev, (kSyncWords + kSyncStride) * sizeof(unsigned)) != hipSuccess) return fail(LHIP_ERR_HIP);
    if (hipMemset(pr->sync_dev, 0, (kSyncWords + kSyncStride) * sizeof(unsigned)) != hipSuccess) return fail(LHIP_ERR_HIP);
    if (has_attention) {
        const int splits = dec_splits(kv_heads);
        const size_t ml = dec_ml_bytes(kv_heads, splits, g);
        const size_t total = ml + static_cast<size_t>(kv_heads) * splits * g * static_cast<size_t>(head_dim) * sizeof(float);
        if (hipMalloc(&pr->ws_dev, total) != hipSuccess) return fail(LHIP_ERR_HIP);
        pr->ap.hkv = static_cast<int>(kv_heads);
        pr->ap.max_seq = static_cast<int>(max_seq);
        pr->ap.splits = splits;
        pr->ap.theta = theta;
        pr->ap.ws_ml = static_cast<float *>(pr->ws_dev);
        pr->ap.ws_acc = reinterpret_cast<float4 *>(static_cast<uint8_t *>(pr->ws_dev) + ml);
    }
    if (hipMemcpy(pr->ops_dev, phases.data(), phases.size() * sizeof(ProgOp), hipMemcpyHostToDevice) != hipSuccess)
        return fail(LHIP_ERR_HIP);
    (void)st;
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

lhip_status lhip_decode_program_status(void *program, int32_t *timed_out) {
    if (!program || !timed_out) return LHIP_ERR_NULL_PTR;
    const Program &pr = *static_cast<const Program *>(program);
    unsigned flag = 0;
    LHIP_HIP_TRY(hipMemcpy(&flag, pr.sync_dev + kSyncWords, sizeof(flag), hipMemcpyDeviceToHost));
    *timed_out = flag != 0;
    return LHIP_OK;
}

lhip_status lhip_decode_program_destroy(void *program) {
    if (!program) return LHIP_OK;
    auto *pr = static_cast<Program *>(program);
    if (pr->ops_dev) (void)hipFree(pr->ops_dev);
    if (pr->sync_dev) (void)hipFree(pr->sync_dev);
    if (pr->ws_dev) (void)hipFree(pr->ws_dev);
    delete pr;
    return LHIP_OK;
}

}  // extern "C"
