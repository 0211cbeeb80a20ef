// Device code of batch-1 decode attention (rotary + cache append + split-KV attention, and the merge of the
// partial softmax states), shared by the two-launch form (attention_decode.hip) and by the persistent decode
// program (decode_program.hip), where both run as phases of one kernel.
//
// Every sum of products below is spelled as explicit fused multiply-adds (or explicitly separate operations), so
// that the instantiations of a body cannot differ in how the compiler contracts them: the forms agree bit for bit.
//
// Template switches:
//   THREADS  threads of the workgroup that calls the body.  The work is laid out for kDecThreads = 256; further
//            threads only take part in the barriers.
//   IO       how the operands that other kernels or workgroups produce / consume are accessed.  PlainIO: ordinary
//            loads and stores (the two-launch form: a kernel boundary orders everything).  TaggedIO: the inputs
//            were written, and the outputs will be read, by other workgroups of the SAME launch, with nothing
//            but the data to synchronise on: every 32-bit value travels as one 64-bit word (value, tag) written
//            and read with agent-coherent accesses (which bypass the caches private to a part of the chip); a
//            reader polls until all the words it needs carry the tag of the phase that produces them.  The KV
//            caches are exempt: rows of earlier positions come from earlier launches, and the row of the new
//            position is served from LDS.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lhip {

constexpr int kDecThreads = 256;
constexpr int kDecTile = 64;

__device__ __forceinline__ float wave_max64(float v) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    return v;
}
__device__ __forceinline__ float wave_sum64(float v) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    return v;
}

// Pointers that reach a kernel through a table in memory (rather than as kernel arguments) are generic to the
// compiler, which then emits flat accesses and waits for the LDS counter as well.  All of them are device memory.
#define LHIP_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ const LHIP_GLOBAL T *as_global(const T *p) {
    return (const LHIP_GLOBAL T *)p;
}
template <typename T>
__device__ __forceinline__ LHIP_GLOBAL T *as_global(T *p) {
    return (LHIP_GLOBAL T *)p;
}

typedef float lhip_f32x4 __attribute__((ext_vector_type(4)));
typedef float lhip_f32x2 __attribute__((ext_vector_type(2)));
// plain 16-byte accesses to device memory
__device__ __forceinline__ float4 ldg4(const float4 *p) {
    const lhip_f32x4 v = *as_global(reinterpret_cast<const lhip_f32x4 *>(p));
    return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stg4(float4 *p, const float4 &v) {
    lhip_f32x4 t;
    t.x = v.x; t.y = v.y; t.z = v.z; t.w = v.w;
    *as_global(reinterpret_cast<lhip_f32x4 *>(p)) = t;
}

// ---- agent-coherent accessors (relaxed atomics at agent scope: single instructions with the coherence bit set)
__device__ __forceinline__ float ld_agent(const float *p) {
    return __hip_atomic_load(as_global(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_agent(float *p, float v) {
    __hip_atomic_store(as_global(p), v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float2 ld_agent2(const float *p) {  // p 8-byte aligned
    const unsigned long long raw =
        __hip_atomic_load(as_global(reinterpret_cast<const unsigned long long *>(p)), __ATOMIC_RELAXED,
                          __HIP_MEMORY_SCOPE_AGENT);
    return make_float2(__uint_as_float(static_cast<unsigned>(raw)), __uint_as_float(static_cast<unsigned>(raw >> 32)));
}
__device__ __forceinline__ void st_agent2(float *p, float a, float b) {  // p 8-byte aligned
    const unsigned long long raw =
        static_cast<unsigned long long>(__float_as_uint(a)) | (static_cast<unsigned long long>(__float_as_uint(b)) << 32);
    __hip_atomic_store(as_global(reinterpret_cast<unsigned long long *>(p)), raw, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float4 ld_agent4(const float4 *p) {
    const float2 lo = ld_agent2(reinterpret_cast<const float *>(p)), hi = ld_agent2(reinterpret_cast<const float *>(p) + 2);
    return make_float4(lo.x, lo.y, hi.x, hi.y);
}
__device__ __forceinline__ void st_agent4(float4 *p, const float4 &v) {
    st_agent2(reinterpret_cast<float *>(p), v.x, v.y);
    st_agent2(reinterpret_cast<float *>(p) + 2, v.z, v.w);
}

// Operand access policies of the bodies below.  Addresses are given as (base, element index): a tagged array
// has the element order of the plain one, 8 bytes per element.
struct PlainIO {
    // Every slot of a workspace may be read whatever it holds (plain memory: nothing waits for a value to appear), so
    // a reader need not know which slots were written before it asks for them.
    static constexpr bool kAnySlot = true;
    __device__ __forceinline__ float ld1(const float *b, size_t i, bool &) const { return as_global(b)[i]; }
    __device__ __forceinline__ float2 ld2(const float *b, size_t i, bool &) const {  // i even
        const lhip_f32x2 v = *as_global(reinterpret_cast<const lhip_f32x2 *>(b + i));
        return make_float2(v.x, v.y);
    }
    __device__ __forceinline__ float4 ld4(const float4 *b, size_t i4, bool &) const { return ldg4(b + i4); }
    __device__ __forceinline__ void st1(float *b, size_t i, float v) const { as_global(b)[i] = v; }
    __device__ __forceinline__ void st4(float4 *b, size_t i4, const float4 &v) const { stg4(b + i4, v); }
    __device__ __forceinline__ bool again(bool) { return false; }
};

constexpr unsigned kTagSpinLimit = 1u << 20;

struct TaggedIO {
    static constexpr bool kAnySlot = false;  // a slot nobody writes this step never shows this step's tag
    unsigned in_tag, out_tag;
    unsigned *abort_flag, *sticky;  // raised when a wait is given up; seen by every other waiter
    unsigned spins = 0;
    __device__ __forceinline__ float ld1(const float *b, size_t i, bool &ok) const {
        const unsigned long long raw = __hip_atomic_load(as_global(reinterpret_cast<const unsigned long long *>(b)) + i,
                                                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        ok = ok && static_cast<unsigned>(raw >> 32) == in_tag;
        return __uint_as_float(static_cast<unsigned>(raw));
    }
    __device__ __forceinline__ float2 ld2(const float *b, size_t i, bool &ok) const {
        const float x = ld1(b, i, ok), y = ld1(b, i + 1, ok);
        return make_float2(x, y);
    }
    __device__ __forceinline__ float4 ld4(const float4 *b, size_t i4, bool &ok) const {
        const float *f = reinterpret_cast<const float *>(b);
        const float x = ld1(f, 4 * i4, ok), y = ld1(f, 4 * i4 + 1, ok), z = ld1(f, 4 * i4 + 2, ok), w = ld1(f, 4 * i4 + 3, ok);
        return make_float4(x, y, z, w);
    }
    __device__ __forceinline__ void st1(float *b, size_t i, float v) const {
        const unsigned long long raw =
            static_cast<unsigned long long>(__float_as_uint(v)) | (static_cast<unsigned long long>(out_tag) << 32);
        __hip_atomic_store(as_global(reinterpret_cast<unsigned long long *>(b)) + i, raw, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
    }
    __device__ __forceinline__ void st4(float4 *b, size_t i4, const float4 &v) const {
        float *f = reinterpret_cast<float *>(b);
        st1(f, 4 * i4, v.x);
        st1(f, 4 * i4 + 1, v.y);
        st1(f, 4 * i4 + 2, v.z);
        st1(f, 4 * i4 + 3, v.w);
    }
    // After a round of loads: true = some word was not there yet, load again.  Bounded: past the limit, or once
    // anybody has given up, the caller goes on with whatever it has.
    __device__ __forceinline__ bool again(bool ok) {
        if (ok) return false;
        ++spins;
        if (spins > kTagSpinLimit) {
            __hip_atomic_store(as_global(abort_flag), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(as_global(sticky), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return false;
        }
        if ((spins & 63u) == 0u &&
            __hip_atomic_load(as_global(abort_flag), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0u)
            return false;
        return true;
    }
};

// sin and cos of the rotary angle pos / theta^(two_j / hd).  Kept out of line: the library routines inside are
// open to re-association, and a copy inlined into each caller could round differently from caller to caller.
__device__ __noinline__ float2 rope_sin_cos(float theta, int two_j, int hd, int pos) {
    const float inv_freq = 1.0f / powf(theta, static_cast<float>(two_j) / static_cast<float>(hd));
    const float ang = static_cast<float>(pos) * inv_freq;
    float sn, cs;
    sincosf(ang, &sn, &cs);
    return make_float2(sn, cs);
}

// Workspace: [float ml[kv_heads][splits][G][2]] padded to a multiple of 256 B, [float acc[kv_heads][splits][G][HD]].
static inline size_t dec_ml_bytes(int64_t kv_heads, int splits, int64_t g) {
    return (static_cast<size_t>(kv_heads) * splits * g * 2 * sizeof(float) + 255) & ~size_t{255};
}
static inline int dec_splits(int64_t kv_heads) {
    int64_t s = 256 / kv_heads;
    return static_cast<int>(s < 1 ? 1 : (s > 64 ? 64 : s));
}
// Key ranges a step's attention is cut into, of the n_splits the workspace has room for.  Normally all of them: at
// batch 1 the kernel is a handful of dependent trips to memory, and the shorter the ranges the fewer trips (32 ranges
// of one tile each at 512-768 keys: 6.6 us; 8 ranges of two tiles: 9.5 us).  `few`: one range per 64-key tile up to
// eight (contexts up to 2048 keys), sixteen beyond - few enough partial states for a consumer to merge them itself
// (lhip_q8_0_matvec_attn_merge_f32).  Workgroups of ranges that hold no keys leave at once.
constexpr int kDecMaxActive = 16;
__host__ __device__ inline int dec_active_splits(int n_keys, int n_splits, bool few) {
    if (!few) return n_splits;
    int eff = n_keys <= 2048 ? (n_keys + 63) / 64 : kDecMaxActive;
    eff = eff > 8 && n_keys <= 2048 ? 8 : eff;
    eff = eff < 1 ? 1 : eff;
    return eff < n_splits ? eff : n_splits;
}
// Weight of a key range's partial state in the merge, exp(its maximum - the overall maximum).  Out of line: the merge
// kernel and the matvec prologue that merges on its own must round alike, and inlined copies of the library routine
// need not.
__device__ __noinline__ float dec_merge_weight(float m, float mx) { return expf(m - mx); }

// LDS of one workgroup in the attention body.
template <int G, int HD>
struct AttnShared {
    static constexpr int C4 = HD / 4;             // float4 columns of a row
    static constexpr int KG = kDecThreads / C4;   // key groups in P.V
    float4 q_s[G][C4];
    float4 knew[C4], vnew[C4];
    float p_s[G][kDecTile];
    float m_s[G], l_s[G], corr_s[G];
    float4 part[KG][G][C4];
};

// One (KV head, key range) piece: rotary on the G query rows and the new key, append of the new key / value to
// the caches when the range holds the new position, attention over the range, partial state to the workspace.
//
// Inside a workgroup (256 working threads), per tile of 64 keys:
//   scores: 4 lanes per key, each reading float4 columns sub, sub+4, ... of the row, so a
//           quad covers 64 contiguous bytes per load; q for the G heads comes from LDS;
//   online softmax: wave w owns heads w, w+4: lane = key;
//   P.V:    HD/4 lanes cover a V row as float4, 256/(HD/4) key groups split the tile.
// The K and V loads of a tile are all issued before the first use.
template <int G, int HD, int THREADS, typename IO>
__device__ __forceinline__ void attention_decode_body(IO io, AttnShared<G, HD> &sh, int kvh, int split,
                                                      const float *__restrict__ qkv, float *__restrict__ k_cache,
                                                      float *__restrict__ v_cache, int pos, int hkv, int max_seq,
                                                      float theta, int n_splits, float *__restrict__ ws_ml,
                                                      float4 *__restrict__ ws_acc, bool few_ranges = false) {
    constexpr int C4 = HD / 4;
    constexpr int KG = kDecThreads / C4;     // key groups in P.V
    constexpr int KPG = kDecTile / KG;       // keys per group and tile
    constexpr int J = HD / 16;               // float4 per lane and key in the scores
    static_assert(KG * KPG == kDecTile && J * 16 == HD, "tile shape");
    static_assert(THREADS >= kDecThreads && THREADS % 64 == 0, "workgroup size");

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const bool on = THREADS == kDecThreads || tid < kDecThreads;  // wave-uniform
    const int hq = hkv * G;
    const int n_keys = min(pos + 1, max_seq);
    const int eff_splits = dec_active_splits(n_keys, n_splits, few_ranges);
    const int chunk = (n_keys + eff_splits - 1) / eff_splits;
    const int k0 = split * chunk, k1 = min(n_keys, k0 + chunk);
    if (k0 >= k1) return;  // uniform over the workgroup: a range without keys has nothing to do, not even the append
    const float inv_sqrt = 1.0f / sqrtf(static_cast<float>(HD));
    const float4 *kc4 = reinterpret_cast<const float4 *>(k_cache) + static_cast<size_t>(kvh) * max_seq * C4;
    const float4 *vc4 = reinterpret_cast<const float4 *>(v_cache) + static_cast<size_t>(kvh) * max_seq * C4;

    // ---- cache rows of a tile of keys: all loads issued before the first use.  The first tile is requested at
    // once, ahead of the wait for q: the caches do not depend on it (the row of the new position, which may not
    // have been written yet, is replaced from LDS below).
    const int sub = tid & 3, kslot = (tid >> 2) & (kDecTile - 1);  // scores: 4 lanes per key
    const int c4 = tid % C4, kgp = (tid / C4) % KG;                // P.V: column and key group
    float4 kreg[J];
    float4 vreg[KPG];
    auto load_tile = [&](int t0) {
        const int key = t0 + kslot;
        const float4 *krow = kc4 + static_cast<size_t>(key < k1 ? key : k0) * C4;
#pragma unroll
        for (int j = 0; j < J; ++j) kreg[j] = ldg4(krow + j * 4 + sub);
#pragma unroll
        for (int u = 0; u < KPG; ++u) {
            const int vkey = t0 + kgp + KG * u;
            vreg[u] = ldg4(vc4 + static_cast<size_t>(vkey < k1 ? vkey : k0) * C4 + c4);
        }
    };
    if (on && k0 < k1) load_tile(k0);

    // ---- rotary on the G query rows and the new key (adjacent pairs, as the rope operator), copy of the new value
    if (on) {
        constexpr int NPAIR = (G + 1) * (HD / 2);
        constexpr int ITER = (NPAIR + kDecThreads - 1) / kDecThreads;
        float2 xr[ITER];
        float vn = 0.f;
        bool ok;
        do {  // the raw values first (in the tagged form: until all of them are there), the arithmetic once
            ok = true;
#pragma unroll
            for (int it = 0; it < ITER; ++it) {
                const int i = min(tid + it * kDecThreads, NPAIR - 1);
                const int r = i / (HD / 2), j = i - r * (HD / 2);
                xr[it] = io.ld2(qkv, static_cast<size_t>(r < G ? kvh * G + r : hq + kvh) * HD + 2 * j, ok);
            }
            if (tid < HD) vn = io.ld1(qkv, static_cast<size_t>(hq + hkv + kvh) * HD + tid, ok);
        } while (io.again(ok));
#pragma unroll
        for (int it = 0; it < ITER; ++it) {
            const int i = tid + it * kDecThreads;
            if (i < NPAIR) {
                const int r = i / (HD / 2), j = i - r * (HD / 2);
                const float2 sc = rope_sin_cos(theta, 2 * j, HD, pos);
                const float sn = sc.x, cs = sc.y;
                float *dst = r < G ? reinterpret_cast<float *>(sh.q_s[r]) : reinterpret_cast<float *>(sh.knew);
                // products rounded one by one, as the rope operator of the graph does
                dst[2 * j] = __fsub_rn(__fmul_rn(xr[it].x, cs), __fmul_rn(xr[it].y, sn));
                dst[2 * j + 1] = __fadd_rn(__fmul_rn(xr[it].x, sn), __fmul_rn(xr[it].y, cs));
            }
        }
        if (tid < HD) reinterpret_cast<float *>(sh.vnew)[tid] = vn;
        if (tid < G) {
            sh.m_s[tid] = -INFINITY;
            sh.l_s[tid] = 0.f;
        }
    }
    __syncthreads();
    if (on && pos < max_seq && pos >= k0 && pos < k1 && tid < C4) {  // this range holds the new position
        stg4(reinterpret_cast<float4 *>(k_cache) + (static_cast<size_t>(kvh) * max_seq + pos) * C4 + tid, sh.knew[tid]);
        stg4(reinterpret_cast<float4 *>(v_cache) + (static_cast<size_t>(kvh) * max_seq + pos) * C4 + tid, sh.vnew[tid]);
    }

    float4 acc[G];
#pragma unroll
    for (int g = 0; g < G; ++g) acc[g] = make_float4(0, 0, 0, 0);
    for (int t0 = k0; t0 < k1; t0 += kDecTile) {
        // ---- the tile's cache rows; the new position is served from LDS (its cache row may not have landed)
        const int key = t0 + kslot;
        const bool live = key < k1;
        if (on) {
            if (t0 != k0) load_tile(t0);
            if (key == pos) {
#pragma unroll
                for (int j = 0; j < J; ++j) kreg[j] = sh.knew[j * 4 + sub];
            }
#pragma unroll
            for (int u = 0; u < KPG; ++u)
                if (t0 + kgp + KG * u == pos) vreg[u] = sh.vnew[c4];
            // ---- scores
            float s[G];
#pragma unroll
            for (int g = 0; g < G; ++g) {
                float d = 0.f;
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    const float4 qv = sh.q_s[g][j * 4 + sub];
                    d = fmaf(qv.x, kreg[j].x, d);
                    d = fmaf(qv.y, kreg[j].y, d);
                    d = fmaf(qv.z, kreg[j].z, d);
                    d = fmaf(qv.w, kreg[j].w, d);
                }
                d += __shfl_xor(d, 1);
                d += __shfl_xor(d, 2);
                s[g] = d * inv_sqrt;
            }
            if (sub == 0) {
#pragma unroll
                for (int g = 0; g < G; ++g) sh.p_s[g][kslot] = live ? s[g] : -INFINITY;
            }
        }
        __syncthreads();
        // ---- online softmax: running max and sum per head, weights back into p_s
        if (on) {
            for (int g = wave; g < G; g += kDecThreads / 64) {
                const float sv = sh.p_s[g][lane];
                const float m_old = sh.m_s[g];
                const float m_new = fmaxf(m_old, wave_max64(sv));  // finite: every tile has a live key
                const float p = expf(sv - m_new);
                const float psum = wave_sum64(p);
                const float c = expf(m_old - m_new);
                sh.p_s[g][lane] = p;
                if (lane == 0) {
                    sh.m_s[g] = m_new;
                    sh.l_s[g] = fmaf(sh.l_s[g], c, psum);
                    sh.corr_s[g] = c;
                }
            }
        }
        __syncthreads();
        // ---- P.V
        if (on) {
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const float c = sh.corr_s[g];
                float4 a = make_float4(acc[g].x * c, acc[g].y * c, acc[g].z * c, acc[g].w * c);
#pragma unroll
                for (int u = 0; u < KPG; ++u) {
                    const float w = sh.p_s[g][kgp + KG * u];  // 0 for keys past the range
                    a.x = fmaf(w, vreg[u].x, a.x); a.y = fmaf(w, vreg[u].y, a.y);
                    a.z = fmaf(w, vreg[u].z, a.z); a.w = fmaf(w, vreg[u].w, a.w);
                }
                acc[g] = a;
            }
        }
        __syncthreads();  // p_s is rewritten by the next tile
    }

    // ---- partial state of this range -> workspace
    if (k0 < k1) {  // uniform over the workgroup
        if (on) {
#pragma unroll
            for (int g = 0; g < G; ++g) sh.part[kgp][g][c4] = acc[g];
        }
        __syncthreads();
        const size_t slot = static_cast<size_t>(kvh) * n_splits + split;
        if (tid < G * C4) {
            const int g = tid / C4, c = tid - g * C4;
            float4 t = sh.part[0][g][c];
#pragma unroll
            for (int q = 1; q < KG; ++q) {
                const float4 u = sh.part[q][g][c];
                t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
            }
            io.st4(ws_acc, (slot * G + g) * C4 + c, t);
        }
        if (tid < G) {
            io.st1(ws_ml, (slot * G + tid) * 2, sh.m_s[tid]);
            io.st1(ws_ml, (slot * G + tid) * 2 + 1, sh.l_s[tid]);
        }
    }
}

// LDS of one workgroup in the merge body.
struct MergeShared {
    float2 ml_s[64];  // (max, sum) of every key range, for the one head
    float4 num_s[kDecThreads];
    float den_s[kDecThreads];
};

// Merge of the partial states of one query head (head = kvh * G + g).  The 256 working threads are HD/4 output
// columns x SG sub-groups; a thread takes the key ranges sg, sg + SG, ..., four per round of loads, the first round
// together with the (max, sum) pairs, so that the usual 32 ranges cost a single memory round trip; the
// sub-groups meet in LDS.
template <int G, int HD, int THREADS, typename IO>
__device__ __forceinline__ void attention_merge_body(IO io, MergeShared &sh, int head, float *__restrict__ out, int pos,
                                                     int max_seq, int n_splits, const float *__restrict__ ws_ml,
                                                     const float4 *__restrict__ ws_acc,
                                                     float *__restrict__ out_copy = nullptr, bool few_ranges = false) {
    constexpr int C4 = HD / 4;
    constexpr int SG = kDecThreads / C4;  // sub-groups: 8 (HD 128) or 16 (HD 64)
    const int tid = threadIdx.x;
    const bool on = THREADS == kDecThreads || tid < kDecThreads;
    const int kvh = head / G, g = head - kvh * G;
    const size_t base = static_cast<size_t>(kvh) * n_splits;
    const int c = tid % C4, sg = (tid / C4) % SG;
    float4 a[4];
    float2 mine = make_float2(0.f, 0.f);
    // With plain memory every range of the launch may be asked for, so the addresses of the first round do not depend
    // on the position: its loads go out here, while the position is still on its way, instead of a trip to memory
    // behind it; what a range without keys left in its slot is discarded below.
    if constexpr (IO::kAnySlot) {
        if (on) {
            bool ok = true;
            if (tid < n_splits) mine = io.ld2(ws_ml, ((base + tid) * G + g) * 2, ok);
#pragma unroll
            for (int u = 0; u < 4; ++u)
                a[u] = io.ld4(ws_acc, ((base + min(sg + u * SG, n_splits - 1)) * G + g) * C4 + c, ok);
        }
    }
    const int n_keys = min(pos + 1, max_seq);
    const int eff_splits = dec_active_splits(n_keys, n_splits, few_ranges);
    const int chunk = (n_keys + eff_splits - 1) / eff_splits;
    const int n_active = (n_keys + chunk - 1) / chunk;  // ranges that held keys (<= 64)
    auto acc_index = [&](int sidx) { return ((base + min(sidx, n_active - 1)) * G + g) * C4 + c; };

    if (on) {
        if constexpr (!IO::kAnySlot) {
            bool ok;
            do {
                ok = true;
                if (tid < n_active) mine = io.ld2(ws_ml, ((base + tid) * G + g) * 2, ok);
#pragma unroll
                for (int u = 0; u < 4; ++u) a[u] = io.ld4(ws_acc, acc_index(sg + u * SG), ok);
            } while (io.again(ok));
        }
        if (tid < n_active) sh.ml_s[tid] = mine;
    }
    __syncthreads();
    float den = 0.f;
    float4 num = make_float4(0, 0, 0, 0);
    if (on) {
        float mx = -INFINITY;
        for (int sidx = 0; sidx < n_active; ++sidx) mx = fmaxf(mx, sh.ml_s[sidx].x);
        for (int s0 = sg; s0 < n_active; s0 += 4 * SG) {
            if (s0 != sg) {  // further rounds (more than 4 * SG ranges)
                bool ok;
                do {
                    ok = true;
#pragma unroll
                    for (int u = 0; u < 4; ++u) a[u] = io.ld4(ws_acc, acc_index(s0 + u * SG), ok);
                } while (io.again(ok));
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int sidx = s0 + u * SG;
                const bool live = sidx < n_active;
                const float2 v = sh.ml_s[live ? sidx : 0];
                const float wgt = live ? dec_merge_weight(v.x, mx) : 0.f;
                const float4 av = live ? a[u] : make_float4(0.f, 0.f, 0.f, 0.f);  // (a slot never written may hold anything)
                den = fmaf(v.y, wgt, den);
                num.x = fmaf(av.x, wgt, num.x); num.y = fmaf(av.y, wgt, num.y);
                num.z = fmaf(av.z, wgt, num.z); num.w = fmaf(av.w, wgt, num.w);
            }
        }
        sh.num_s[sg * C4 + c] = num;
        sh.den_s[sg * C4 + c] = den;
    }
    __syncthreads();
    if (on && sg == 0) {
        for (int q = 1; q < SG; ++q) {
            const float4 u = sh.num_s[q * C4 + c];
            num.x += u.x; num.y += u.y; num.z += u.z; num.w += u.w;
            den += sh.den_s[q * C4 + c];
        }
        const float inv = 1.0f / den;
        const float4 o = make_float4(num.x * inv, num.y * inv, num.z * inv, num.w * inv);
        io.st4(reinterpret_cast<float4 *>(out), static_cast<size_t>(head) * C4 + c, o);
        // the tagged form writes a shadow array: the caller's own buffer gets the plain values as well
        if (out_copy != nullptr) stg4(reinterpret_cast<float4 *>(out_copy) + static_cast<size_t>(head) * C4 + c, o);
    }
}

}  // namespace lhip
