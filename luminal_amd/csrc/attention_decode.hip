// Batch-1 decode attention with rotary embedding and KV append folded in.
//
// What the reference's graph does for one new token (examples/llama/src/model.rs:52-72
// rotary, :108-110 cache concat, :112-139 grouped-query attention) as ONE launch:
//   q, k of the new token are rotated; k and v are appended to the caches at *pos;
//   out[h] = softmax(q_h . K / sqrt(hd)) V over positions 0..*pos.
//
// Shape of the launch.  At batch 1 the work is a read of the two caches, which one
// workgroup per head cannot pull fast enough (it exposes several dependent memory round
// trips on a handful of CUs).  So the keys of each KV head are cut into `splits` ranges,
// one workgroup each (grid = kv_heads x splits, about one workgroup per CU), and the G
// query heads that share a KV head are served by the same workgroup, which therefore
// reads every cache row once.  Each workgroup writes its partial softmax state (max, sum,
// weighted V) to a workspace and a second, small kernel merges the partials into the output
// rows.  (Merging in the same launch needs device-scope release/acquire fences in every
// workgroup; on this part each is a write-back plus invalidate of a whole L2 and the 256 of
// them cost more than the second launch.)
//
// Inside a workgroup (256 threads), per tile of 64 keys:
//   scores: 4 lanes per key, each reading float4 columns sub, sub+4, ... of the row, so a
//           quad covers 64 contiguous bytes per load; q for the G heads comes from LDS;
//   online softmax: wave w owns heads w, w+4: lane = key;
//   P.V:    HD/4 lanes cover a V row as float4, 256/(HD/4) key groups split the tile.
// The K and V loads of a tile are all issued before the first use.
#include "common.h"

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

// Workspace: [float ml[kv_heads][splits][G][2]] padded to a multiple of 256 B, [float acc[kv_heads][splits][G][HD]].
static inline size_t dec_ml_bytes(int64_t kv_heads, int splits, int64_t g) {
    return (static_cast<size_t>(kv_heads) * splits * g * 2 * sizeof(float) + 255) & ~size_t{255};
}
static inline int dec_splits(int64_t kv_heads) {
    int64_t s = 256 / kv_heads;
    return static_cast<int>(s < 1 ? 1 : (s > 64 ? 64 : s));
}

template <int G, int HD>
__global__ __launch_bounds__(kDecThreads) void attention_decode_kernel(
    const float *__restrict__ qkv, float *__restrict__ k_cache, float *__restrict__ v_cache,
    const int *__restrict__ pos_dev, int hkv, int max_seq, float theta, int n_splits,
    float *__restrict__ ws_ml, float4 *__restrict__ ws_acc) {
    constexpr int C4 = HD / 4;               // float4 columns of a row
    constexpr int KG = kDecThreads / C4;     // key groups in P.V
    constexpr int KPG = kDecTile / KG;       // keys per group and tile
    constexpr int J = HD / 16;               // float4 per lane and key in the scores
    static_assert(KG * KPG == kDecTile && J * 16 == HD, "tile shape");
    __shared__ float4 q_s[G][C4];
    __shared__ float4 knew[C4], vnew[C4];
    __shared__ float p_s[G][kDecTile];
    __shared__ float m_s[G], l_s[G], corr_s[G];
    __shared__ float4 part[KG][G][C4];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int kvh = blockIdx.x, split = blockIdx.y;
    const int hq = hkv * G;
    const int pos = *pos_dev;
    const int n_keys = min(pos + 1, max_seq);
    const int chunk = (n_keys + n_splits - 1) / n_splits;
    const int k0 = split * chunk, k1 = min(n_keys, k0 + chunk);
    const float inv_sqrt = 1.0f / sqrtf(static_cast<float>(HD));
    const float4 *kc4 = reinterpret_cast<const float4 *>(k_cache) + static_cast<size_t>(kvh) * max_seq * C4;
    const float4 *vc4 = reinterpret_cast<const float4 *>(v_cache) + static_cast<size_t>(kvh) * max_seq * C4;

    // ---- rotary on the G query rows and the new key (adjacent pairs, as the rope operator), copy of the new value
    for (int i = tid; i < (G + 1) * (HD / 2); i += kDecThreads) {
        const int r = i / (HD / 2), j = i - r * (HD / 2);
        const float *row = qkv + static_cast<size_t>(r < G ? kvh * G + r : hq + kvh) * HD;
        const float inv_freq = 1.0f / powf(theta, static_cast<float>(2 * j) / static_cast<float>(HD));
        const float ang = static_cast<float>(pos) * inv_freq;
        float sn, cs;
        sincosf(ang, &sn, &cs);
        const float x0 = row[2 * j], x1 = row[2 * j + 1];
        float *dst = r < G ? reinterpret_cast<float *>(q_s[r]) : reinterpret_cast<float *>(knew);
        dst[2 * j] = x0 * cs - x1 * sn;
        dst[2 * j + 1] = x0 * sn + x1 * cs;
    }
    for (int i = tid; i < HD; i += kDecThreads)
        reinterpret_cast<float *>(vnew)[i] = qkv[static_cast<size_t>(hq + hkv + kvh) * HD + i];
    if (tid < G) {
        m_s[tid] = -INFINITY;
        l_s[tid] = 0.f;
    }
    __syncthreads();
    if (pos < max_seq && pos >= k0 && pos < k1 && tid < C4) {  // this workgroup's range holds the new position
        reinterpret_cast<float4 *>(k_cache)[(static_cast<size_t>(kvh) * max_seq + pos) * C4 + tid] = knew[tid];
        reinterpret_cast<float4 *>(v_cache)[(static_cast<size_t>(kvh) * max_seq + pos) * C4 + tid] = vnew[tid];
    }

    float4 acc[G];
#pragma unroll
    for (int g = 0; g < G; ++g) acc[g] = make_float4(0, 0, 0, 0);
    const int sub = tid & 3, kslot = tid >> 2;  // scores: 4 lanes per key
    const int c4 = tid % C4, kgp = tid / C4;    // P.V: column and key group

    for (int t0 = k0; t0 < k1; t0 += kDecTile) {
        // ---- all loads of the tile; the new position is served from LDS (its cache row may not have landed)
        const int key = t0 + kslot;
        const bool live = key < k1;
        const float4 *krow = kc4 + static_cast<size_t>(live ? key : k0) * C4;
        float4 kreg[J];
#pragma unroll
        for (int j = 0; j < J; ++j) kreg[j] = (key == pos) ? knew[j * 4 + sub] : krow[j * 4 + sub];
        float4 vreg[KPG];
#pragma unroll
        for (int u = 0; u < KPG; ++u) {
            const int vkey = t0 + kgp + KG * u;
            vreg[u] = (vkey == pos) ? vnew[c4] : vc4[static_cast<size_t>(vkey < k1 ? vkey : k0) * C4 + c4];
        }
        // ---- scores
        float s[G];
#pragma unroll
        for (int g = 0; g < G; ++g) {
            float d = 0.f;
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const float4 qv = q_s[g][j * 4 + sub];
                d += qv.x * kreg[j].x + qv.y * kreg[j].y + qv.z * kreg[j].z + qv.w * kreg[j].w;
            }
            d += __shfl_xor(d, 1);
            d += __shfl_xor(d, 2);
            s[g] = d * inv_sqrt;
        }
        if (sub == 0) {
#pragma unroll
            for (int g = 0; g < G; ++g) p_s[g][kslot] = live ? s[g] : -INFINITY;
        }
        __syncthreads();
        // ---- online softmax: running max and sum per head, weights back into p_s
        for (int g = wave; g < G; g += kDecThreads / 64) {
            const float sv = p_s[g][lane];
            const float m_old = m_s[g];
            const float m_new = fmaxf(m_old, wave_max64(sv));  // finite: every tile has a live key
            const float p = expf(sv - m_new);
            const float psum = wave_sum64(p);
            const float c = expf(m_old - m_new);
            p_s[g][lane] = p;
            if (lane == 0) {
                m_s[g] = m_new;
                l_s[g] = l_s[g] * c + psum;
                corr_s[g] = c;
            }
        }
        __syncthreads();
        // ---- P.V
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float c = corr_s[g];
            float4 a = make_float4(acc[g].x * c, acc[g].y * c, acc[g].z * c, acc[g].w * c);
#pragma unroll
            for (int u = 0; u < KPG; ++u) {
                const float w = p_s[g][kgp + KG * u];  // 0 for keys past the range
                a.x += w * vreg[u].x; a.y += w * vreg[u].y; a.z += w * vreg[u].z; a.w += w * vreg[u].w;
            }
            acc[g] = a;
        }
        __syncthreads();  // p_s is rewritten by the next tile
    }

    // ---- partial state of this range -> workspace
    if (k0 < k1) {
#pragma unroll
        for (int g = 0; g < G; ++g) part[kgp][g][c4] = acc[g];
        __syncthreads();
        const size_t slot = static_cast<size_t>(kvh) * n_splits + split;
        if (tid < G * C4) {
            const int g = tid / C4, c = tid - g * C4;
            float4 t = part[0][g][c];
#pragma unroll
            for (int q = 1; q < KG; ++q) {
                const float4 u = part[q][g][c];
                t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
            }
            ws_acc[(slot * G + g) * C4 + c] = t;
        }
        if (tid < G) {
            ws_ml[(slot * G + tid) * 2] = m_s[tid];
            ws_ml[(slot * G + tid) * 2 + 1] = l_s[tid];
        }
    }
}

// Merge of the partial states: one workgroup per KV head.  The (max, sum) pairs go to LDS in one round trip,
// then the 256 threads split the ranges between them (SG threads per output float4, four loads in flight each)
// and meet in LDS.
template <int G, int HD>
__global__ __launch_bounds__(kDecThreads) void attention_merge_kernel(float *__restrict__ out,
                                                                      const int *__restrict__ pos_dev, int max_seq,
                                                                      int n_splits, const float *__restrict__ ws_ml,
                                                                      const float4 *__restrict__ ws_acc) {
    constexpr int C4 = HD / 4;
    constexpr int P = G * C4;              // output float4s of this KV head
    constexpr int SG = kDecThreads / P;    // threads per output
    static_assert(P * SG == kDecThreads, "merge shape");
    __shared__ float2 ml_s[64 * G];
    __shared__ float4 num_s[kDecThreads];
    __shared__ float den_s[kDecThreads];
    const int tid = threadIdx.x, kvh = blockIdx.x;
    const int n_keys = min(*pos_dev + 1, max_seq);
    const int chunk = (n_keys + n_splits - 1) / n_splits;
    const int n_active = (n_keys + chunk - 1) / chunk;  // ranges that held keys
    const size_t base = static_cast<size_t>(kvh) * n_splits;
    for (int i = tid; i < n_active * G; i += kDecThreads) ml_s[i] = reinterpret_cast<const float2 *>(ws_ml)[base * G + i];
    __syncthreads();
    const int pair = tid % P, sg = tid / P;
    const int g = pair / C4, c = pair - g * C4;
    float mx = -INFINITY;
    for (int sidx = 0; sidx < n_active; ++sidx) mx = fmaxf(mx, ml_s[sidx * G + g].x);
    float den = 0.f;
    float4 num = make_float4(0, 0, 0, 0);
    for (int s0 = sg; s0 < n_active; s0 += 4 * SG) {
        float4 a[4];
        float w[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int sidx = s0 + u * SG;
            const bool on = sidx < n_active;
            a[u] = ws_acc[((base + (on ? sidx : 0)) * G + g) * C4 + c];
            const float2 v = ml_s[(on ? sidx : 0) * G + g];
            w[u] = on ? expf(v.x - mx) : 0.f;
            den += v.y * w[u];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            num.x += a[u].x * w[u]; num.y += a[u].y * w[u]; num.z += a[u].z * w[u]; num.w += a[u].w * w[u];
        }
    }
    num_s[sg * P + pair] = num;
    den_s[sg * P + pair] = den;
    __syncthreads();
    if (sg == 0) {
        for (int q = 1; q < SG; ++q) {
            const float4 u = num_s[q * P + pair];
            num.x += u.x; num.y += u.y; num.z += u.z; num.w += u.w;
            den += den_s[q * P + pair];
        }
        const float inv = 1.0f / den;
        reinterpret_cast<float4 *>(out)[static_cast<size_t>(kvh * G + g) * C4 + c] =
            make_float4(num.x * inv, num.y * inv, num.z * inv, num.w * inv);
    }
}

template <int G, int HD>
static lhip_status launch_decode(const float *qkv, float *kc, float *vc, float *out, const int *pos, int hkv, int max_seq,
                                 float theta, void *workspace, hipStream_t s) {
    const int splits = dec_splits(hkv);
    auto *base = static_cast<uint8_t *>(workspace);
    float *ml = reinterpret_cast<float *>(base);
    float4 *acc = reinterpret_cast<float4 *>(base + dec_ml_bytes(hkv, splits, G));
    hipLaunchKernelGGL((attention_decode_kernel<G, HD>), dim3(static_cast<unsigned>(hkv), static_cast<unsigned>(splits)),
                       dim3(kDecThreads), 0, s, qkv, kc, vc, pos, hkv, max_seq, theta, splits, ml, acc);
    LHIP_CHECK_LAUNCH();
    hipLaunchKernelGGL((attention_merge_kernel<G, HD>), dim3(static_cast<unsigned>(hkv)), dim3(kDecThreads), 0, s, out,
                       pos, max_seq, splits, ml, acc);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

static bool dec_supported(int64_t q_heads, int64_t kv_heads, int64_t head_dim) {
    if (kv_heads <= 0 || q_heads <= 0 || q_heads % kv_heads != 0) return false;
    const int64_t g = q_heads / kv_heads;
    return (g == 1 || g == 2 || g == 4 || g == 8) && (head_dim == 64 || head_dim == 128);
}

}  // namespace lhip

using namespace lhip;

extern "C" {

size_t lhip_attention_decode_workspace_nbytes(int64_t q_heads, int64_t kv_heads, int64_t head_dim) {
    if (!dec_supported(q_heads, kv_heads, head_dim) || kv_heads > 65535) return 0;
    const size_t g = static_cast<size_t>(q_heads / kv_heads);
    const int splits = dec_splits(kv_heads);
    const size_t slots = static_cast<size_t>(kv_heads) * splits * g;
    return dec_ml_bytes(kv_heads, splits, static_cast<int64_t>(g)) +
           slots * static_cast<size_t>(head_dim) * sizeof(float);
}

lhip_status lhip_attention_decode_f32(const float *qkv_dev, float *k_cache_dev, float *v_cache_dev, float *out_dev,
                                      const int32_t *pos_dev, int64_t q_heads, int64_t kv_heads, int64_t head_dim,
                                      int64_t max_seq, float theta, void *workspace_dev, void *stream) {
    if (!qkv_dev || !k_cache_dev || !v_cache_dev || !out_dev || !pos_dev || !workspace_dev) return LHIP_ERR_NULL_PTR;
    if (q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || max_seq <= 0 || q_heads % kv_heads != 0 ||
        max_seq > kMaxDim || kv_heads > 65535)
        return LHIP_ERR_INVALID_SHAPE;
    if (!dec_supported(q_heads, kv_heads, head_dim)) return LHIP_ERR_UNSUPPORTED;
    if (!aligned(qkv_dev, 16) || !aligned(k_cache_dev, 16) || !aligned(v_cache_dev, 16) || !aligned(out_dev, 16) ||
        !aligned(workspace_dev, 256))
        return LHIP_ERR_MISALIGNED;
    const int g = static_cast<int>(q_heads / kv_heads);
    const int hkv = static_cast<int>(kv_heads), ms = static_cast<int>(max_seq);
    hipStream_t s = as_stream(stream);
#define LHIP_CASE(G, HD) \
    if (g == G && head_dim == HD) \
        return launch_decode<G, HD>(qkv_dev, k_cache_dev, v_cache_dev, out_dev, pos_dev, hkv, ms, theta, workspace_dev, s);
    LHIP_CASE(1, 64) LHIP_CASE(2, 64) LHIP_CASE(4, 64) LHIP_CASE(8, 64)
    LHIP_CASE(1, 128) LHIP_CASE(2, 128) LHIP_CASE(4, 128) LHIP_CASE(8, 128)
#undef LHIP_CASE
    return LHIP_ERR_UNSUPPORTED;
}

}  // extern "C"
