// Causal grouped-query attention for a block of prompt tokens on the bf16 matrix cores.
//
// Same operator and work split as attention_prefill.hip (one workgroup per (KV head, 32 query tokens), one wave
// per query head of the group, 32-key tiles staged once in LDS for all of them), for callers whose attention
// output feeds a bf16 GEMM anyway: Q (pre-scaled), K, V and the soft-max weights are rounded to bf16 for
// v_mfma_f32_32x32x16_bf16, sums and the soft-max itself stay f32.  Sixteen MFMAs per wave and tile instead of 128.
//
// Per wave and key tile, lane = (c, h), c = lane % 32, h = lane / 32:
//   S^T = K Q^T   : A = K tile (row = key c, 8 consecutive head-dim elements per step and lane half, 16-byte LDS
//                   reads of the bf16 K rows), B = Q^T from registers.  Result layout as in the f32 kernel: lane
//                   (c, h) holds query c, keys 8*(v/4) + 4*h + v%4, v = 0..15.
//   O^T += V^T P^T: B = P^T is those registers, converted: MFMA step s (16 keys) takes registers 8s .. 8s+7, i.e.
//                   lane half h supplies keys 16s + 8a + 4h + b (a = 0..1, b = 0..3) in slots 4a + b.  A = V^T
//                   must present the same keys in the same slots, so V is stored transposed in LDS with bits 2
//                   and 3 of the key index swapped: a lane's eight keys are then one 16-byte read.
#include "common.h"

namespace lhip {

typedef float pv16f __attribute__((ext_vector_type(16)));
typedef __bf16 pbf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 pbf16x4 __attribute__((ext_vector_type(4)));

constexpr int kBfTileK = 32;  // keys per tile
constexpr int kBfTileQ = 32;  // queries per workgroup
constexpr int kBfVPitch = 144;  // bytes per row of V^T in LDS (64 used): free of bank conflicts for these reads

template <int G, int HD>
__global__ __launch_bounds__(64 * G) void attention_prefill_bf16_kernel(const float *__restrict__ qkv,
                                                                        const float *__restrict__ k_cache,
                                                                        const float *__restrict__ v_cache,
                                                                        __bf16 *__restrict__ out,
                                                                        const int *__restrict__ pos_dev, int tokens,
                                                                        int hkv, int max_seq) {
    constexpr int THREADS = 64 * G;
    constexpr int KPITCH = (HD * 2) % 256 == 0 ? HD * 2 + 144 : HD * 2 + 16;  // bytes; 144 mod 256 either way
    constexpr int STEPS = HD / 16;                 // MFMA steps of S^T
    constexpr int OB = HD / 32;                    // 32-row blocks of O^T
    constexpr int K_F4 = kBfTileK * HD / 4;        // float4 of a K tile
    constexpr int KLD = K_F4 / THREADS;            // float4 of K per thread and tile
    constexpr int V_UNITS = (kBfTileK / 4) * (HD / 4);  // (4 keys) x (4 head-dim) blocks of a V tile
    constexpr int VU = V_UNITS >= THREADS ? V_UNITS / THREADS : 1;
    static_assert(K_F4 % THREADS == 0 && KLD >= 1 && KLD <= 8 && (V_UNITS % THREADS == 0 || V_UNITS < THREADS), "staging split");
    constexpr int K_BYTES = kBfTileK * KPITCH, V_BYTES = HD * kBfVPitch;
    __shared__ __attribute__((aligned(16))) unsigned char k_s[2][K_BYTES];
    __shared__ __attribute__((aligned(16))) unsigned char v_s[2][V_BYTES];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 31, h = lane >> 5;
    const int kvh = blockIdx.x, qb = blockIdx.y;
    const int hq = hkv * G;
    const int pos0 = *pos_dev;
    const int q0 = qb * kBfTileQ;
    const int head = kvh * G + wave;
    const int my_q = q0 + c;
    const int my_pos = pos0 + my_q;
    const int n_keys = min(pos0 + min(tokens, q0 + kBfTileQ), max_seq);
    const int n_tiles = (n_keys + kBfTileK - 1) / kBfTileK;
    const float inv_sqrt = 1.0f / sqrtf(static_cast<float>(HD));

    // ---- Q^T operand of every step: Q[my_q][16 step + 8 h .. + 8) / sqrt(HD), bf16
    pbf16x8 qv[STEPS];
    {
        const float *qrow = qkv + (static_cast<size_t>(min(my_q, tokens - 1)) * (hq + 2 * hkv) + head) * HD + 8 * h;
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const float4 a = *reinterpret_cast<const float4 *>(qrow + 16 * s), b = *reinterpret_cast<const float4 *>(qrow + 16 * s + 4);
            qv[s] = pbf16x8{static_cast<__bf16>(a.x * inv_sqrt), static_cast<__bf16>(a.y * inv_sqrt),
                            static_cast<__bf16>(a.z * inv_sqrt), static_cast<__bf16>(a.w * inv_sqrt),
                            static_cast<__bf16>(b.x * inv_sqrt), static_cast<__bf16>(b.y * inv_sqrt),
                            static_cast<__bf16>(b.z * inv_sqrt), static_cast<__bf16>(b.w * inv_sqrt)};
        }
    }

    // ---- tile staging: global f32 -> registers -> bf16 in LDS (K row-major, V transposed)
    const float4 *kc4 = reinterpret_cast<const float4 *>(k_cache) + static_cast<size_t>(kvh) * max_seq * (HD / 4);
    const float4 *vc4 = reinterpret_cast<const float4 *>(v_cache) + static_cast<size_t>(kvh) * max_seq * (HD / 4);
    const bool v_thread = tid * VU < V_UNITS;  // THREADS > V_UNITS: the first V_UNITS threads transpose V
    float4 kst[KLD], vst[VU][4];
    auto load_tile = [&](int t) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < KLD; ++i) {
            const int f = tid + i * THREADS;
            const int row = f / (HD / 4), col = f - row * (HD / 4);
            const int key = min(t * kBfTileK + row, n_keys - 1);  // rows past the end repeat the last key (masked)
            kst[i] = kc4[static_cast<size_t>(key) * (HD / 4) + col];
        }
        if (v_thread) {
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                const int unit = tid * VU + u;
                const int kg = unit / (HD / 4), dq = unit - kg * (HD / 4);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int key = min(t * kBfTileK + 4 * kg + i, n_keys - 1);
                    vst[u][i] = vc4[static_cast<size_t>(key) * (HD / 4) + dq];
                }
            }
        }
    };
    auto store_tile = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < KLD; ++i) {
            const int f = tid + i * THREADS;
            const int row = f / (HD / 4), col = f - row * (HD / 4);
            const pbf16x4 w = {static_cast<__bf16>(kst[i].x), static_cast<__bf16>(kst[i].y), static_cast<__bf16>(kst[i].z),
                               static_cast<__bf16>(kst[i].w)};
            *reinterpret_cast<pbf16x4 *>(&k_s[buf][row * KPITCH + col * 8]) = w;
        }
        if (v_thread) {
#pragma unroll
            for (int u = 0; u < VU; ++u) {
                const int unit = tid * VU + u;
                const int kg = unit / (HD / 4), dq = unit - kg * (HD / 4);
                const int key = 4 * kg;  // first of four consecutive keys; V^T column = key with bits 2 and 3 swapped
                const int pos = (key & 16) | ((key & 4) << 1) | ((key & 8) >> 1);
                const float *v0 = &vst[u][0].x, *v1 = &vst[u][1].x, *v2 = &vst[u][2].x, *v3 = &vst[u][3].x;
#pragma unroll
                for (int dd = 0; dd < 4; ++dd) {
                    const pbf16x4 w = {static_cast<__bf16>(v0[dd]), static_cast<__bf16>(v1[dd]), static_cast<__bf16>(v2[dd]),
                                       static_cast<__bf16>(v3[dd])};
                    *reinterpret_cast<pbf16x4 *>(&v_s[buf][(4 * dq + dd) * kBfVPitch + pos * 2]) = w;
                }
            }
        }
    };

    pv16f o_acc[OB];
#pragma unroll
    for (int j = 0; j < OB; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) o_acc[j][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    load_tile(0);
    store_tile(0);
    if (n_tiles > 1) load_tile(1);
    __syncthreads();
    for (int t = 0; t < n_tiles; ++t) {
        const int buf = t & 1;
        // tile t+1 (requested during tile t-1) goes into the other buffer, which every wave left at the last barrier
        if (t + 1 < n_tiles) store_tile(buf ^ 1);
        if (t + 2 < n_tiles) load_tile(t + 2);
        // ---- S^T = K Q^T
        pv16f s_acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) s_acc[v] = 0.f;
        const unsigned char *krow = &k_s[buf][c * KPITCH + h * 16];
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
            s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(*reinterpret_cast<const pbf16x8 *>(krow + s * 32), qv[s], s_acc, 0, 0, 0);
        // ---- causal mask, running max / sum, weights in place
        float tmax = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = t * kBfTileK + 8 * (v >> 2) + 4 * h + (v & 3);
            if (key > my_pos || key >= n_keys) s_acc[v] = -INFINITY;
            tmax = fmaxf(tmax, s_acc[v]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float m_new = fmaxf(m_run, tmax);  // finite from the first tile on: key 0 is visible to every query
        const float corr = expf(m_run - m_new);
        // weights rounded to bf16 once, and the running sum takes the rounded values: the result stays a convex
        // combination of the (rounded) V rows
        pbf16x8 pb[2];
        float psum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const __bf16 w = static_cast<__bf16>(expf(s_acc[v] - m_new));
            pb[v >> 3][v & 7] = w;
            psum += static_cast<float>(w);
        }
        psum += __shfl_xor(psum, 32);
        l_run = l_run * corr + psum;
        m_run = m_new;
#pragma unroll
        for (int j = 0; j < OB; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) o_acc[j][v] *= corr;
        // ---- O^T += V^T P^T
        const unsigned char *vrow = &v_s[buf][c * kBfVPitch + h * 16];
#pragma unroll
        for (int j = 0; j < OB; ++j)
#pragma unroll
            for (int s = 0; s < 2; ++s)
                o_acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                    *reinterpret_cast<const pbf16x8 *>(vrow + j * 32 * kBfVPitch + s * 32), pb[s], o_acc[j], 0, 0, 0);
        __syncthreads();
    }

    // ---- out[q][head*HD + 32 j + 8 a + 4 h + b] = O^T[..][q] / l: four consecutive head-dim elements per store
    if (my_q < tokens) {
        const float inv = 1.0f / l_run;
        __bf16 *orow = out + (static_cast<size_t>(my_q) * hq + head) * HD;
#pragma unroll
        for (int j = 0; j < OB; ++j)
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                const pbf16x4 w = {static_cast<__bf16>(o_acc[j][4 * a] * inv), static_cast<__bf16>(o_acc[j][4 * a + 1] * inv),
                                   static_cast<__bf16>(o_acc[j][4 * a + 2] * inv), static_cast<__bf16>(o_acc[j][4 * a + 3] * inv)};
                *reinterpret_cast<pbf16x4 *>(orow + 32 * j + 8 * a + 4 * h) = w;
            }
    }
}

// Launches the kernel for the head shapes it is built for; false if (q_heads / kv_heads, head_dim) is not one.
bool attention_prefill_bf16_launch(const float *qkv, const float *kc, const float *vc, void *out, const int *pos, int tokens,
                                   int q_heads, int kv_heads, int head_dim, int max_seq, hipStream_t s) {
    if (q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads != 0) return false;
    const int g = q_heads / kv_heads;
    const dim3 grid(static_cast<unsigned>(kv_heads), static_cast<unsigned>((tokens + kBfTileQ - 1) / kBfTileQ));
    if (kv_heads > 65535 || grid.y > 65535) return false;
#define LHIP_CASE(G, HD)                                                                                              \
    if (g == G && head_dim == HD) {                                                                                   \
        hipLaunchKernelGGL((attention_prefill_bf16_kernel<G, HD>), grid, dim3(64 * G), 0, s, qkv, kc, vc,             \
                           static_cast<__bf16 *>(out), pos, tokens, kv_heads, max_seq);                               \
        return true;                                                                                                  \
    }
    LHIP_CASE(2, 64) LHIP_CASE(4, 64) LHIP_CASE(8, 64)
    LHIP_CASE(2, 128) LHIP_CASE(4, 128) LHIP_CASE(8, 128)
#undef LHIP_CASE
    return false;
}

}  // namespace lhip
