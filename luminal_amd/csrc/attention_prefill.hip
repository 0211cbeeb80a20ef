// Causal grouped-query attention for a block of prompt tokens on the f32 matrix cores.
//
// Same operator as attention_kernel in llama_ops.hip (examples/llama/src/model.rs:112-139: scores = q.k/sqrt(hd),
// causal mask, softmax, times V, over the KV cache that already holds the new tokens), for many query tokens:
// a flash-attention sweep with v_mfma_f32_32x32x2_f32, so inputs, products and sums stay f32 and the result meets
// the same bar as the scalar kernel.
//
// Work split: one workgroup per (KV head, block of 32 query tokens); its G waves are the G query heads that share
// the KV head, so they walk the same key tiles (32 keys each, staged once in LDS for all of them) under the same
// causal limit.
//
// Per wave and key tile, with lane = (c, h), c = lane % 32, h = lane / 32:
//   S^T = K Q^T   (32 keys x 32 queries): A = K, B = Q^T.  The summation index of an MFMA step is free to name
//                 any head-dim element as long as A and B agree; lane half h takes elements h*HD/2 + step, so a
//                 lane's Q values are HD/2 consecutive floats kept in registers for the whole sweep and its K
//                 values come from LDS as 16-byte reads.
//                 Result layout: lane (c, h) holds query c, keys 8*(v/4) + 4*h + v%4, v = 0..15 — a query's
//                 scores are in one lane's registers (plus the other half), so the running max and sum need one
//                 cross-half exchange per tile and no LDS.
//   O^T += V^T P^T (HD x 32 queries): B = P^T is exactly the score registers (step (a, b) uses key 8a + 4h + b =
//                 register 4a + b); A = V^T: lane (c, h) reads V[key][4c .. 4c+3] as one 16-byte LDS read and
//                 uses its four floats for four output blocks, i.e. output row r of block j is head-dim 4r + j.
// The accumulators of O^T have the query in the lane as well, so rescaling by exp(m_old - m_new) is per lane.
#include "common.h"

namespace lhip {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kPfTileK = 32;  // keys per tile
constexpr int kPfTileQ = 32;  // queries per workgroup

template <int G, int HD, typename OutT>
// Register budget: with the default (as many waves per SIMD as the LDS allows) the compiler spills the prefetched
// tile to scratch right after requesting it, i.e. waits for the loads it was meant to overlap.  One wave per SIMD
// at head_dim 128 (Q 64 + O 64 + staging 32 registers and the sweep's temporaries), two otherwise.
__global__ __launch_bounds__(64 * G) __attribute__((amdgpu_waves_per_eu(1, (HD == 128 && G <= 4) ? 1 : 2)))
void attention_prefill_kernel(const float *__restrict__ qkv,
                                                                  const float *__restrict__ k_cache,
                                                                  const float *__restrict__ v_cache,
                                                                  OutT *__restrict__ out,
                                                                  const int *__restrict__ pos_dev, int tokens, int hkv,
                                                                  int max_seq) {
    constexpr int THREADS = 64 * G;
    constexpr int KP = HD + 4;             // LDS pitch of a K row in floats (16-byte reads of 8 rows hit 32 banks once)
    constexpr int HALF = HD / 2;           // head-dim elements per lane half
    constexpr int OB = HD / 32;            // output blocks of 32 rows of O^T; OB == 4 for HD = 128, 2 for HD = 64
    constexpr int VW = HD / 32;            // floats of a V row per lane (= OB)
    constexpr int TILE_F4 = kPfTileK * HD / 4;
    constexpr int LD = (TILE_F4 + THREADS - 1) / THREADS;  // float4 per thread and tile and matrix
    constexpr bool PREFETCH = LD <= 4;     // keep the next tile in registers during the sweep of this one
    __shared__ __attribute__((aligned(16))) float k_s[kPfTileK * KP];
    __shared__ __attribute__((aligned(16))) float v_s[kPfTileK * HD];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 31, h = lane >> 5;
    const int kvh = blockIdx.x, qb = blockIdx.y;
    const int hq = hkv * G;
    const int pos0 = *pos_dev;
    const int q0 = qb * kPfTileQ;
    const int head = kvh * G + wave;
    const int my_q = q0 + c;                               // this lane's query token
    const int my_pos = pos0 + my_q;                         // its position: keys 0..my_pos are visible
    const int n_keys = min(pos0 + min(tokens, q0 + kPfTileQ), max_seq);  // keys this workgroup can see at all
    const int n_tiles = (n_keys + kPfTileK - 1) / kPfTileK;
    const float inv_sqrt = 1.0f / sqrtf(static_cast<float>(HD));

    // ---- Q of this lane: HD/2 floats, pre-scaled by 1/sqrt(HD)
    float qreg[HALF];
    {
        const float *qrow = qkv + (static_cast<size_t>(min(my_q, tokens - 1)) * (hq + 2 * hkv) + head) * HD + h * HALF;
#pragma unroll
        for (int j = 0; j < HALF / 4; ++j) {
            const float4 t = reinterpret_cast<const float4 *>(qrow)[j];
            qreg[4 * j] = t.x * inv_sqrt; qreg[4 * j + 1] = t.y * inv_sqrt;
            qreg[4 * j + 2] = t.z * inv_sqrt; qreg[4 * j + 3] = t.w * inv_sqrt;
        }
    }

    // ---- tile staging: global -> registers -> LDS
    const float4 *kc4 = reinterpret_cast<const float4 *>(k_cache) + static_cast<size_t>(kvh) * max_seq * (HD / 4);
    const float4 *vc4 = reinterpret_cast<const float4 *>(v_cache) + static_cast<size_t>(kvh) * max_seq * (HD / 4);
    constexpr int NST = PREFETCH ? LD : 1;
    constexpr bool EXACT = TILE_F4 % THREADS == 0;  // every thread has a piece in every round: no test, so the
                                                    // staging registers are plain registers, not a private array
    float4 kst[NST], vst[NST];
    auto load_tile = [&](int t) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NST; ++i) {
            const int f = tid + i * THREADS;  // float4 index inside the tile: row = f / (HD/4)
            const int row = f / (HD / 4), col = f - row * (HD / 4);
            const int key = min(t * kPfTileK + row, n_keys - 1);  // rows past the end repeat the last key (masked)
            if (EXACT || f < TILE_F4) {
                kst[i] = kc4[static_cast<size_t>(key) * (HD / 4) + col];
                vst[i] = vc4[static_cast<size_t>(key) * (HD / 4) + col];
            }
        }
    };
    auto store_tile = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < NST; ++i) {
            const int f = tid + i * THREADS;
            const int row = f / (HD / 4), col = f - row * (HD / 4);
            if (EXACT || f < TILE_F4) {
                *reinterpret_cast<float4 *>(&k_s[row * KP + col * 4]) = kst[i];
                *reinterpret_cast<float4 *>(&v_s[row * HD + col * 4]) = vst[i];
            }
        }
    };
    // Few waves (G = 1, 2): the tile is too many registers per thread to hold, copy it through in pieces.
    auto copy_tile = [&](int t) {
        for (int f = tid; f < TILE_F4; f += THREADS) {
            const int row = f / (HD / 4), col = f - row * (HD / 4);
            const int key = min(t * kPfTileK + row, n_keys - 1);
            *reinterpret_cast<float4 *>(&k_s[row * KP + col * 4]) = kc4[static_cast<size_t>(key) * (HD / 4) + col];
            *reinterpret_cast<float4 *>(&v_s[row * HD + col * 4]) = vc4[static_cast<size_t>(key) * (HD / 4) + col];
        }
    };

    v16f o_acc[OB];
#pragma unroll
    for (int j = 0; j < OB; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) o_acc[j][v] = 0.f;
    float m_run = -INFINITY, l_run = 0.f;

    if (PREFETCH) {
        load_tile(0);
        store_tile();
    } else {
        copy_tile(0);
    }
    __syncthreads();
    for (int t = 0; t < n_tiles; ++t) {
        if (PREFETCH && t + 1 < n_tiles) load_tile(t + 1);
        // ---- S^T = K Q^T
        v16f s_acc;
#pragma unroll
        for (int v = 0; v < 16; ++v) s_acc[v] = 0.f;
        const float *krow = &k_s[c * KP + h * HALF];
#pragma unroll
        for (int j = 0; j < HALF / 4; ++j) {
            const float4 kk = *reinterpret_cast<const float4 *>(krow + 4 * j);
            s_acc = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.x, qreg[4 * j], s_acc, 0, 0, 0);
            s_acc = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.y, qreg[4 * j + 1], s_acc, 0, 0, 0);
            s_acc = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.z, qreg[4 * j + 2], s_acc, 0, 0, 0);
            s_acc = __builtin_amdgcn_mfma_f32_32x32x2f32(kk.w, qreg[4 * j + 3], s_acc, 0, 0, 0);
        }
        // ---- causal mask, running max / sum, weights in place
        float tmax = -INFINITY;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = t * kPfTileK + 8 * (v >> 2) + 4 * h + (v & 3);
            if (key > my_pos || key >= n_keys) s_acc[v] = -INFINITY;
            tmax = fmaxf(tmax, s_acc[v]);
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
        const float m_new = fmaxf(m_run, tmax);  // finite from the first tile on: key 0 is visible to every query
        const float corr = expf(m_run - m_new);
        float psum = 0.f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            s_acc[v] = expf(s_acc[v] - m_new);
            psum += s_acc[v];
        }
        psum += __shfl_xor(psum, 32);
        l_run = l_run * corr + psum;
        m_run = m_new;
#pragma unroll
        for (int j = 0; j < OB; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) o_acc[j][v] *= corr;
        // ---- O^T += V^T P^T
#pragma unroll
        for (int a = 0; a < 4; ++a)
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int key = 8 * a + 4 * h + b;
                const float p = s_acc[4 * a + b];
                const float *vrow = &v_s[key * HD + VW * c];
                if constexpr (VW == 4) {
                    const float4 vv = *reinterpret_cast<const float4 *>(vrow);
                    o_acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.x, p, o_acc[0], 0, 0, 0);
                    o_acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.y, p, o_acc[1], 0, 0, 0);
                    o_acc[2] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.z, p, o_acc[2], 0, 0, 0);
                    o_acc[3] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.w, p, o_acc[3], 0, 0, 0);
                } else {
                    const float2 vv = *reinterpret_cast<const float2 *>(vrow);
                    o_acc[0] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.x, p, o_acc[0], 0, 0, 0);
                    o_acc[1] = __builtin_amdgcn_mfma_f32_32x32x2f32(vv.y, p, o_acc[1], 0, 0, 0);
                }
            }
        // ---- next tile (one LDS buffer: a tile's sweep is thousands of cycles, the two barriers are noise)
        __syncthreads();
        if (t + 1 < n_tiles) {
            if (PREFETCH) store_tile();
            else copy_tile(t + 1);
        }
        __syncthreads();
    }

    // ---- out[q][head*HD + VW*row + j] = O^T[j][row][q] / l
    if (my_q < tokens) {
        const float inv = 1.0f / l_run;
        OutT *orow = out + (static_cast<size_t>(my_q) * hq + head) * HD;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int row = 8 * (v >> 2) + 4 * h + (v & 3);
            if constexpr (VW == 4) {
#pragma unroll
                for (int j = 0; j < 4; ++j) orow[4 * row + j] = static_cast<OutT>(o_acc[j][v] * inv);
            } else {
#pragma unroll
                for (int j = 0; j < 2; ++j) orow[2 * row + j] = static_cast<OutT>(o_acc[j][v] * inv);
            }
        }
    }
}

// Launcher used by lhip_attention_f32 for prompt-sized calls; false if this shape is not built.
bool attention_prefill_launch(const float *qkv, const float *kc, const float *vc, void *out, bool out_bf16, const int *pos,
                              int tokens, int q_heads, int kv_heads, int head_dim, int max_seq, hipStream_t s) {
    if (q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads != 0) return false;
    const int g = q_heads / kv_heads;
    const dim3 grid(static_cast<unsigned>(kv_heads), static_cast<unsigned>((tokens + kPfTileQ - 1) / kPfTileQ));
    if (kv_heads > 65535 || grid.y > 65535) return false;
#define LHIP_CASE(G, HD)                                                                                            \
    if (g == G && head_dim == HD) {                                                                                 \
        if (out_bf16)                                                                                               \
            hipLaunchKernelGGL((attention_prefill_kernel<G, HD, __bf16>), grid, dim3(64 * G), 0, s, qkv, kc, vc,    \
                               static_cast<__bf16 *>(out), pos, tokens, kv_heads, max_seq);                         \
        else                                                                                                        \
            hipLaunchKernelGGL((attention_prefill_kernel<G, HD, float>), grid, dim3(64 * G), 0, s, qkv, kc, vc,     \
                               static_cast<float *>(out), pos, tokens, kv_heads, max_seq);                          \
        return true;                                                                                                \
    }
    LHIP_CASE(1, 64) LHIP_CASE(2, 64) LHIP_CASE(4, 64) LHIP_CASE(8, 64)
    LHIP_CASE(1, 128) LHIP_CASE(2, 128) LHIP_CASE(4, 128) LHIP_CASE(8, 128)
#undef LHIP_CASE
    return false;
}

}  // namespace lhip
