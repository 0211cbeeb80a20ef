// The non-matmul operators of the Llama-3 decode loop, in f32, so that a
// Q8_0 model can run end to end on the device around the quantized matmuls.
// Each restates what the reference builds from primitive ops
// (examples/llama/src/model.rs; crates/luminal_nn/src/norm.rs:56-71;
// src/hl_ops/unary.rs:93-104,126-130,169-177).  They are small, memory-bound
// and written for correctness first: at batch 1 more than 95 % of the bytes a
// decode step touches are the quantized weights.
//
// Positions are read from device memory (`pos_dev`), so a whole decode step can
// be captured once in a HIP graph and replayed while the position advances on
// the device.
#include "common.h"

namespace lhip {

// attention_prefill.hip: matrix-core kernel for prompt-sized calls; false if the shape is not built.
bool attention_prefill_launch(const float *qkv, const float *kc, const float *vc, void *out, bool out_bf16, const int *pos,
                              int tokens, int q_heads, int kv_heads, int head_dim, int max_seq, hipStream_t s);
// attention_prefill_bf16.hip: the same sweep with bf16 matrix-core operands, bf16 out.
bool attention_prefill_bf16_launch(const float *qkv, const float *kc, const float *vc, void *out, const int *pos, int tokens,
                                   int q_heads, int kv_heads, int head_dim, int max_seq, hipStream_t s);

__device__ __forceinline__ float block_sum(float v, float *red) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();  // protect red against the previous use
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < static_cast<int>(blockDim.x >> 6); ++w) t += red[w];
    return t;
}

__device__ __forceinline__ float block_max(float v, float *red) {
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
    if (lane == 0) red[wave] = v;
    __syncthreads();
    float t = red[0];
    for (int w = 1; w < static_cast<int>(blockDim.x >> 6); ++w) t = fmaxf(t, red[w]);
    return t;
}

// out[t][:] = table[(int)idx[t]][:]   (Embedding / CPU Gather, crates/luminal_cpu/src/binary.rs:175-191)
__global__ __launch_bounds__(256) void gather_rows_kernel(const float4 *__restrict__ table,
                                                          const float *__restrict__ idx, float4 *__restrict__ out,
                                                          int n_rows, int dim4) {
    const int t = blockIdx.x;
    const float fi = idx[t];
    const long row = (fi >= 0.0f && fi < 2147483648.0f) ? static_cast<long>(fi) : -1;
    float4 *o = out + static_cast<size_t>(t) * dim4;
    for (int j = threadIdx.x; j < dim4; j += 256)
        o[j] = (row >= 0 && row < n_rows) ? table[static_cast<size_t>(row) * dim4 + j] : make_float4(0, 0, 0, 0);
}

// y = (x [+ res]) * 1/sqrt(mean(x^2) + eps) * w ; if res is given, x_out receives x + res
// (LayerNorm with mean_norm = false: std_norm then weight, norm.rs:56-71, unary.rs:93-104).
// One block of 1024 threads per row; each thread keeps up to 4 float4 of the row in
// registers between the two passes (dim <= 16384, dim % 4 == 0); x_out may alias x.
template <typename OutT>
__device__ __forceinline__ void store4(OutT *p, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void store4<float>(float *p, float a, float b, float c, float d) {
    *reinterpret_cast<float4 *>(p) = make_float4(a, b, c, d);
}
template <>
__device__ __forceinline__ void store4<__bf16>(__bf16 *p, float a, float b, float c, float d) {  // round to nearest even
    typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
    *reinterpret_cast<bf16x4 *>(p) = bf16x4{static_cast<__bf16>(a), static_cast<__bf16>(b), static_cast<__bf16>(c),
                                            static_cast<__bf16>(d)};
}

template <typename OutT>
__global__ __launch_bounds__(1024) void rms_norm_kernel(const float *x, const float *res, float *x_out,
                                                        const float *__restrict__ w, OutT *__restrict__ y, int dim,
                                                        float eps) {
    __shared__ float red[16];
    const size_t base = static_cast<size_t>(blockIdx.x) * dim;
    const int dim4 = dim >> 2;
    const float4 *x4 = reinterpret_cast<const float4 *>(x + base);
    const float4 *r4 = res ? reinterpret_cast<const float4 *>(res + base) : nullptr;
    float4 v[4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int j = threadIdx.x + i * 1024;
        v[i] = make_float4(0, 0, 0, 0);
        if (j < dim4) {
            v[i] = x4[j];
            if (r4) {
                const float4 r = r4[j];
                v[i].x += r.x; v[i].y += r.y; v[i].z += r.z; v[i].w += r.w;
            }
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int j = threadIdx.x + i * 1024;
        if (j < dim4) {
            if (r4) reinterpret_cast<float4 *>(x_out + base)[j] = v[i];
            ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
        }
    }
    const float total = block_sum(ss, red);
    const float scale = 1.0f / sqrtf(total / static_cast<float>(dim) + eps);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int j = threadIdx.x + i * 1024;
        if (j < dim4) {
            const float4 g = reinterpret_cast<const float4 *>(w)[j];
            store4<OutT>(y + base + 4 * j, v[i].x * scale * g.x, v[i].y * scale * g.y, v[i].z * scale * g.z,
                         v[i].w * scale * g.w);
        }
    }
}

// Rotary embedding on adjacent pairs (the ggml layout of model.rs:52-72) for the q and k
// parts of a fused qkv row, then k and v are appended to the cache at position pos0 + s.
// qkv: [S][(hq + 2*hkv) * hd]; caches: [hkv][max_seq][hd].  One block per (token, head).
__global__ __launch_bounds__(64) void rope_kv_kernel(float *__restrict__ qkv, float *__restrict__ k_cache,
                                                     float *__restrict__ v_cache, const int *__restrict__ pos_dev,
                                                     int hq, int hkv, int hd, int max_seq, float theta) {
    const int s = blockIdx.x, head = blockIdx.y;  // head in [0, hq + 2*hkv)
    const int pos = *pos_dev + s;
    float *row = qkv + (static_cast<size_t>(s) * (hq + 2 * hkv) + head) * hd;
    const int half = hd / 2;
    if (head < hq + hkv) {  // q or k: rotate
        for (int j = threadIdx.x; j < half; j += 64) {
            const float inv_freq = 1.0f / powf(theta, static_cast<float>(2 * j) / static_cast<float>(hd));
            const float ang = static_cast<float>(pos) * inv_freq;
            float sn, cs;
            sincosf(ang, &sn, &cs);
            const float x0 = row[2 * j], x1 = row[2 * j + 1];
            const float y0 = x0 * cs - x1 * sn, y1 = x0 * sn + x1 * cs;
            row[2 * j] = y0;
            row[2 * j + 1] = y1;
            if (head >= hq && pos < max_seq) {
                float *kc = k_cache + (static_cast<size_t>(head - hq) * max_seq + pos) * hd;
                kc[2 * j] = y0;
                kc[2 * j + 1] = y1;
            }
        }
    } else if (pos < max_seq) {  // v: copy
        float *vc = v_cache + (static_cast<size_t>(head - hq - hkv) * max_seq + pos) * hd;
        for (int j = threadIdx.x; j < hd; j += 64) vc[j] = row[j];
    }
}

// Causal grouped-query attention for S query tokens at positions pos0 .. pos0+S-1 over the
// cache (model.rs:112-139): scores = q.k / sqrt(hd), masked positions get f16::MIN added (they
// vanish in the softmax, so they are skipped), softmax, times V.  One block per (token, q head).
// q is read from the fused qkv rows; out: [S][hq*hd].  Dynamic LDS: max_seq floats.
//
// Scores: 16 lanes share a key (each holds hd/16 elements of q in registers); the block's
// 1024 threads score 64 keys per round and 8 rounds per trip, so up to 512 key rows are
// requested before the first one is used — a decode step over a few hundred keys is one or
// two memory round trips instead of one per key.
// P.V: 32 lanes cover hd as float4 and 32 such groups split the keys, 8 keys per group and
// trip; partial sums meet in LDS.  Requires hd % 64 == 0 (hd = 64, 128, 192, 256).
constexpr int kAttnThreads = 1024;

__global__ __launch_bounds__(kAttnThreads) void attention_kernel(const float *__restrict__ qkv,
                                                                  const float *__restrict__ k_cache,
                                                                  const float *__restrict__ v_cache,
                                                                  float *__restrict__ out,
                                                                  const int *__restrict__ pos_dev, int hq, int hkv,
                                                                  int hd, int max_seq) {
    extern __shared__ float sc[];  // scores of this query
    __shared__ float red[16];
    __shared__ float4 part[32][64];  // P.V partial sums: 32 key groups x hd/4 float4
    const int s = blockIdx.x, h = blockIdx.y;
    const int n_keys = min(*pos_dev + s + 1, max_seq);
    const int kvh = h / (hq / hkv);
    const float *q = qkv + (static_cast<size_t>(s) * (hq + 2 * hkv) + h) * hd;
    const float *kc = k_cache + static_cast<size_t>(kvh) * max_seq * hd;
    const float *vc = v_cache + static_cast<size_t>(kvh) * max_seq * hd;
    const float inv_sqrt = 1.0f / sqrtf(static_cast<float>(hd));

    // ---- scores
    const int sub = threadIdx.x & 15;    // which slice of hd
    const int kslot = threadIdx.x >> 4;  // which of the 64 keys of a round
    const int per = hd / 16;             // 4, 8, 12 or 16 floats per lane, as float4s
    float4 qr[4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
        qr[j] = (j * 4 < per) ? *reinterpret_cast<const float4 *>(q + sub * per + j * 4) : make_float4(0, 0, 0, 0);
    float mx = -3.0e38f;
    for (int p0 = 0; p0 < n_keys; p0 += 512) {
        float d[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int p = p0 + u * 64 + kslot;
            d[u] = 0.f;
            if (p < n_keys) {
                const float *kr = kc + static_cast<size_t>(p) * hd + sub * per;
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    if (j * 4 < per) {
                        const float4 kv = *reinterpret_cast<const float4 *>(kr + j * 4);
                        d[u] += qr[j].x * kv.x + qr[j].y * kv.y + qr[j].z * kv.z + qr[j].w * kv.w;
                    }
            }
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            float v = d[u];
            for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o);
            v *= inv_sqrt;
            const int p = p0 + u * 64 + kslot;
            if (p < n_keys) {
                if (sub == 0) sc[p] = v;
                mx = fmaxf(mx, v);
            }
        }
    }
    mx = block_max(mx, red);
    float sum = 0.f;
    for (int p = threadIdx.x; p < n_keys; p += kAttnThreads) {
        const float e = expf(sc[p] - mx);
        sc[p] = e;
        sum += e;
    }
    sum = block_sum(sum, red);  // also makes the exponentials visible to every thread
    const float inv = 1.0f / sum;

    // ---- P.V
    const int c4 = threadIdx.x & 31;  // float4 column (and c4 + 32 when hd > 128)
    const int kg = threadIdx.x >> 5;  // key group 0..31
    const int hd4 = hd / 4;
    float4 a0 = make_float4(0, 0, 0, 0), a1 = make_float4(0, 0, 0, 0);
    const bool lo_col = c4 < hd4, hi_col = c4 + 32 < hd4;
    for (int p0 = kg; p0 < n_keys; p0 += 256) {  // 8 keys per trip and group: their loads are independent
        float w[8];
        float4 v0[8], v1[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int p = p0 + 32 * u;
            const bool live = p < n_keys;
            const float4 *vr = reinterpret_cast<const float4 *>(vc + static_cast<size_t>(live ? p : 0) * hd);
            w[u] = live ? sc[p] : 0.f;
            v0[u] = lo_col ? vr[c4] : make_float4(0, 0, 0, 0);
            v1[u] = hi_col ? vr[c4 + 32] : make_float4(0, 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            a0.x += w[u] * v0[u].x; a0.y += w[u] * v0[u].y; a0.z += w[u] * v0[u].z; a0.w += w[u] * v0[u].w;
            a1.x += w[u] * v1[u].x; a1.y += w[u] * v1[u].y; a1.z += w[u] * v1[u].z; a1.w += w[u] * v1[u].w;
        }
    }
    part[kg][c4] = a0;
    part[kg][c4 + 32] = a1;
    __syncthreads();
    if (threadIdx.x < hd4) {
        float4 t = part[0][threadIdx.x];
        for (int g = 1; g < 32; ++g) {
            const float4 u = part[g][threadIdx.x];
            t.x += u.x; t.y += u.y; t.z += u.z; t.w += u.w;
        }
        float4 *o = reinterpret_cast<float4 *>(out + (static_cast<size_t>(s) * hq + h) * hd);
        o[threadIdx.x] = make_float4(t.x * inv, t.y * inv, t.z * inv, t.w * inv);
    }
}

// out[s][j] = up * swish(gate), gate = gu[s][j], up = gu[s][f + j]   (model.rs:24-32)
template <typename OutT>
__global__ __launch_bounds__(256) void swiglu_kernel(const float *__restrict__ gu, OutT *__restrict__ out, int f,
                                                     size_t total, int interleaved) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= total) return;
    const size_t s = i / f;
    const int j = static_cast<int>(i - s * f);
    const float g = gu[s * 2 * f + (interleaved ? 2 * j : j)];
    const float u = gu[s * 2 * f + (interleaved ? 2 * j + 1 : f + j)];
    out[i] = static_cast<OutT>(swiglu_value(g, u));
}

__global__ __launch_bounds__(256) void cast_f32_bf16_kernel(const float *__restrict__ x, __bf16 *__restrict__ y,
                                                            size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) y[i] = static_cast<__bf16>(x[i]);  // round to nearest even
}

__global__ __launch_bounds__(256) void cast_bf16_f32_kernel(const __bf16 *__restrict__ x, float *__restrict__ y,
                                                            size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) y[i] = static_cast<float>(x[i]);
}

__global__ __launch_bounds__(256) void add_kernel(float *__restrict__ x, const float *__restrict__ y, size_t n) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) x[i] += y[i];
}

// Greedy pick: index of the largest value; on exact ties the last one, as itertools'
// position_max_by does in the reference's loop (examples/llama/src/main.rs:194-198).  The
// index is written as f32 (token ids travel as f32 in luminal) and as int32, and the position
// counter is advanced by `advance`.
__global__ __launch_bounds__(1024) void argmax_kernel(const float *__restrict__ x, int n, float *__restrict__ id_f32,
                                                      int *__restrict__ id_i32, int *__restrict__ pos_dev,
                                                      int advance) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    float v = -3.4e38f;
    int idx = -1;
    auto take = [&](float c, int j) {
        if (idx < 0 || c > v || (c == v && j > idx)) {
            v = c;
            idx = j;
        }
    };
    const int n4 = ((reinterpret_cast<uintptr_t>(x) & 15) == 0) ? n >> 2 : 0;  // vector part
    const float4 *x4 = reinterpret_cast<const float4 *>(x);
    constexpr int U = 16;  // independent loads per trip: a 128k-entry row is two memory round trips
    for (int j0 = threadIdx.x; j0 < n4; j0 += U * 1024) {
        float4 c[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = j0 + u * 1024;
            c[u] = j < n4 ? x4[j] : make_float4(-3.4e38f, -3.4e38f, -3.4e38f, -3.4e38f);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = (j0 + u * 1024) * 4;
            if (j0 + u * 1024 < n4) {
                take(c[u].x, j); take(c[u].y, j + 1); take(c[u].z, j + 2); take(c[u].w, j + 3);
            }
        }
    }
    for (int j = n4 * 4 + threadIdx.x; j < n; j += 1024) take(x[j], j);
    for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(v, o);
        const int oi = __shfl_xor(idx, o);
        if (oi >= 0 && (idx < 0 || ov > v || (ov == v && oi > idx))) {
            v = ov;
            idx = oi;
        }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
        bv[wave] = v;
        bi[wave] = idx;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < 16; ++w)
            if (bi[w] >= 0 && (bi[0] < 0 || bv[w] > bv[0] || (bv[w] == bv[0] && bi[w] > bi[0]))) {
                bv[0] = bv[w];
                bi[0] = bi[w];
            }
        if (id_f32) *id_f32 = static_cast<float>(bi[0]);
        if (id_i32) *id_i32 = bi[0];
        if (pos_dev) *pos_dev += advance;
    }
}

// The same pick in two launches for long rows: kArgmaxBlocks workgroups each leave the best (value, index) of
// their contiguous part (one memory round trip instead of a single workgroup's many), a wave picks among those
// and the n % 4 trailing entries.  The partial results live in a small per-device array; calls that overlap on
// one device race for it, like every other call that shares scratch memory.
constexpr int kArgmaxBlocks = 64;
static __device__ __align__(256) float argmax_part[2 * kArgmaxBlocks];

__device__ inline void argmax_take(float &v, int &idx, float c, int j) {
    if (j >= 0 && (idx < 0 || c > v || (c == v && j > idx))) {
        v = c;
        idx = j;
    }
}

__global__ __launch_bounds__(1024) void argmax_partial_kernel(const float4 *__restrict__ x4, int n4,
                                                              float *__restrict__ part) {
    __shared__ float bv[16];
    __shared__ int bi[16];
    const int per = (n4 + kArgmaxBlocks - 1) / kArgmaxBlocks;
    const int begin = blockIdx.x * per, end = min(n4, begin + per);
    float v = -3.4e38f;
    int idx = -1;
    constexpr int U = 2;
    for (int j0 = begin + threadIdx.x; j0 < end; j0 += U * 1024) {
        float4 c[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = j0 + u * 1024;
            c[u] = j < end ? x4[j] : make_float4(0.f, 0.f, 0.f, 0.f);
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int j = j0 + u * 1024;
            if (j < end) {
                argmax_take(v, idx, c[u].x, 4 * j); argmax_take(v, idx, c[u].y, 4 * j + 1);
                argmax_take(v, idx, c[u].z, 4 * j + 2); argmax_take(v, idx, c[u].w, 4 * j + 3);
            }
        }
    }
    for (int o = 32; o > 0; o >>= 1) argmax_take(v, idx, __shfl_xor(v, o), __shfl_xor(idx, o));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) {
        bv[wave] = v;
        bi[wave] = idx;
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        v = lane < 16 ? bv[lane] : 0.f;
        idx = lane < 16 ? bi[lane] : -1;
        for (int o = 8; o > 0; o >>= 1) argmax_take(v, idx, __shfl_xor(v, o), __shfl_xor(idx, o));
        if (lane == 0) {
            part[2 * blockIdx.x] = v;
            part[2 * blockIdx.x + 1] = __int_as_float(idx);
        }
    }
}

__global__ __launch_bounds__(64) void argmax_final_kernel(const float *__restrict__ part, const float *__restrict__ x,
                                                          int n4, int n, float *__restrict__ id_f32,
                                                          int *__restrict__ id_i32, int *__restrict__ pos_dev,
                                                          int advance) {
    const int lane = threadIdx.x;
    float v = part[2 * lane];
    int idx = __float_as_int(part[2 * lane + 1]);
    const int t = 4 * n4 + lane;  // at most three trailing entries
    if (t < n) argmax_take(v, idx, x[t], t);
    for (int o = 32; o > 0; o >>= 1) argmax_take(v, idx, __shfl_xor(v, o), __shfl_xor(idx, o));
    if (lane == 0) {
        if (id_f32) *id_f32 = static_cast<float>(idx);
        if (id_i32) *id_i32 = idx;
        if (pos_dev) *pos_dev += advance;
    }
}

lhip_status argmax_impl(const float *x_dev, int64_t n, float *id_f32_dev, int32_t *id_i32_dev, int32_t *pos_dev,
                        int32_t advance, float *workspace, void *stream);

static float *argmax_part_ptr() {
    static float *ptrs[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    float *p = __atomic_load_n(&ptrs[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        if (hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(argmax_part)) != hipSuccess) return nullptr;
        __atomic_store_n(&ptrs[dev], p, __ATOMIC_RELEASE);
    }
    return p;
}

template <typename OutT>
static lhip_status rms_norm_any(const float *x_dev, const float *residual_dev, float *x_out_dev, const float *w_dev,
                                OutT *y_dev, int64_t rows, int64_t dim, float eps, void *stream) {
    if (!x_dev || !w_dev || !y_dev || (residual_dev && !x_out_dev)) return LHIP_ERR_NULL_PTR;
    if (rows <= 0 || dim <= 0 || rows > kMaxDim || dim > 16384 || dim % 4 != 0) return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(x_dev, 16) || !aligned(w_dev, 16) || !aligned(y_dev, 4 * sizeof(OutT)) ||
        (residual_dev && (!aligned(residual_dev, 16) || !aligned(x_out_dev, 16))))
        return LHIP_ERR_MISALIGNED;
    hipLaunchKernelGGL(rms_norm_kernel<OutT>, dim3(static_cast<unsigned>(rows)), dim3(1024), 0, as_stream(stream), x_dev,
                       residual_dev, x_out_dev, w_dev, y_dev, static_cast<int>(dim), eps);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

template <typename OutT>
static lhip_status swiglu_any(const float *gate_up_dev, OutT *out_dev, int64_t rows, int64_t f, int interleaved,
                              void *stream) {
    if (!gate_up_dev || !out_dev) return LHIP_ERR_NULL_PTR;
    if (rows <= 0 || f <= 0 || rows > kMaxDim || f > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
    const size_t total = static_cast<size_t>(rows) * static_cast<size_t>(f);
    hipLaunchKernelGGL(swiglu_kernel<OutT>, dim3(static_cast<unsigned>((total + 255) / 256)), dim3(256), 0,
                       as_stream(stream), gate_up_dev, out_dev, static_cast<int>(f), total, interleaved);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

}  // namespace lhip

using namespace lhip;

extern "C" {

lhip_status lhip_gather_rows_f32(const float *table_dev, const float *idx_dev, float *out_dev, int64_t n_idx,
                                 int64_t n_rows, int64_t dim, void *stream) {
    if (!table_dev || !idx_dev || !out_dev) return LHIP_ERR_NULL_PTR;
    if (n_idx <= 0 || n_rows <= 0 || dim <= 0 || dim % 4 != 0 || n_idx > kMaxDim || n_rows > kMaxDim || dim > kMaxDim)
        return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(table_dev, 16) || !aligned(out_dev, 16)) return LHIP_ERR_MISALIGNED;
    hipLaunchKernelGGL(gather_rows_kernel, dim3(static_cast<unsigned>(n_idx)), dim3(256), 0, as_stream(stream),
                       reinterpret_cast<const float4 *>(table_dev), idx_dev, reinterpret_cast<float4 *>(out_dev),
                       static_cast<int>(n_rows), static_cast<int>(dim / 4));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_rms_norm_f32(const float *x_dev, const float *residual_dev, float *x_out_dev, const float *w_dev,
                              float *y_dev, int64_t rows, int64_t dim, float eps, void *stream) {
    return rms_norm_any<float>(x_dev, residual_dev, x_out_dev, w_dev, y_dev, rows, dim, eps, stream);
}

lhip_status lhip_rms_norm_f32_bf16out(const float *x_dev, const float *residual_dev, float *x_out_dev,
                                      const float *w_dev, void *y_bf16_dev, int64_t rows, int64_t dim, float eps,
                                      void *stream) {
    return rms_norm_any<__bf16>(x_dev, residual_dev, x_out_dev, w_dev, static_cast<__bf16 *>(y_bf16_dev), rows, dim, eps,
                                stream);
}

lhip_status lhip_rope_kv_append_f32(float *qkv_dev, float *k_cache_dev, float *v_cache_dev, const int32_t *pos_dev,
                                    int64_t tokens, int64_t q_heads, int64_t kv_heads, int64_t head_dim,
                                    int64_t max_seq, float theta, void *stream) {
    if (!qkv_dev || !k_cache_dev || !v_cache_dev || !pos_dev) return LHIP_ERR_NULL_PTR;
    if (tokens <= 0 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || head_dim % 2 != 0 || max_seq <= 0 ||
        q_heads % kv_heads != 0 || tokens > kMaxDim || q_heads + 2 * kv_heads > 65535 || max_seq > kMaxDim)
        return LHIP_ERR_INVALID_SHAPE;
    hipLaunchKernelGGL(rope_kv_kernel, dim3(static_cast<unsigned>(tokens), static_cast<unsigned>(q_heads + 2 * kv_heads)),
                       dim3(64), 0, as_stream(stream), qkv_dev, k_cache_dev, v_cache_dev, pos_dev,
                       static_cast<int>(q_heads), static_cast<int>(kv_heads), static_cast<int>(head_dim),
                       static_cast<int>(max_seq), theta);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_attention_f32(const float *qkv_dev, const float *k_cache_dev, const float *v_cache_dev,
                               float *out_dev, const int32_t *pos_dev, int64_t tokens, int64_t q_heads,
                               int64_t kv_heads, int64_t head_dim, int64_t max_seq, void *stream) {
    if (!qkv_dev || !k_cache_dev || !v_cache_dev || !out_dev || !pos_dev) return LHIP_ERR_NULL_PTR;
    if (tokens <= 0 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || head_dim > 256 || head_dim % 64 != 0 ||
        max_seq <= 0 || q_heads % kv_heads != 0 || tokens > kMaxDim || q_heads > 65535 || max_seq > 12000)
        return LHIP_ERR_INVALID_SHAPE;  // the score row of one query lives in LDS
    if (tokens >= 8 && aligned(qkv_dev, 16) && aligned(k_cache_dev, 16) && aligned(v_cache_dev, 16) && aligned(out_dev, 16) &&
        attention_prefill_launch(qkv_dev, k_cache_dev, v_cache_dev, out_dev, false, pos_dev, static_cast<int>(tokens),
                                 static_cast<int>(q_heads), static_cast<int>(kv_heads), static_cast<int>(head_dim),
                                 static_cast<int>(max_seq), as_stream(stream))) {
        LHIP_CHECK_LAUNCH();
        return LHIP_OK;
    }
    // the score row is dynamic LDS on top of 32.1 KiB of static arrays: past 64 KiB in all the kernel has to opt in
    static LdsOptIn opt;
    if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(attention_kernel), static_cast<size_t>(max_seq) * sizeof(float),
                                    static_cast<size_t>(max_seq) * sizeof(float) + sizeof(float4) * 32 * 64 + 64 > 64 * 1024))
        return st;
    hipLaunchKernelGGL(attention_kernel, dim3(static_cast<unsigned>(tokens), static_cast<unsigned>(q_heads)),
                       dim3(kAttnThreads),
                       static_cast<size_t>(max_seq) * sizeof(float), as_stream(stream), qkv_dev, k_cache_dev,
                       v_cache_dev, out_dev, pos_dev, static_cast<int>(q_heads), static_cast<int>(kv_heads),
                       static_cast<int>(head_dim), static_cast<int>(max_seq));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_attention_f32_bf16out(const float *qkv_dev, const float *k_cache_dev, const float *v_cache_dev,
                                       void *out_bf16_dev, const int32_t *pos_dev, int64_t tokens, int64_t q_heads,
                                       int64_t kv_heads, int64_t head_dim, int64_t max_seq, void *stream) {
    if (!qkv_dev || !k_cache_dev || !v_cache_dev || !out_bf16_dev || !pos_dev) return LHIP_ERR_NULL_PTR;
    if (tokens <= 0 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || max_seq <= 0 || q_heads % kv_heads != 0 ||
        tokens > kMaxDim || max_seq > kMaxDim)
        return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(qkv_dev, 16) || !aligned(k_cache_dev, 16) || !aligned(v_cache_dev, 16) || !aligned(out_bf16_dev, 8))
        return LHIP_ERR_MISALIGNED;
    if (!attention_prefill_launch(qkv_dev, k_cache_dev, v_cache_dev, out_bf16_dev, true, pos_dev, static_cast<int>(tokens),
                                  static_cast<int>(q_heads), static_cast<int>(kv_heads), static_cast<int>(head_dim),
                                  static_cast<int>(max_seq), as_stream(stream)))
        return LHIP_ERR_UNSUPPORTED;  // only the matrix-core kernel writes bf16
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_attention_bf16(const float *qkv_dev, const float *k_cache_dev, const float *v_cache_dev,
                                void *out_bf16_dev, const int32_t *pos_dev, int64_t tokens, int64_t q_heads,
                                int64_t kv_heads, int64_t head_dim, int64_t max_seq, void *stream) {
    if (!qkv_dev || !k_cache_dev || !v_cache_dev || !out_bf16_dev || !pos_dev) return LHIP_ERR_NULL_PTR;
    if (tokens <= 0 || q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || max_seq <= 0 || q_heads % kv_heads != 0 ||
        tokens > kMaxDim || max_seq > kMaxDim)
        return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(qkv_dev, 16) || !aligned(k_cache_dev, 16) || !aligned(v_cache_dev, 16) || !aligned(out_bf16_dev, 8))
        return LHIP_ERR_MISALIGNED;
    if (!attention_prefill_bf16_launch(qkv_dev, k_cache_dev, v_cache_dev, out_bf16_dev, pos_dev, static_cast<int>(tokens),
                                       static_cast<int>(q_heads), static_cast<int>(kv_heads), static_cast<int>(head_dim),
                                       static_cast<int>(max_seq), as_stream(stream)))
        return LHIP_ERR_UNSUPPORTED;
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_swiglu_f32(const float *gate_up_dev, float *out_dev, int64_t rows, int64_t f, int interleaved,
                            void *stream) {
    return swiglu_any<float>(gate_up_dev, out_dev, rows, f, interleaved, stream);
}

lhip_status lhip_swiglu_f32_bf16out(const float *gate_up_dev, void *out_bf16_dev, int64_t rows, int64_t f,
                                    int interleaved, void *stream) {
    return swiglu_any<__bf16>(gate_up_dev, static_cast<__bf16 *>(out_bf16_dev), rows, f, interleaved, stream);
}

lhip_status lhip_add_f32(float *x_dev, const float *y_dev, int64_t n, void *stream) {
    if (!x_dev || !y_dev) return LHIP_ERR_NULL_PTR;
    if (n <= 0) return LHIP_ERR_INVALID_SHAPE;
    hipLaunchKernelGGL(add_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0, as_stream(stream), x_dev,
                       y_dev, static_cast<size_t>(n));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_cast_f32_to_bf16(const float *x_dev, void *y_dev, int64_t n, void *stream) {
    if (!x_dev || !y_dev) return LHIP_ERR_NULL_PTR;
    if (n <= 0) return LHIP_ERR_INVALID_SHAPE;
    hipLaunchKernelGGL(cast_f32_bf16_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0,
                       as_stream(stream), x_dev, static_cast<__bf16 *>(y_dev), static_cast<size_t>(n));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_cast_bf16_to_f32(const void *x_dev, float *y_dev, int64_t n, void *stream) {
    if (!x_dev || !y_dev) return LHIP_ERR_NULL_PTR;
    if (n <= 0) return LHIP_ERR_INVALID_SHAPE;
    hipLaunchKernelGGL(cast_bf16_f32_kernel, dim3(static_cast<unsigned>((n + 255) / 256)), dim3(256), 0,
                       as_stream(stream), static_cast<const __bf16 *>(x_dev), y_dev, static_cast<size_t>(n));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_argmax_f32(const float *x_dev, int64_t n, float *id_f32_dev, int32_t *id_i32_dev, int32_t *pos_dev,
                            int32_t advance, void *stream) {
    return argmax_impl(x_dev, n, id_f32_dev, id_i32_dev, pos_dev, advance, nullptr, stream);
}

lhip_status lhip_argmax_f32_ws(const float *x_dev, int64_t n, float *id_f32_dev, int32_t *id_i32_dev, int32_t *pos_dev,
                               int32_t advance, void *workspace_dev, void *stream) {
    if (!workspace_dev) return LHIP_ERR_NULL_PTR;
    if (!aligned(workspace_dev, 8)) return LHIP_ERR_MISALIGNED;
    return argmax_impl(x_dev, n, id_f32_dev, id_i32_dev, pos_dev, advance, static_cast<float *>(workspace_dev), stream);
}

}  // extern "C"

namespace lhip {

lhip_status argmax_impl(const float *x_dev, int64_t n, float *id_f32_dev, int32_t *id_i32_dev, int32_t *pos_dev,
                        int32_t advance, float *workspace, void *stream) {
    if (!x_dev || (!id_f32_dev && !id_i32_dev)) return LHIP_ERR_NULL_PTR;
    if (n <= 0 || n > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
    if (n >= 16384 && aligned(x_dev, 16)) {  // long rows: partial picks over the chip, then one wave
        float *part = workspace ? workspace : argmax_part_ptr();
        if (!part) return LHIP_ERR_HIP;
        const int n4 = static_cast<int>(n >> 2);
        hipLaunchKernelGGL(argmax_partial_kernel, dim3(kArgmaxBlocks), dim3(1024), 0, as_stream(stream),
                           reinterpret_cast<const float4 *>(x_dev), n4, part);
        LHIP_CHECK_LAUNCH();
        hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(64), 0, as_stream(stream), part, x_dev, n4,
                           static_cast<int>(n), id_f32_dev, id_i32_dev, pos_dev, advance);
        LHIP_CHECK_LAUNCH();
        return LHIP_OK;
    }
    hipLaunchKernelGGL(argmax_kernel, dim3(1), dim3(1024), 0, as_stream(stream), x_dev, static_cast<int>(n), id_f32_dev,
                       id_i32_dev, pos_dev, advance);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

}  // namespace lhip
