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

#include "common.h"

namespace lhip {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Sum over the 64 lanes of a wavefront; every lane returns the total.
__device__ __forceinline__ float wave_sum(float v) {
    // xor 1, xor 2 inside quads, then mirror inside 8 and inside 16 lanes.
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    // Each row of 16 lanes now holds its row sum in every lane.
    const int b = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
}

__device__ __forceinline__ float sb(uint32_t w, int i) {
    return static_cast<float>(static_cast<int8_t>((w >> (8 * i)) & 0xff));
}

// Dot product of 16 int8 quants with 16 f32 activations.
__device__ __forceinline__ float dot16(const u32x4 &q, const float4 (&x)[4]) {
    float s = sb(q.x, 0) * x[0].x;
    s = fmaf(sb(q.x, 1), x[0].y, s);
    s = fmaf(sb(q.x, 2), x[0].z, s);
    s = fmaf(sb(q.x, 3), x[0].w, s);
    s = fmaf(sb(q.y, 0), x[1].x, s);
    s = fmaf(sb(q.y, 1), x[1].y, s);
    s = fmaf(sb(q.y, 2), x[1].z, s);
    s = fmaf(sb(q.y, 3), x[1].w, s);
    s = fmaf(sb(q.z, 0), x[2].x, s);
    s = fmaf(sb(q.z, 1), x[2].y, s);
    s = fmaf(sb(q.z, 2), x[2].z, s);
    s = fmaf(sb(q.z, 3), x[2].w, s);
    s = fmaf(sb(q.w, 0), x[3].x, s);
    s = fmaf(sb(q.w, 1), x[3].y, s);
    s = fmaf(sb(q.w, 2), x[3].z, s);
    s = fmaf(sb(q.w, 3), x[3].w, s);
    return s;
}

// R rows per wave, W waves per workgroup, U slices of 1024 quants per step.
// grid.x covers ceil(n / (R*W)) row tiles, grid.y the rows of x (m).
template <int R, int W, int U>
__global__ __launch_bounds__(W * 64) void q8_gemv_f32_kernel(const int8_t *__restrict__ qs,
                                                              const __half *__restrict__ ds,
                                                              const float *__restrict__ x, float *__restrict__ y,
                                                              int n, int k) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row0 = (blockIdx.x * W + wave) * R;
    if (row0 >= n) return;  // wave-uniform

    x += static_cast<size_t>(blockIdx.y) * k;
    y += static_cast<size_t>(blockIdx.y) * n;

    const int nblk = k >> 5;
    const int8_t *qrow[R];
    const __half *drow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        // Rows past the end re-read the last row; their sums are not stored.
        const int row = min(row0 + r, n - 1);
        qrow[r] = qs + static_cast<size_t>(row) * k;
        drow[r] = ds + static_cast<size_t>(row) * nblk;
    }

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;

    int kofs = lane * 16;
    // Full steps: U slices, no bounds checks.
    for (; kofs + (U - 1) * 1024 < k; kofs += U * 1024) {
        u32x4 q[U][R];
        __half d[U][R];
        float4 xv[U][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ko = kofs + u * 1024;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                q[u][r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(qrow[r] + ko));
                d[u][r] = drow[r][ko >> 5];
            }
            const float4 *xp = reinterpret_cast<const float4 *>(x + ko);
#pragma unroll
            for (int j = 0; j < 4; ++j) xv[u][j] = xp[j];
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = fmaf(dot16(q[u][r], xv[u]), __half2float(d[u][r]), acc[r]);
    }
    // Tail: remaining slices one at a time (lanes past K idle).
    for (; kofs < k; kofs += 1024) {
        float4 xv[4];
        const float4 *xp = reinterpret_cast<const float4 *>(x + kofs);
#pragma unroll
        for (int j = 0; j < 4; ++j) xv[j] = xp[j];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const u32x4 q = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(qrow[r] + kofs));
            acc[r] = fmaf(dot16(q, xv), __half2float(drow[r][kofs >> 5]), acc[r]);
        }
    }

    float out = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float s = wave_sum(acc[r]);
        if (lane == r) out = s;
    }
    if (lane < R && row0 + lane < n) y[row0 + lane] = out;
}

template <int R, int W, int U>
static lhip_status launch(const int8_t *qs, const __half *ds, const float *x, float *y, int m, int n, int k,
                          hipStream_t s) {
    const unsigned tiles = static_cast<unsigned>((n + R * W - 1) / (R * W));
    hipLaunchKernelGGL((q8_gemv_f32_kernel<R, W, U>), dim3(tiles, static_cast<unsigned>(m)), dim3(W * 64), 0, s, qs,
                       ds, x, y, n, k);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

// Launch-shape table.  rows_per_wave in {1,2,4,8}, k_unroll in {1,2,4}.
static lhip_status dispatch(int rows_per_wave, int k_unroll, const int8_t *qs, const __half *ds, const float *x,
                            float *y, int m, int n, int k, hipStream_t s) {
#define LHIP_CASE(R, U) \
    if (rows_per_wave == R && k_unroll == U) return launch<R, 4, U>(qs, ds, x, y, m, n, k, s);
    LHIP_CASE(1, 1) LHIP_CASE(1, 2) LHIP_CASE(1, 4)
    LHIP_CASE(2, 1) LHIP_CASE(2, 2) LHIP_CASE(2, 4)
    LHIP_CASE(4, 1) LHIP_CASE(4, 2) LHIP_CASE(4, 4)
    LHIP_CASE(8, 1) LHIP_CASE(8, 2)
#undef LHIP_CASE
    return LHIP_ERR_UNSUPPORTED;
}

// Heuristic: keep at least ~8 waves per CU (256 CUs) when N allows it, and
// as many 16-byte loads in flight per lane as the registers carry.
static void choose(int n, int k, int *rows_per_wave, int *k_unroll) {
    int r = 4;
    if (n < 8192) r = 2;
    if (n < 4096) r = 1;
    int u = (k >= 4096) ? 4 : (k >= 2048 ? 2 : 1);
    if (r == 4 && u == 4) u = 2;
    *rows_per_wave = r;
    *k_unroll = u;
}

static lhip_status check_args(const void *planar, const float *x, float *y, int64_t m, int64_t n, int64_t k) {
    if (!planar || !x || !y) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (m <= 0 || m > 65535) return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(planar, 256) || !aligned(x, 16) || !aligned(y, 4)) return LHIP_ERR_MISALIGNED;
    // Rows of x start at multiples of K floats; K % 32 == 0 keeps them 16-byte aligned.
    return LHIP_OK;
}

}  // namespace lhip

using namespace lhip;

extern "C" {

lhip_status lhip_q8_0_matmul_f32_cfg(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                     int64_t k, int rows_per_wave, int k_unroll, void *stream) {
    if (lhip_status s = check_args(planar_dev, x_dev, y_dev, m, n, k)) return s;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    return dispatch(rows_per_wave, k_unroll, reinterpret_cast<const int8_t *>(base),
                    reinterpret_cast<const __half *>(base + q8_scale_offset(n, k)), x_dev, y_dev, static_cast<int>(m),
                    static_cast<int>(n), static_cast<int>(k), as_stream(stream));
}

lhip_status lhip_q8_0_matmul_f32(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                 int64_t k, void *stream) {
    if (lhip_status s = check_args(planar_dev, x_dev, y_dev, m, n, k)) return s;
    int r, u;
    choose(static_cast<int>(n), static_cast<int>(k), &r, &u);
    return lhip_q8_0_matmul_f32_cfg(planar_dev, x_dev, y_dev, m, n, k, r, u, stream);
}

}  // extern "C"
