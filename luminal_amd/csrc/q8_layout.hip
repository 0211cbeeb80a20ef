// Q8_0 storage kernels: raw GGUF blocks <-> planar, dequantise, row gather.
//
// Raw block (34 B): little-endian f16 scale, then 32 int8 quants
// (crates/luminal_cuda/src/quantized.rs:30-33).  Raw rows are only 2-byte
// aligned, so these kernels move 16-bit units: unit u of the raw stream lies
// in block u/17; unit u%17 == 0 is the scale, the others are quant pairs.
// All of this is HBM-bound byte shuffling with both sides fully coalesced.
#include <hip/hip_fp16.h>

#include "common.h"

namespace lhip {

constexpr int kThreads = 256;

__global__ __launch_bounds__(kThreads) void q8_repack_kernel(const uint16_t *__restrict__ raw,
                                                              uint16_t *__restrict__ qs,
                                                              uint16_t *__restrict__ ds, size_t n_units) {
    size_t u = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * kThreads;
    for (; u < n_units; u += stride) {
        const size_t blk = u / 17;
        const unsigned off = static_cast<unsigned>(u - blk * 17);
        const uint16_t v = raw[u];
        if (off == 0)
            ds[blk] = v;
        else
            qs[blk * 16 + (off - 1)] = v;
    }
}

__global__ __launch_bounds__(kThreads) void q8_unpack_kernel(const uint16_t *__restrict__ qs,
                                                              const uint16_t *__restrict__ ds,
                                                              uint16_t *__restrict__ raw, size_t n_units) {
    size_t u = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * kThreads;
    for (; u < n_units; u += stride) {
        const size_t blk = u / 17;
        const unsigned off = static_cast<unsigned>(u - blk * 17);
        raw[u] = (off == 0) ? ds[blk] : qs[blk * 16 + (off - 1)];
    }
}

// Rows of two planar (n, k) weights taken alternately into one planar (2n, k) weight: row 2j = a's row j, row
// 2j + 1 = b's row j.  Quants move as 16-byte pieces (a row is k bytes, k a multiple of 32), scales as 16-bit units.
__global__ __launch_bounds__(kThreads) void q8_interleave_rows_kernel(const uint4 *__restrict__ qa, const uint4 *__restrict__ qb,
                                                                       uint4 *__restrict__ qo,
                                                                       const uint16_t *__restrict__ da,
                                                                       const uint16_t *__restrict__ db,
                                                                       uint16_t *__restrict__ dout, size_t n_pieces,
                                                                       size_t n_scales, unsigned pieces_per_row,
                                                                       unsigned scales_per_row) {
    const size_t first = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * kThreads;
    for (size_t c = first; c < n_pieces; c += stride) {
        const size_t row = c / pieces_per_row, at = (row >> 1) * pieces_per_row + (c - row * pieces_per_row);
        qo[c] = (row & 1) ? qb[at] : qa[at];
    }
    for (size_t c = first; c < n_scales; c += stride) {
        const size_t row = c / scales_per_row, at = (row >> 1) * scales_per_row + (c - row * scales_per_row);
        dout[c] = (row & 1) ? db[at] : da[at];
    }
}

// One thread dequantises 4 consecutive quants: w = (float)q * (float)d.  The
// product of an int8 and a binary16 value is exact in binary32.
__device__ __forceinline__ float4 dequant4(uint32_t q4, float d) {
    float4 o;
    o.x = static_cast<float>(static_cast<int8_t>(q4 & 0xff)) * d;
    o.y = static_cast<float>(static_cast<int8_t>((q4 >> 8) & 0xff)) * d;
    o.z = static_cast<float>(static_cast<int8_t>((q4 >> 16) & 0xff)) * d;
    o.w = static_cast<float>(static_cast<int8_t>(q4 >> 24)) * d;
    return o;
}

__global__ __launch_bounds__(kThreads) void q8_dequant_kernel(const uint32_t *__restrict__ qs,
                                                               const __half *__restrict__ ds,
                                                               float4 *__restrict__ out, size_t n_quads) {
    size_t i = static_cast<size_t>(blockIdx.x) * kThreads + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * kThreads;
    for (; i < n_quads; i += stride) out[i] = dequant4(qs[i], __half2float(ds[i >> 3]));
}

// Four dequantised weights in the output type: f32 as they are (the product is exact), or rounded once to f16
// (what `(half)q * (half)d` gives: crates/luminal_cuda/src/quantized.rs:196-199 multiplies in T).
struct Half4 {
    __half2 lo, hi;
};
__device__ __forceinline__ void store_quad(float4 *o, int j, float4 v) { o[j] = v; }
__device__ __forceinline__ void store_quad(Half4 *o, int j, float4 v) {
    o[j] = Half4{__floats2half2_rn(v.x, v.y), __floats2half2_rn(v.z, v.w)};
}

// grid.x = index row, threads stride over the K/4 quads of that row.
template <typename Quad>
__global__ __launch_bounds__(kThreads) void q8_gather_kernel(const uint32_t *__restrict__ qs,
                                                              const __half *__restrict__ ds,
                                                              const float *__restrict__ idx,
                                                              Quad *__restrict__ out, int n, int k) {
    const int t = blockIdx.x;
    const float fi = idx[t];
    // `as usize` in the reference's CPU gather truncates toward zero.
    const long row = (fi >= 0.0f && fi < 2147483648.0f) ? static_cast<long>(fi) : -1;
    const int quads = k >> 2;
    Quad *o = out + static_cast<size_t>(t) * quads;
    if (row < 0 || row >= n) {
        for (int j = threadIdx.x; j < quads; j += kThreads) store_quad(o, j, make_float4(0.f, 0.f, 0.f, 0.f));
        return;
    }
    const uint32_t *q = qs + static_cast<size_t>(row) * quads;
    const __half *d = ds + static_cast<size_t>(row) * (k >> 5);
    for (int j = threadIdx.x; j < quads; j += kThreads) store_quad(o, j, dequant4(q[j], __half2float(d[j >> 3])));
}

static inline unsigned grid_for(size_t items) {
    size_t g = (items + kThreads - 1) / kThreads;
    // Grid-stride loops: cap the grid at a few waves per SIMD of the whole chip.
    const size_t cap = 256u * 64u;
    return static_cast<unsigned>(g < cap ? (g ? g : 1) : cap);
}

}  // namespace lhip

using namespace lhip;

extern "C" {

size_t lhip_q8_0_raw_nbytes(int64_t n, int64_t k) {
    if (check_q8_shape(n, k) != LHIP_OK) return 0;
    size_t e = static_cast<size_t>(n) * static_cast<size_t>(k);
    return e + e / 16;
}

size_t lhip_q8_0_planar_nbytes(int64_t n, int64_t k) {
    if (check_q8_shape(n, k) != LHIP_OK) return 0;
    return q8_planar_nbytes(n, k);
}

size_t lhip_q8_0_planar_scale_offset(int64_t n, int64_t k) {
    if (check_q8_shape(n, k) != LHIP_OK) return 0;
    return q8_scale_offset(n, k);
}

lhip_status lhip_q8_0_repack(const void *raw_dev, void *planar_dev, int64_t n, int64_t k, void *stream) {
    if (!raw_dev || !planar_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (!aligned(raw_dev, 2) || !aligned(planar_dev, 256)) return LHIP_ERR_MISALIGNED;
    const size_t n_units = static_cast<size_t>(n) * (k / 32) * 17;
    auto *base = static_cast<uint8_t *>(planar_dev);
    hipLaunchKernelGGL(q8_repack_kernel, dim3(grid_for(n_units)), dim3(kThreads), 0, as_stream(stream),
                       static_cast<const uint16_t *>(raw_dev), reinterpret_cast<uint16_t *>(base),
                       reinterpret_cast<uint16_t *>(base + q8_scale_offset(n, k)), n_units);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_q8_0_unpack(const void *planar_dev, void *raw_dev, int64_t n, int64_t k, void *stream) {
    if (!raw_dev || !planar_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (!aligned(raw_dev, 2) || !aligned(planar_dev, 256)) return LHIP_ERR_MISALIGNED;
    const size_t n_units = static_cast<size_t>(n) * (k / 32) * 17;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    hipLaunchKernelGGL(q8_unpack_kernel, dim3(grid_for(n_units)), dim3(kThreads), 0, as_stream(stream),
                       reinterpret_cast<const uint16_t *>(base),
                       reinterpret_cast<const uint16_t *>(base + q8_scale_offset(n, k)),
                       static_cast<uint16_t *>(raw_dev), n_units);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_q8_0_interleave_rows(const void *a_planar_dev, const void *b_planar_dev, void *out_planar_dev, int64_t n,
                                      int64_t k, void *stream) {
    if (!a_planar_dev || !b_planar_dev || !out_planar_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (lhip_status s = check_q8_shape(2 * n, k)) return s;
    if (!aligned(a_planar_dev, 256) || !aligned(b_planar_dev, 256) || !aligned(out_planar_dev, 256)) return LHIP_ERR_MISALIGNED;
    auto *a = static_cast<const uint8_t *>(a_planar_dev), *b = static_cast<const uint8_t *>(b_planar_dev);
    auto *o = static_cast<uint8_t *>(out_planar_dev);
    const size_t rows = static_cast<size_t>(2 * n);
    const unsigned pieces_per_row = static_cast<unsigned>(k / 16), scales_per_row = static_cast<unsigned>(k / 32);
    hipLaunchKernelGGL(q8_interleave_rows_kernel, dim3(grid_for(rows * pieces_per_row)), dim3(kThreads), 0, as_stream(stream),
                       reinterpret_cast<const uint4 *>(a), reinterpret_cast<const uint4 *>(b), reinterpret_cast<uint4 *>(o),
                       reinterpret_cast<const uint16_t *>(a + q8_scale_offset(n, k)),
                       reinterpret_cast<const uint16_t *>(b + q8_scale_offset(n, k)),
                       reinterpret_cast<uint16_t *>(o + q8_scale_offset(2 * n, k)), rows * pieces_per_row,
                       rows * scales_per_row, pieces_per_row, scales_per_row);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_q8_0_dequant_f32(const void *planar_dev, float *out_dev, int64_t n, int64_t k, void *stream) {
    if (!planar_dev || !out_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (!aligned(planar_dev, 256) || !aligned(out_dev, 16)) return LHIP_ERR_MISALIGNED;
    const size_t n_quads = static_cast<size_t>(n) * static_cast<size_t>(k) / 4;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    hipLaunchKernelGGL(q8_dequant_kernel, dim3(grid_for(n_quads)), dim3(kThreads), 0, as_stream(stream),
                       reinterpret_cast<const uint32_t *>(base),
                       reinterpret_cast<const __half *>(base + q8_scale_offset(n, k)),
                       reinterpret_cast<float4 *>(out_dev), n_quads);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_q8_0_gather_f32(const void *planar_dev, const float *idx_dev, float *out_dev, int64_t n_idx,
                                 int64_t n, int64_t k, void *stream) {
    if (!planar_dev || !idx_dev || !out_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (n_idx <= 0 || n_idx > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(planar_dev, 256) || !aligned(out_dev, 16) || !aligned(idx_dev, 4)) return LHIP_ERR_MISALIGNED;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    hipLaunchKernelGGL(q8_gather_kernel<float4>, dim3(static_cast<unsigned>(n_idx)), dim3(kThreads), 0, as_stream(stream),
                       reinterpret_cast<const uint32_t *>(base),
                       reinterpret_cast<const __half *>(base + q8_scale_offset(n, k)), idx_dev,
                       reinterpret_cast<float4 *>(out_dev), static_cast<int>(n), static_cast<int>(k));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_q8_0_gather_f16(const void *planar_dev, const float *idx_dev, void *out_f16_dev, int64_t n_idx,
                                 int64_t n, int64_t k, void *stream) {
    if (!planar_dev || !idx_dev || !out_f16_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (n_idx <= 0 || n_idx > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(planar_dev, 256) || !aligned(out_f16_dev, 8) || !aligned(idx_dev, 4)) return LHIP_ERR_MISALIGNED;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    hipLaunchKernelGGL(q8_gather_kernel<Half4>, dim3(static_cast<unsigned>(n_idx)), dim3(kThreads), 0, as_stream(stream),
                       reinterpret_cast<const uint32_t *>(base),
                       reinterpret_cast<const __half *>(base + q8_scale_offset(n, k)), idx_dev,
                       reinterpret_cast<Half4 *>(out_f16_dev), static_cast<int>(n), static_cast<int>(k));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

}  // extern "C"
