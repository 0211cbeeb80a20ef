// MXFP4 storage kernels: raw blocks <-> planar, exact dequantisation to f32.
//
// MXFP4 is not in the reference (no e2m1/e8m0 anywhere in its tree); the
// convention follows its Q8_0 path (examples/llama/src/loader.rs:227-241):
// dequantise exactly to f32, then matmul.  Format (OCP Microscaling, as in
// gpt-oss checkpoints): a block is 32 e2m1 values, two per byte with the even
// element in the low nibble, followed by one e8m0 scale byte (2^(e-127), 0xff =
// NaN): 17 bytes per 32 weights.
//
// Planar form used by the kernels: a nibble plane tiled in the order the
// block-scaled MFMA consumes it (panels of 16 rows x chunks of 128 columns, see
// mx_piece in common.h), then a scale plane in the same order.  Rows are padded
// to a multiple of 16 and K to a multiple of 128 with zero weights and scale 2^0.
#include "common.h"

namespace lhip {

constexpr int kLayoutThreads = 256;

// Padding pieces: zero nibbles, scale 127 (2^0).  One thread per piece.
__global__ __launch_bounds__(kLayoutThreads) void mx_fill_kernel(uint4 *__restrict__ nib, uint8_t *__restrict__ sc,
                                                                 size_t n_pieces) {
    size_t i = static_cast<size_t>(blockIdx.x) * kLayoutThreads + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * kLayoutThreads;
    for (; i < n_pieces; i += stride) {
        nib[i] = make_uint4(0, 0, 0, 0);
        sc[i] = 127;
    }
}

// One thread per raw byte: byte b of the stream lies in block b/17; b%17 == 16 is the scale.
__global__ __launch_bounds__(kLayoutThreads) void mx_repack_kernel(const uint8_t *__restrict__ raw,
                                                                   uint8_t *__restrict__ nib,
                                                                   uint8_t *__restrict__ sc, size_t n_bytes,
                                                                   int blocks_per_row, int chunks) {
    size_t b = static_cast<size_t>(blockIdx.x) * kLayoutThreads + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * kLayoutThreads;
    for (; b < n_bytes; b += stride) {
        const size_t blk = b / 17;
        const unsigned off = static_cast<unsigned>(b - blk * 17);
        const size_t row = blk / blocks_per_row;
        const size_t piece = mx_piece(row, blk - row * blocks_per_row, chunks);
        const uint8_t v = raw[b];
        if (off == 16)
            sc[piece] = v;
        else
            nib[piece * 16 + off] = v;
    }
}

__global__ __launch_bounds__(kLayoutThreads) void mx_unpack_kernel(const uint8_t *__restrict__ nib,
                                                                   const uint8_t *__restrict__ sc,
                                                                   uint8_t *__restrict__ raw, size_t n_bytes,
                                                                   int blocks_per_row, int chunks) {
    size_t b = static_cast<size_t>(blockIdx.x) * kLayoutThreads + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * kLayoutThreads;
    for (; b < n_bytes; b += stride) {
        const size_t blk = b / 17;
        const unsigned off = static_cast<unsigned>(b - blk * 17);
        const size_t row = blk / blocks_per_row;
        const size_t piece = mx_piece(row, blk - row * blocks_per_row, chunks);
        raw[b] = (off == 16) ? sc[piece] : nib[piece * 16 + off];
    }
}

// e2m1 code -> f32: sign, 2 exponent bits, 1 mantissa bit; exponent 0 is subnormal (0 or 0.5).
__device__ __forceinline__ float e2m1_to_f32(unsigned c) {
    const unsigned m = c & 7u;
    // magnitudes 0, .5, 1, 1.5, 2, 3, 4, 6
    float v = (m < 2u) ? 0.5f * static_cast<float>(m)
                       : __uint_as_float(((126u + (m >> 1)) << 23) | ((m & 1u) << 22));
    return (c & 8u) ? -v : v;
}

// e8m0 -> f32: 2^(e-127); e = 0 is the f32 subnormal 2^-127, e = 255 is NaN.
__device__ __forceinline__ float e8m0_to_f32(unsigned e) {
    if (e == 255u) return __uint_as_float(0x7fc00000u);
    if (e == 0u) return __uint_as_float(0x00400000u);
    return __uint_as_float(e << 23);
}

// One thread per nibble byte of the row-major result: two weights.
__global__ __launch_bounds__(kLayoutThreads) void mx_dequant_kernel(const uint8_t *__restrict__ nib,
                                                                    const uint8_t *__restrict__ sc,
                                                                    float2 *__restrict__ out, size_t n_pairs,
                                                                    int blocks_per_row, int chunks) {
    size_t i = static_cast<size_t>(blockIdx.x) * kLayoutThreads + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * kLayoutThreads;
    for (; i < n_pairs; i += stride) {
        const size_t blk = i >> 4;
        const size_t row = blk / blocks_per_row;
        const size_t piece = mx_piece(row, blk - row * blocks_per_row, chunks);
        const unsigned b = nib[piece * 16 + (i & 15)];
        const float s = e8m0_to_f32(sc[piece]);
        out[i] = make_float2(e2m1_to_f32(b & 15u) * s, e2m1_to_f32(b >> 4) * s);
    }
}

static inline unsigned layout_grid(size_t items) {
    size_t g = (items + kLayoutThreads - 1) / kLayoutThreads;
    const size_t cap = 256u * 64u;
    return static_cast<unsigned>(g < cap ? (g ? g : 1) : cap);
}

}  // namespace lhip

using namespace lhip;

extern "C" {

size_t lhip_mxfp4_raw_nbytes(int64_t n, int64_t k) {
    if (check_q8_shape(n, k) != LHIP_OK) return 0;
    return static_cast<size_t>(n) * static_cast<size_t>(k / 32) * 17;
}

size_t lhip_mxfp4_planar_nbytes(int64_t n, int64_t k) {
    if (check_q8_shape(n, k) != LHIP_OK) return 0;
    return mx_planar_nbytes(n, k);
}

size_t lhip_mxfp4_planar_scale_offset(int64_t n, int64_t k) {
    if (check_q8_shape(n, k) != LHIP_OK) return 0;
    return mx_scale_offset(n, k);
}

lhip_status lhip_mxfp4_repack(const void *raw_dev, void *planar_dev, int64_t n, int64_t k, void *stream) {
    if (!raw_dev || !planar_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (!aligned(planar_dev, 256)) return LHIP_ERR_MISALIGNED;
    const size_t n_bytes = static_cast<size_t>(n) * (k / 32) * 17;
    auto *base = static_cast<uint8_t *>(planar_dev);
    const size_t n_pieces = mx_scale_offset(n, k) / 16;
    if (n % 16 != 0 || k % 128 != 0) {  // padding pieces exist: give them zero weights and scale 2^0 first
        hipLaunchKernelGGL(mx_fill_kernel, dim3(layout_grid(n_pieces)), dim3(kLayoutThreads), 0, as_stream(stream),
                           reinterpret_cast<uint4 *>(base), base + mx_scale_offset(n, k), n_pieces);
        LHIP_CHECK_LAUNCH();
    }
    hipLaunchKernelGGL(mx_repack_kernel, dim3(layout_grid(n_bytes)), dim3(kLayoutThreads), 0, as_stream(stream),
                       static_cast<const uint8_t *>(raw_dev), base, base + mx_scale_offset(n, k), n_bytes,
                       static_cast<int>(k / 32), static_cast<int>(mx_chunks(k)));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_mxfp4_unpack(const void *planar_dev, void *raw_dev, int64_t n, int64_t k, void *stream) {
    if (!raw_dev || !planar_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (!aligned(planar_dev, 256)) return LHIP_ERR_MISALIGNED;
    const size_t n_bytes = static_cast<size_t>(n) * (k / 32) * 17;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    hipLaunchKernelGGL(mx_unpack_kernel, dim3(layout_grid(n_bytes)), dim3(kLayoutThreads), 0, as_stream(stream), base,
                       base + mx_scale_offset(n, k), static_cast<uint8_t *>(raw_dev), n_bytes,
                       static_cast<int>(k / 32), static_cast<int>(mx_chunks(k)));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_mxfp4_dequant_f32(const void *planar_dev, float *out_dev, int64_t n, int64_t k, void *stream) {
    if (!planar_dev || !out_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (!aligned(planar_dev, 256) || !aligned(out_dev, 8)) return LHIP_ERR_MISALIGNED;
    const size_t n_pairs = static_cast<size_t>(n) * static_cast<size_t>(k) / 2;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    hipLaunchKernelGGL(mx_dequant_kernel, dim3(layout_grid(n_pairs)), dim3(kLayoutThreads), 0, as_stream(stream), base,
                       base + mx_scale_offset(n, k), reinterpret_cast<float2 *>(out_dev), n_pairs,
                       static_cast<int>(k / 32), static_cast<int>(mx_chunks(k)));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

}  // extern "C"
