// Calibration kernels: a plain copy and a read-only pass of known size.
// Both move 16 bytes per lane per load with a grid-stride loop; they exist to
// scale hardware byte counters and to find the streaming rate of the part.
#include "common.h"

namespace lhip {

typedef uint32_t cu32x4 __attribute__((ext_vector_type(4)));
constexpr unsigned kReadSlots = 1024;  // out_dev of lhip_read_bytes holds this many words

__global__ __launch_bounds__(256) void copy_kernel(cu32x4 *__restrict__ dst, const cu32x4 *__restrict__ src,
                                                   size_t n16) {
    size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    for (; i < n16; i += stride) dst[i] = __builtin_nontemporal_load(src + i);
}

__global__ __launch_bounds__(256) void read_kernel(const cu32x4 *__restrict__ src, size_t n16,
                                                   uint32_t *__restrict__ out) {
    size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t stride = static_cast<size_t>(gridDim.x) * 256;
    cu32x4 a = {0, 0, 0, 0};
    // four independent loads in flight per lane
    for (; i + 3 * stride < n16; i += 4 * stride) {
        cu32x4 v0 = __builtin_nontemporal_load(src + i);
        cu32x4 v1 = __builtin_nontemporal_load(src + i + stride);
        cu32x4 v2 = __builtin_nontemporal_load(src + i + 2 * stride);
        cu32x4 v3 = __builtin_nontemporal_load(src + i + 3 * stride);
        a ^= v0 ^ v1 ^ v2 ^ v3;
    }
    for (; i < n16; i += stride) a ^= __builtin_nontemporal_load(src + i);
    uint32_t x = a.x ^ a.y ^ a.z ^ a.w;
    for (int o = 32; o > 0; o >>= 1) x ^= __shfl_xor(x, o);
    // one plain store per wavefront into a slot of its own (no atomics: they
    // would serialise on one address and dominate the timing)
    if ((threadIdx.x & 63) == 0) out[(blockIdx.x * 4 + (threadIdx.x >> 6)) & (kReadSlots - 1)] = x;
}

// ---------------------------------------------------------------------------
// Issue-rate probes: a register-only loop of one instruction kind, eight independent accumulators (or results) per
// wave so that nothing waits on a dependency; lane 0 of every wave leaves the shader-clock cycles and the 100 MHz
// wall-clock ticks its loop took.  They back the matrix-pipe ceilings that the roofline figures are priced against.
// ---------------------------------------------------------------------------
typedef int rv8i __attribute__((ext_vector_type(8)));
typedef float rv4f __attribute__((ext_vector_type(4)));
typedef float rv16f __attribute__((ext_vector_type(16)));
typedef __bf16 rv8bf __attribute__((ext_vector_type(8)));
typedef __bf16 rv2bf __attribute__((ext_vector_type(2)));
constexpr int kRateAcc = 8;

__device__ __forceinline__ void rate_leave(uint64_t *out, uint64_t c0, uint64_t w0, float keep) {
    const uint64_t c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
    if ((threadIdx.x & 63) == 0) {
        uint64_t *o = out + 2 * (static_cast<size_t>(blockIdx.x) * (blockDim.x >> 6) + (threadIdx.x >> 6));
        o[0] = c1 - c0;
        o[1] = w1 - w0;
    }
    if (keep == 1.2345e-30f) out[0] = 0;  // keeps the loop's results alive
}

// The loops are written as inline assembly, one instruction per accumulator and nothing else: with the builtins the
// register allocator rotated the accumulators of some operand widths through VGPRs on every trip (thirty register
// moves per eight instructions), and the loop measured those.
typedef int rv4i __attribute__((ext_vector_type(4)));
typedef int rv6i __attribute__((ext_vector_type(6)));

template <int FA, int FB>  // operand formats of v_mfma_scale_f32_16x16x128_f8f6f4: 0 = fp8 (e4m3), 2 = fp6 (e2m3), 4 = fp4 (e2m1)
__global__ __launch_bounds__(256) void rate_scaled_kernel(uint64_t *out, int iters) {
    static_assert((FA == 0 || FA == 2 || FA == 4) && (FB == 0 || FB == 4), "formats");
    rv8i a8, b8;
    for (int i = 0; i < 8; ++i) {
        a8[i] = 0x3c3c3c3c + static_cast<int>(threadIdx.x) * (i + 1);
        b8[i] = 0x22222222 + static_cast<int>(threadIdx.x) * (3 * i + 1);
    }
    const rv6i a6 = {a8[0], a8[1], a8[2], a8[3], a8[4], a8[5]};
    const rv4i a4 = {a8[0], a8[1], a8[2], a8[3]}, b4 = {b8[0], b8[1], b8[2], b8[3]};
    const int sc = 127;
    rv4f acc[kRateAcc];
    for (int j = 0; j < kRateAcc; ++j) acc[j] = rv4f{0, 0, 0, 0};
    const uint64_t c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < kRateAcc; ++j) {
            if constexpr (FA == 0 && FB == 0)
                asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0]"
                             : "+a"(acc[j]) : "v"(a8), "v"(b8), "v"(sc));
            else if constexpr (FA == 0 && FB == 4)
                asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0] blgp:4"
                             : "+a"(acc[j]) : "v"(a8), "v"(b4), "v"(sc));
            else if constexpr (FA == 4 && FB == 4)
                asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0] cbsz:4 blgp:4"
                             : "+a"(acc[j]) : "v"(a4), "v"(b4), "v"(sc));
            else
                asm volatile("v_mfma_scale_f32_16x16x128_f8f6f4 %0, %1, %2, %0, %3, %3 op_sel_hi:[0,0,0] cbsz:2 blgp:4"
                             : "+a"(acc[j]) : "v"(a6), "v"(b4), "v"(sc));
        }
    }
    float s = 0;
    for (int j = 0; j < kRateAcc; ++j) s += acc[j][0] + acc[j][3];
    rate_leave(out, c0, w0, s);
}

template <bool WIDE>  // true: v_mfma_f32_32x32x16_bf16, false: v_mfma_f32_16x16x32_bf16
__global__ __launch_bounds__(256) void rate_bf16_kernel(uint64_t *out, int iters) {
    rv8bf a, b;
    for (int i = 0; i < 8; ++i) {
        a[i] = static_cast<__bf16>(static_cast<float>((threadIdx.x + i) & 3));
        b[i] = static_cast<__bf16>(static_cast<float>(i & 1));
    }
    const uint64_t c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    float s = 0;
    if constexpr (WIDE) {
        rv16f acc[kRateAcc / 2];
        for (int j = 0; j < kRateAcc / 2; ++j)
            for (int q = 0; q < 16; ++q) acc[j][q] = 0;
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < kRateAcc / 2; ++j)
                asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(acc[j]) : "v"(a), "v"(b));
        }
        for (int j = 0; j < kRateAcc / 2; ++j) s += acc[j][0] + acc[j][5];
    } else {
        rv4f acc[kRateAcc];
        for (int j = 0; j < kRateAcc; ++j) acc[j] = rv4f{0, 0, 0, 0};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < kRateAcc; ++j)
                asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[j]) : "v"(a), "v"(b));
        }
        for (int j = 0; j < kRateAcc; ++j) s += acc[j][0] + acc[j][3];
    }
    rate_leave(out, c0, w0, s);
}

// v_cvt_scalef32_pk_bf16_fp4: the expansion of two MXFP4 codes to a bf16 pair (the exact expert GEMMs' weight path).
__global__ __launch_bounds__(256) void rate_cvt_fp4_kernel(uint64_t *out, int iters) {
    uint32_t q[kRateAcc];
    for (int j = 0; j < kRateAcc; ++j) q[j] = 0x12345678u * (threadIdx.x + j + 1);
    const float scale = __uint_as_float((120u + (threadIdx.x & 7u)) << 23);
    const uint64_t c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
    uint32_t x = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < kRateAcc; ++j) {
            const rv2bf p = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[j], scale, 0);
            q[j] ^= __builtin_bit_cast(uint32_t, p);  // the next conversion of slot j depends on this one only
        }
    }
    for (int j = 0; j < kRateAcc; ++j) x ^= q[j];
    rate_leave(out, c0, w0, x == 0x9e3779b9u ? 1.2345e-30f : 0.f);
}

}  // namespace lhip

using namespace lhip;

extern "C" {

lhip_status lhip_copy_bytes(void *dst_dev, const void *src_dev, size_t nbytes, void *stream) {
    if (!dst_dev || !src_dev) return LHIP_ERR_NULL_PTR;
    if (nbytes == 0 || nbytes % 16 != 0) return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(dst_dev, 16) || !aligned(src_dev, 16)) return LHIP_ERR_MISALIGNED;
    const size_t n16 = nbytes / 16;
    size_t grid = (n16 + 255) / 256;
    if (grid > 256u * 32u) grid = 256u * 32u;
    hipLaunchKernelGGL(copy_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, as_stream(stream),
                       static_cast<cu32x4 *>(dst_dev), static_cast<const cu32x4 *>(src_dev), n16);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_read_bytes(const void *src_dev, size_t nbytes, uint32_t *out_dev, void *stream) {
    if (!src_dev || !out_dev) return LHIP_ERR_NULL_PTR;
    if (nbytes == 0 || nbytes % 16 != 0) return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(src_dev, 16) || !aligned(out_dev, 4)) return LHIP_ERR_MISALIGNED;
    const size_t n16 = nbytes / 16;
    size_t grid = (n16 + 1023) / 1024;
    if (grid == 0) grid = 1;
    if (grid > 256u * 16u) grid = 256u * 16u;
    hipLaunchKernelGGL(read_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0, as_stream(stream),
                       static_cast<const cu32x4 *>(src_dev), n16, out_dev);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status lhip_issue_rate_probe(int32_t kind, int32_t iters, int32_t waves_per_simd, uint64_t *out_dev, void *stream) {
    if (!out_dev) return LHIP_ERR_NULL_PTR;
    if (iters <= 0 || waves_per_simd < 1 || waves_per_simd > 8) return LHIP_ERR_INVALID_SHAPE;
    if (!aligned(out_dev, 8)) return LHIP_ERR_MISALIGNED;
    const dim3 grid(static_cast<unsigned>(256 * waves_per_simd)), block(256);  // a workgroup is one wave per SIMD of a CU
    hipStream_t s = as_stream(stream);
    switch (kind) {
        case LHIP_RATE_MFMA_BF16_32X32X16: hipLaunchKernelGGL(rate_bf16_kernel<true>, grid, block, 0, s, out_dev, iters); break;
        case LHIP_RATE_MFMA_BF16_16X16X32: hipLaunchKernelGGL(rate_bf16_kernel<false>, grid, block, 0, s, out_dev, iters); break;
        case LHIP_RATE_MFMA_SCALE_FP8_FP8: hipLaunchKernelGGL((rate_scaled_kernel<0, 0>), grid, block, 0, s, out_dev, iters); break;
        case LHIP_RATE_MFMA_SCALE_FP8_FP4: hipLaunchKernelGGL((rate_scaled_kernel<0, 4>), grid, block, 0, s, out_dev, iters); break;
        case LHIP_RATE_MFMA_SCALE_FP4_FP4: hipLaunchKernelGGL((rate_scaled_kernel<4, 4>), grid, block, 0, s, out_dev, iters); break;
        case LHIP_RATE_MFMA_SCALE_FP6_FP4: hipLaunchKernelGGL((rate_scaled_kernel<2, 4>), grid, block, 0, s, out_dev, iters); break;
        case LHIP_RATE_CVT_BF16_FP4: hipLaunchKernelGGL(rate_cvt_fp4_kernel, grid, block, 0, s, out_dev, iters); break;
        default: return LHIP_ERR_INVALID_SHAPE;
    }
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

}  // extern "C"
