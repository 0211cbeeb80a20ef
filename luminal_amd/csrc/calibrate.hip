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

}  // extern "C"
