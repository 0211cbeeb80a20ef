/* Kernel ABI of luminal_hip_kernels.hsaco (gfx950 code object, wave64).
 *
 * Counterpart of the reference's kernel-level interface: one
 *   extern "C" __global__ void kernel(out, weights, inp, ...)
 * per quantized matvec, compiled to a module and looked up by name
 * (crates/luminal_cuda/src/quantized.rs:42-50, crates/luminal_cuda/src/lib.rs:237-258),
 * launched with an explicit LaunchConfig (quantized.rs:131-148).  Here the module is built
 * ahead of time (python -m luminal_amd.build) and holds a small family of kernels; the
 * library function lhip_q8_0_gemv_kernel_plan (luminal_hip.h) picks the member and the
 * launch shape for a weight.  A host needs only hipModuleLoad, hipModuleGetFunction and
 * hipModuleLaunchKernel to run them.
 *
 * What a kernel computes: y[r][j] = sum_i x[r][i] * W[j][i] for r < gridDim.y, j < n, with
 * the arithmetic of the library's matvec (quants as f32, partial sum per half block times
 * float(d), f32 accumulation, fixed reduction order), so the output equals
 * lhip_q8_0_matmul_f32 / _f16 at the same (m, n, k) bit for bit whenever the library takes
 * its matvec route (m below the handful of rows from which it switches to the matrix cores).
 *
 * Arguments (kernarg segment, 40 bytes, natural alignment, no padding; the `args` array
 * of hipModuleLaunchKernel holds pointers to these six values in this order):
 *
 *   offset  size  name  meaning
 *        0     8  qs    const int8_t *   quant plane of the planar weight: the planar buffer
 *                                        itself (256-byte aligned), int8[n][k]
 *        8     8  ds    const uint16_t * scale plane, f16 codes [n][k/32]:
 *                                        planar + lhip_q8_0_planar_scale_offset(n, k)
 *       16     8  x     const T *        activations, T[m][k], 16-byte aligned (f32) / 8-byte (f16)
 *       24     8  y     T *              output, T[m][n]
 *       32     4  n     int32            weight rows (output width), 1 .. 2^30
 *       36     4  k     int32            inner dimension, multiple of 32
 *
 * T is float for the _f32_ kernels and IEEE binary16 for the _f16_ kernels (sums are f32 in
 * both).
 *
 * Launch rules.  block = (W * 64, 1, 1) with W wavefronts as the name says; grid.y = m
 * (1 .. 65535), grid.z = 1.
 *
 *   lhip_kernel_q8_0_gemv_{f32,f16}_oneshot_r{1,2,4}
 *       R rows per wavefront, W = 4.  grid.x = ceil(n / (4 R)), no dynamic LDS.  Any k.
 *
 *   lhip_kernel_q8_0_gemv_{f32,f16}_pipe_r{R}s{S}w{W}   (r1s1w4, r1s2w4, r1s1w16, r1s2w16, r2s4w4)
 *       persistent and software pipelined: R rows x S slices of 1024 quants per step, W
 *       wavefronts per workgroup.  Needs k % (1024 S) == 0 and k <= 16384.  Dynamic LDS =
 *       4 k bytes (the activation row staged as f32).  grid.x = any value from 1 to
 *       ceil(ceil(n / R) / W): every wavefront walks row groups with stride grid.x * W, so the
 *       result does not depend on grid.x; the plan caps it at 256 CUs x the workgroups per
 *       CU that fit (3 for W = 4, 1 for W = 16 and for r2s4w4).
 *
 * The kernels read every weight byte once with non-temporal loads, write y with plain
 * stores, use no atomics and no scratch buffer, and make no assumption about the stream
 * they run on. */
#ifndef LUMINAL_HIP_KERNELS_H
#define LUMINAL_HIP_KERNELS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The kernarg segment as a C struct, for hosts that pass HIP_LAUNCH_PARAM_BUFFER_POINTER
 * instead of an argument array.  T as above. */
typedef struct lhip_q8_0_gemv_kernargs {
    const int8_t *qs;
    const uint16_t *ds;
    const void *x;
    void *y;
    int32_t n;
    int32_t k;
} lhip_q8_0_gemv_kernargs;

#define LHIP_KERNEL_MODULE_FILE "luminal_hip_kernels.hsaco"

/* Symbols of the code object. */
#define LHIP_KERNEL_Q8_0_GEMV_NAMES                                                               \
    "lhip_kernel_q8_0_gemv_f32_oneshot_r1", "lhip_kernel_q8_0_gemv_f32_oneshot_r2",              \
    "lhip_kernel_q8_0_gemv_f32_oneshot_r4", "lhip_kernel_q8_0_gemv_f32_pipe_r1s1w4",             \
    "lhip_kernel_q8_0_gemv_f32_pipe_r1s2w4", "lhip_kernel_q8_0_gemv_f32_pipe_r1s1w16",           \
    "lhip_kernel_q8_0_gemv_f32_pipe_r1s2w16", "lhip_kernel_q8_0_gemv_f32_pipe_r2s4w4",           \
    "lhip_kernel_q8_0_gemv_f16_oneshot_r1", "lhip_kernel_q8_0_gemv_f16_oneshot_r2",              \
    "lhip_kernel_q8_0_gemv_f16_oneshot_r4", "lhip_kernel_q8_0_gemv_f16_pipe_r1s1w4",             \
    "lhip_kernel_q8_0_gemv_f16_pipe_r1s2w4", "lhip_kernel_q8_0_gemv_f16_pipe_r1s1w16",           \
    "lhip_kernel_q8_0_gemv_f16_pipe_r1s2w16", "lhip_kernel_q8_0_gemv_f16_pipe_r2s4w4"

#ifdef __cplusplus
}
#endif

#endif /* LUMINAL_HIP_KERNELS_H */
