// Code-object build of the Q8_0 matrix-vector kernels: the same device code the library launches
// (q8_gemv_device.h), exported under C names so a host that owns its own HIP context can run them with
// hipModuleLoad / hipModuleGetFunction / hipModuleLaunchKernel and nothing else.  This is the shape of the
// reference's kernel interface, `extern "C" __global__ void kernel(...)` found by name in a loaded module
// (crates/luminal_cuda/src/quantized.rs:42-50, crates/luminal_cuda/src/lib.rs:237-258), with two differences:
// the code object is built ahead of time instead of per weight node, and the launch shape is not baked in.
//
// Compiled with `hipcc --genco --offload-arch=gfx950` into luminal_hip_kernels.hsaco; argument layout, grid and
// alignment rules are stated in include/luminal_hip_kernels.h.
#include "../q8_gemv_device.h"

using namespace lhip;

// One-shot kernel: any K that is a multiple of 32.  R rows per wavefront, 4 wavefronts per workgroup.
#define LHIP_ONESHOT(R)                                                                                             \
    extern "C" __global__ __launch_bounds__(256) void lhip_kernel_q8_0_gemv_f32_oneshot_r##R(                       \
        const int8_t *qs, const uint16_t *ds, const float *x, float *y, int n, int k) {                            \
        q8_gemv_oneshot_body<R, 4, 1, float>(qs, reinterpret_cast<const __half *>(ds), x, y, n, k);                 \
    }                                                                                                               \
    extern "C" __global__ __launch_bounds__(256) void lhip_kernel_q8_0_gemv_f16_oneshot_r##R(                       \
        const int8_t *qs, const uint16_t *ds, const __half *x, __half *y, int n, int k) {                          \
        q8_gemv_oneshot_body<R, 4, 1, __half>(qs, reinterpret_cast<const __half *>(ds), x, y, n, k);                \
    }

// Persistent pipelined kernel: K a multiple of S * 1024 and at most 16384; K * 4 bytes of dynamic LDS.
#define LHIP_PIPE(R, S, W)                                                                                          \
    extern "C" __global__ __launch_bounds__(W * 64) void lhip_kernel_q8_0_gemv_f32_pipe_r##R##s##S##w##W(           \
        const int8_t *qs, const uint16_t *ds, const float *x, float *y, int n, int k) {                            \
        q8_gemv_pipe_body<R, S, W, float>(qs, ds, x, y, n, k);                                                      \
    }                                                                                                               \
    extern "C" __global__ __launch_bounds__(W * 64) void lhip_kernel_q8_0_gemv_f16_pipe_r##R##s##S##w##W(           \
        const int8_t *qs, const uint16_t *ds, const __half *x, __half *y, int n, int k) {                          \
        q8_gemv_pipe_body<R, S, W, __half>(qs, ds, x, y, n, k);                                                     \
    }

LHIP_ONESHOT(1)
LHIP_ONESHOT(2)
LHIP_ONESHOT(4)
LHIP_PIPE(1, 1, 4)
LHIP_PIPE(1, 2, 4)
LHIP_PIPE(1, 1, 16)
LHIP_PIPE(1, 2, 16)
LHIP_PIPE(2, 4, 4)
