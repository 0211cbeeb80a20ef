// Shared internals of the luminal_hip library: status plumbing, argument
// checks, and the planar Q8_0 layout arithmetic.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

#include "../../include/luminal_hip.h"

namespace lhip {

// Records the failing hipError_t for lhip_last_hip_error().
lhip_status hip_failed(hipError_t e);

#define LHIP_HIP_TRY(expr)                                        \
    do {                                                          \
        hipError_t _e = (expr);                                   \
        if (_e != hipSuccess) return ::lhip::hip_failed(_e);      \
    } while (0)

// Kernel launches report configuration errors through hipGetLastError.
#define LHIP_CHECK_LAUNCH() LHIP_HIP_TRY(hipGetLastError())

// Kernels that use more than 64 KiB of dynamic LDS have to be told so once (per device); remembered here so that a
// launch costs no hipFuncSetAttribute call after the first.  One object per kernel (a function-local static of its
// launcher).
struct LdsOptIn {
    size_t bytes[64] = {};  // largest size set so far, per device
};
static inline lhip_status lds_opt_in(LdsOptIn &st, const void *kernel, size_t lds_bytes, bool needed) {
    if (!needed) return LHIP_OK;
    int dev = 0;
    LHIP_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return LHIP_ERR_UNSUPPORTED;
    if (__atomic_load_n(&st.bytes[dev], __ATOMIC_RELAXED) >= lds_bytes) return LHIP_OK;
    LHIP_HIP_TRY(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    __atomic_store_n(&st.bytes[dev], lds_bytes, __ATOMIC_RELAXED);
    return LHIP_OK;
}

static inline lhip_status lds_opt_in(LdsOptIn &st, const void *kernel, size_t lds_bytes) {
    return lds_opt_in(st, kernel, lds_bytes, lds_bytes > 64 * 1024);
}

static inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

static inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

// Largest dimension accepted: keeps every int32 index computed in the kernels
// (rows, columns, blocks per row) in range.
constexpr int64_t kMaxDim = (int64_t{1} << 30);

static inline lhip_status check_q8_shape(int64_t n, int64_t k) {
    if (n <= 0 || k <= 0 || n > kMaxDim || k > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
    if (k % 32 != 0) return LHIP_ERR_INVALID_SHAPE;
    return LHIP_OK;
}

// Planar Q8_0: [int8 qs[N][K]] padded to 256 B, then [f16 d[N][K/32]].
static inline size_t q8_scale_offset(int64_t n, int64_t k) {
    size_t q = static_cast<size_t>(n) * static_cast<size_t>(k);
    return (q + 255) & ~size_t{255};
}
static inline size_t q8_planar_nbytes(int64_t n, int64_t k) {
    return q8_scale_offset(n, k) + static_cast<size_t>(n) * static_cast<size_t>(k / 32) * 2;
}

// Planar MXFP4, tiled for the block-scaled MFMA: rows are grouped into panels of
// 16 and K into chunks of 128 (both padded with zero weights / scale 2^0).  Tile
// (panel, chunk) is 1 KiB of nibble bytes: 64 pieces of 16 bytes, piece g*16 + r
// holding block (chunk*4 + g) of row (panel*16 + r) — the order in which the 64
// lanes of a wavefront consume them, so one wave load is one contiguous KiB.
// The scale plane has the same order, one byte per piece.
static inline int64_t mx_panels(int64_t n) { return (n + 15) / 16; }
static inline int64_t mx_chunks(int64_t k) { return (k + 127) / 128; }
static inline size_t mx_scale_offset(int64_t n, int64_t k) {
    return static_cast<size_t>(mx_panels(n)) * static_cast<size_t>(mx_chunks(k)) * 1024;
}
static inline size_t mx_planar_nbytes(int64_t n, int64_t k) {
    return mx_scale_offset(n, k) + static_cast<size_t>(mx_panels(n)) * static_cast<size_t>(mx_chunks(k)) * 64;
}
// up * swish(gate) in f32 (examples/llama/src/model.rs:24-32, src/hl_ops/unary.rs:169-177): one definition, so the
// element-wise kernel and the GEMM epilogue give the same bits.
__device__ __forceinline__ float swiglu_value(float gate, float up) { return up * (gate * (1.0f / (1.0f + expf(-gate)))); }

// Piece index (in units of 16 nibble bytes / 1 scale byte) of block kb of row.
__host__ __device__ static inline size_t mx_piece(int64_t row, int64_t kb, int64_t chunks) {
    return (static_cast<size_t>(row >> 4) * chunks + (kb >> 2)) * 64 + (kb & 3) * 16 + (row & 15);
}

}  // namespace lhip
