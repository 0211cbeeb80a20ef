/*
 * luminal_hip — C ABI of the MI355X (gfx950) quantized-matmul backend.
 *
 * This is the surface a `luminal_hip` Rust crate binds with `extern "C"`:
 * plain pointers and sizes, no C++ or framework types.  Every device pointer
 * is an ordinary HIP allocation (hipMalloc, or lhip_malloc below); `stream`
 * is a hipStream_t passed as void* (NULL = the default stream).  All launches
 * are asynchronous on `stream`; nothing here synchronises except
 * lhip_stream_sync and the two blocking copies.  The caller owns every buffer
 * and the library never frees or keeps one.
 *
 * Where the reference panics (unwrap/assert!/panic!), these functions return
 * a status instead; a Rust wrapper turns non-zero into panic! to keep the
 * reference's behaviour.
 *
 * Reference files cited below are relative to the luminal source tree.
 */
#ifndef LUMINAL_HIP_H
#define LUMINAL_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int32_t lhip_status;
enum {
    LHIP_OK = 0,
    LHIP_ERR_NULL_PTR = 1,      /* a required pointer argument is NULL */
    LHIP_ERR_INVALID_SHAPE = 2, /* zero dim, K % 32 != 0, dim too large ... */
    LHIP_ERR_MISALIGNED = 3,    /* a device pointer misses its required alignment */
    LHIP_ERR_HIP = 4,           /* a HIP runtime call failed: see lhip_last_hip_error */
    LHIP_ERR_UNSUPPORTED = 5    /* valid arguments, but no kernel for this case */
};

/* Human-readable name of a status code (static storage). */
const char *lhip_status_string(lhip_status s);
/* hipError_t of the most recent LHIP_ERR_HIP on this thread (0 if none). */
int lhip_last_hip_error(void);
/* Library version, "major.minor.patch". */
const char *lhip_version(void);

/* ---- device plumbing ------------------------------------------------------
 * Counterparts of what luminal_cuda takes from cudarc: CudaContext::new(0)
 * (crates/luminal_cuda/src/quantized.rs:247), stream.alloc / memcpy_stod /
 * memcpy_dtov (quantized.rs:144, examples/llama/src/loader.rs:157,
 * crates/luminal_cuda/src/prim.rs:60-75). */
lhip_status lhip_init(int device);
lhip_status lhip_malloc(void **dptr, size_t nbytes);
lhip_status lhip_free(void *dptr);
lhip_status lhip_memcpy_h2d(void *dst_dev, const void *src_host, size_t nbytes, void *stream);
lhip_status lhip_memcpy_d2h(void *dst_host, const void *src_dev, size_t nbytes, void *stream);
lhip_status lhip_stream_sync(void *stream);

/* ---- Q8_0 weight storage ---------------------------------------------------
 * A weight (N, K) arrives as raw GGUF Q8_0 blocks: N*K/32 blocks of 34 bytes
 * {f16 d; int8 qs[32]}, row-major, N*K + N*K/16 bytes — exactly the bytes the
 * reference's loader copies to the device
 * (examples/llama/src/loader.rs:124-130,156-158; block struct
 * crates/luminal_cuda/src/quantized.rs:30-33).
 *
 * The kernels read a "planar" re-arrangement of the same bytes made once at
 * load: all quants first (int8[N][K], so every 16-byte load is aligned), then
 * all scales (f16[N][K/32]).  Same byte count apart from padding the quant
 * plane to 256 B.  K % 32 == 0 is required (as in the reference, which
 * computes K/32 blocks per row, quantized.rs:58). */

/* Bytes of the raw GGUF form: N*K + N*K/16. */
size_t lhip_q8_0_raw_nbytes(int64_t n, int64_t k);
/* Bytes of the planar form (what to allocate for `planar`). */
size_t lhip_q8_0_planar_nbytes(int64_t n, int64_t k);
/* Byte offset of the scale plane inside the planar buffer. */
size_t lhip_q8_0_planar_scale_offset(int64_t n, int64_t k);
/* raw (device) -> planar (device).  `planar` must be 256-byte aligned, `raw`
 * 2-byte aligned.  The buffers must not overlap. */
lhip_status lhip_q8_0_repack(const void *raw_dev, void *planar_dev, int64_t n, int64_t k, void *stream);
/* planar (device) -> raw (device): inverse of lhip_q8_0_repack. */
lhip_status lhip_q8_0_unpack(const void *planar_dev, void *raw_dev, int64_t n, int64_t k, void *stream);
/* Two planar (n, k) weights -> one planar (2n, k) weight with their rows taken alternately (row 2j = a's row j,
 * row 2j + 1 = b's row j): the (gate, up) row order that epilogue 2 of lhip_q8_0_matvec_fused_f32 and
 * lhip_q8_0_matmul_bf16_swiglu read.  No counterpart in the reference, which keeps gate and up as separate tensors
 * (examples/llama/src/model.rs:17-32); a compiler pass that fuses the two projections makes this weight once.
 * All three buffers 256-byte aligned, out_planar_dev of lhip_q8_0_planar_nbytes(2n, k) bytes, no overlap. */
lhip_status lhip_q8_0_interleave_rows(const void *a_planar_dev, const void *b_planar_dev, void *out_planar_dev, int64_t n,
                                      int64_t k, void *stream);

/* ---- Q8_0 operators --------------------------------------------------------
 */

/* Dequantise a planar weight to f32[N][K]: w = (float)q * (float)d, exact.
 * Restates the reference's CPU loader (examples/llama/src/loader.rs:227-241). */
lhip_status lhip_q8_0_dequant_f32(const void *planar_dev, float *out_dev, int64_t n, int64_t k, void *stream);

/* y[m][n] = sum_k x[m][k] * W[n][k], f32 activations, f32 accumulate, f32 out.
 * Replaces QuantizedMatmul<f32>::process + its matvec kernel
 * (crates/luminal_cuda/src/quantized.rs:42-109,116-168): x is (m, K) row-major
 * with m = batch*m of the reference's launch (grid z, quantized.rs:159), y is
 * (m, N).  x and y must be 16-byte aligned. */
lhip_status lhip_q8_0_matmul_f32(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                 int64_t k, void *stream);

/* The same operator for several activation rows on the matrix cores.  The reference's launch (quantized.rs:159) is
 * one matvec per activation row, i.e. the weights are streamed once per row; this form streams them once per 64
 * rows.  The int8 codes go to the matrix cores as they are (exact in bf16), x as three bf16 limbs (an f16 x as
 * two) whose sum is the value exactly; per Q8_0 block the limb products are summed in f32 and the block's scale is applied to that
 * sum, as the matvec kernels do.  Every product is exact, so the result differs from the matvec form only by the
 * order of the f32 additions (measured 5e-7 to 9e-7 of the rms for both), and products of small integers stay
 * exact.  The f16 form is the f32 form on the widened inputs, rounded once.  Any m >= 1.
 * LHIP_ERR_UNSUPPORTED unless K % 512 == 0, N % 4 == 0, x 16-byte and y 16-byte (f16: 8-byte) aligned.
 * lhip_q8_0_matmul_f32 and lhip_q8_0_matmul_f16 take this form by themselves from a few rows on (two for N*K >=
 * 2^28 codes, three from 2^25, four from 2^23, six below: the measured crossovers with the matvec form) where those
 * conditions hold (the _cfg entry never does).  May keep partial sums in the library's scratch array, see the
 * note on overlapping calls at lhip_q8_0_matmul_bf16. */
lhip_status lhip_q8_0_matmul_f32_gemm(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                      int64_t k, void *stream);
lhip_status lhip_q8_0_matmul_f16_gemm(const void *planar_dev, const void *x_f16_dev, void *y_f16_dev, int64_t m,
                                      int64_t n, int64_t k, void *stream);

/* Same operator with the launch shape given by the caller instead of chosen by
 * the library (for tuning and for tests that cover every shape).
 * blocks_per_cu in 1..16 runs the persistent pipelined kernel with that many
 * resident workgroups of waves_per_block (4, 8 or 16) wavefronts per compute
 * unit (rows_per_wave in {1,2,4}, k_unroll = 1024-quant slices per pipeline
 * step in {1,2,4}, K <= 16384 and a multiple of k_unroll*1024);
 * blocks_per_cu == 0 runs the one-shot kernel (rows_per_wave in {1,2,4,8},
 * k_unroll in {1,2,4}, any K; waves_per_block ignored).  LHIP_ERR_UNSUPPORTED
 * for a combination that is not built. */
lhip_status lhip_q8_0_matmul_f32_cfg(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                     int64_t k, int rows_per_wave, int k_unroll, int blocks_per_cu,
                                     int waves_per_block, void *stream);

/* Kernel-level route to the same matvec, for a host that launches kernels itself the way
 * the reference does (module loaded once, function found by name, launched with explicit
 * grid / block / arguments: crates/luminal_cuda/src/lib.rs:237-258,
 * crates/luminal_cuda/src/quantized.rs:42-50,131-148).  luminal_hip_kernels.hsaco holds the
 * matvec kernels under C names (include/luminal_hip_kernels.h states their arguments).
 * This call names the kernel and launch shape lhip_q8_0_matmul_f32 / _f16 would use for
 * an (n, k) weight at few activation rows, so that
 *   hipModuleLoad(&mod, ".../luminal_hip_kernels.hsaco");
 *   hipModuleGetFunction(&fn, mod, kernel_name);
 *   grid[1] = m;   // activation rows, 1..65535
 *   hipModuleLaunchKernel(fn, grid[0], grid[1], grid[2], block[0], block[1], block[2],
 *                         lds_bytes, stream, args, NULL);
 * gives the bits of the library call.  It touches no device.  f16 != 0 selects the f16
 * activation type.  kernel_name receives a NUL-terminated string (64 bytes are enough). */
lhip_status lhip_q8_0_gemv_kernel_plan(int64_t n, int64_t k, int f16, char *kernel_name, size_t kernel_name_cap,
                                       uint32_t grid[3], uint32_t block[3], uint32_t *lds_bytes);

/* Batch-1 decode matvec with fusions.  No counterpart in the reference, whose graph runs
 * each piece as its own operator (RMSNorm: examples/llama/src/model.rs:150-160 through
 * luminal_nn, the sibling projections model.rs:95-100 and :24-32, the residual adds
 * model.rs:163-172); a compiler pass that finds those patterns around QuantizedMatmul
 * nodes emits one call instead.
 *   count (1..4) weights planar_dev[i] of shape (n[i], K) read the same x (K floats) and
 *   write y_dev[i] (n[i] floats);
 *   norm_weight_dev != NULL: x is replaced by x * (1/sqrt(mean(x^2) + eps)) * norm_weight;
 *   epilogue 0: y = W x;  1: y = residual + W x (count == 1; y may be residual itself);
 *   2: rows are (gate, up) pairs, row 2j = gate_j and row 2j+1 = up_j, and
 *      y[j] = up_j * gate_j / (1 + exp(-gate_j)) for j < n/2 (n even).
 * K must be a multiple of 1024 and at most 16384 (LHIP_ERR_UNSUPPORTED otherwise: run
 * the separate operators).  x and norm_weight 16-byte aligned. */
lhip_status lhip_q8_0_matvec_fused_f32(const void *const *planar_dev, float *const *y_dev, const int64_t *n, int count,
                                       const float *x_dev, int64_t k, const float *norm_weight_dev, float eps,
                                       const float *residual_dev, int epilogue, void *stream);
/* Same with an explicit launch shape: (rows_per_wave, k_unroll, waves_per_block) one of
 * (2,4,4) (1,2,4) (2,2,4) (1,1,4) (2,1,4) (1,2,16) (2,2,8) (1,1,16) (2,1,8), epilogue 2
 * needs rows_per_wave 2; blocks_per_cu in 1..16. */
lhip_status lhip_q8_0_matvec_fused_f32_cfg(const void *const *planar_dev, float *const *y_dev, const int64_t *n,
                                           int count, const float *x_dev, int64_t k, const float *norm_weight_dev,
                                           float eps, const float *residual_dev, int epilogue, int rows_per_wave,
                                           int k_unroll, int waves_per_block, int blocks_per_cu, void *stream);

/* Prefill GEMM: y[m][n] = sum_k x[m][k] * W[n][k] with bf16 activations
 * (x (m, K) row-major, 16-byte aligned), f32 accumulation on the matrix cores
 * and bf16 output (y (m, N) row-major).  The reference has no bf16 type and no
 * Q8_0 GEMM on CUDA (crates/luminal_cuda/src/quantized.rs:146-164 re-runs the
 * matvec per row); the counterpart is the Metal GEMM
 * (crates/luminal_metal/src/quantized.rs:54-61,63-199,353-376), which rounds
 * q*d to the activation type before its matrix unit.  Here the weights stay
 * exact: the int8 codes go to the matrix cores as they are (exact in bf16) and
 * every Q8_0 block's f32 sum is multiplied by the block's scale in f32, the
 * arithmetic of the reference's matvec kernel (quantized.rs:93-96).  With bf16
 * activations every product is exact, so the f32 result differs from the exact
 * one only by the roundings of the f32 additions, and the bf16 result by one
 * more rounding.  K must be a multiple of 64 (LHIP_ERR_UNSUPPORTED otherwise).
 *
 * With m <= 128 (and K % 512 == 0, N % 4 == 0, y aligned to 8 bytes; 16 for the f32
 * form below) the three entry points take a kernel that is bound by streaming the
 * weights rather than by the matrix cores.  When the 128-row strips of the weight
 * alone would not fill the chip it also splits K, keeps the f32 partial sums in a
 * 32 MiB scratch array that the library owns (a __device__ array: nothing is
 * allocated, one copy per device) and adds them in a fixed order in a second
 * launch.  Every such call on a device shares that array: calls with m <= 128 that
 * may overlap on one device (different streams, different host threads) race on it
 * and must be ordered by the caller.  Results do not depend on timing.
 * Above 128 rows the same array holds the planes of the K-sliced plans (few 256x128 tiles and a long K; the column
 * tiles that more than 256 tiles leave over after whole rounds of 256 workgroups: tile ids 120 + S and 200 of
 * lhip_q8_0_matmul_bf16_cfg), so the same rule applies to every shape for which
 * lhip_q8_0_matmul_bf16_workspace_nbytes is not zero; lhip_q8_0_matmul_bf16_ws takes the planes from the caller
 * instead and may overlap freely. */
lhip_status lhip_q8_0_matmul_bf16(const void *planar_dev, const void *x_dev, void *y_dev, int64_t m, int64_t n,
                                  int64_t k, void *stream);
/* Same GEMM with the f32 accumulators stored as they are (y (m, N) f32, 4-byte aligned): what a caller
 * whose surrounding operators are f32 wants instead of a bf16 round trip. */
lhip_status lhip_q8_0_matmul_bf16_f32out(const void *planar_dev, const void *x_dev, float *y_dev, int64_t m, int64_t n,
                                         int64_t k, void *stream);
/* Same GEMM over a weight whose rows are (gate, up) pairs (row 2j = gate_j, row 2j+1 = up_j, the order the fused
 * matvec's SwiGLU epilogue uses), writing out[r][j] = up * swish(gate) (examples/llama/src/model.rs:24-32) as bf16,
 * (m, N/2) row-major, 4-byte aligned: the f32 accumulators never leave the kernel.  Bit-equal to
 * lhip_q8_0_matmul_bf16_f32out followed by lhip_swiglu_f32_bf16out(interleaved).  N % 4 == 0. */
lhip_status lhip_q8_0_matmul_bf16_swiglu(const void *planar_dev, const void *x_dev, void *out_dev, int64_t m, int64_t n,
                                         int64_t k, void *stream);
/* Same with the output tile chosen by the caller: tile 0 = 256x128 (8 waves),
 * 1 = 128x128, 2 = 128x64, 3 = 64x64 (4 waves each),
 * 5 = the weight-streaming kernel described above, here for any m <= 8192 in passes of 128 rows
 * (LHIP_ERR_UNSUPPORTED for shapes it does not cover),
 * 50 + S = the same with S slices of K (S clamped to K / 512), 120 + S = the 256x128
 * tile over S slices of K with the partial sums in the same scratch array (2 <= S <= 16,
 * K / 64 / S a whole multiple of 4, S * m * N <= 8 Mi; what the plain entry
 * points take for K >= 8192 when whole-K tiles would leave most of the chip idle, so
 * the note on overlapping calls above applies to those shapes too),
 * 200 = the 256x128 tile in whole rounds of 256 workgroups and the column tiles left over in 2 to 8 slices of K
 * through the same scratch array (what the plain entry points take when more than 256 tiles would end in a
 * partly filled round: K >= 2048, the number of 256-row tiles a divisor of 256; LHIP_ERR_UNSUPPORTED where there
 * is no such remainder). */
lhip_status lhip_q8_0_matmul_bf16_cfg(const void *planar_dev, const void *x_dev, void *y_dev, int64_t m, int64_t n,
                                      int64_t k, int tile, void *stream);

/* Row gather: out[t][j] = dequant(W[(int)idx[t]][j]), idx carried as f32 like
 * the reference's (crates/luminal_cuda/src/quantized.rs:191-198,202-233), but
 * read from device memory.  An index outside [0, n) yields a row of zeros. */
lhip_status lhip_q8_0_gather_f32(const void *planar_dev, const float *idx_dev, float *out_dev, int64_t n_idx,
                                 int64_t n, int64_t k, void *stream);

/* The reference's second activation type, T = f16 (QuantizedMatmul<f16> / QuantizedGather<f16>,
 * crates/luminal_cuda/src/quantized.rs:42-109,170-233; its llama example runs in f16): x and y are IEEE binary16
 * (x 8-byte aligned), every product and sum is f32 as in the kernel there (:72,94-96) and the result is rounded to
 * f16 once at the store (:106); the gather rounds q*d to f16 once, which equals the product taken in half
 * precision.  Same shapes, launch choice and errors as the f32 forms. */
lhip_status lhip_q8_0_matmul_f16(const void *planar_dev, const void *x_f16_dev, void *y_f16_dev, int64_t m, int64_t n,
                                 int64_t k, void *stream);
lhip_status lhip_q8_0_gather_f16(const void *planar_dev, const float *idx_dev, void *out_f16_dev, int64_t n_idx,
                                 int64_t n, int64_t k, void *stream);

/* Re-entrant forms of lhip_q8_0_matmul_f32 / _f16.  With several activation rows those operators may cut K into
 * slices whose partial sums meet in a scratch array the library keeps per device, so two of their calls that overlap
 * in time on one device (different streams) race; the reference's operators (quantized.rs:116-149) have no such
 * constraint.  These forms keep the partial sums in the caller's workspace instead and touch no shared state:
 *   workspace_dev of lhip_q8_0_matmul_workspace_nbytes(m, n, k) bytes (256-byte aligned; 0 bytes: none is needed,
 *   NULL is fine) gives the plan, and the bits, of the plain call;
 *   a smaller one, or NULL, means fewer or no K slices: same accuracy, last bits may differ, and a short-and-small
 *   product (few rows, few weight rows) leaves compute units idle.
 * Calls sharing a workspace must be ordered on one stream.  Other arguments and errors as the plain forms. */
size_t lhip_q8_0_matmul_workspace_nbytes(int64_t m, int64_t n, int64_t k);
lhip_status lhip_q8_0_matmul_f32_ws(const void *planar_dev, const float *x_dev, float *y_dev, int64_t m, int64_t n,
                                    int64_t k, void *workspace_dev, size_t workspace_nbytes, void *stream);
lhip_status lhip_q8_0_matmul_f16_ws(const void *planar_dev, const void *x_f16_dev, void *y_f16_dev, int64_t m, int64_t n,
                                    int64_t k, void *workspace_dev, size_t workspace_nbytes, void *stream);

/* The bf16 prefill GEMM with the caller's workspace: lhip_q8_0_matmul_bf16 (out_form LHIP_GEMM_OUT_BF16),
 * _bf16_f32out (LHIP_GEMM_OUT_F32) and _bf16_swiglu (LHIP_GEMM_OUT_SWIGLU) keep the partial planes of their K-sliced
 * plans in the same per-device scratch array as the operators above and share its constraint.  This form touches no
 * shared state: workspace_dev of lhip_q8_0_matmul_bf16_workspace_nbytes(m, n, k, out_form) bytes (256-byte aligned;
 * 0: none is needed, NULL is fine) gives the plan, and the bits, of the plain call; a smaller one, or NULL, means fewer
 * or no K slices (same accuracy, last bits may differ, short-and-small products leave compute units idle).  No
 * counterpart in the reference (it has no bf16 operator). */
#define LHIP_GEMM_OUT_BF16 0
#define LHIP_GEMM_OUT_F32 1
#define LHIP_GEMM_OUT_SWIGLU 2
size_t lhip_q8_0_matmul_bf16_workspace_nbytes(int64_t m, int64_t n, int64_t k, int32_t out_form);
lhip_status lhip_q8_0_matmul_bf16_ws(const void *planar_dev, const void *x_dev, void *y_dev, int64_t m, int64_t n, int64_t k,
                                     int32_t out_form, void *workspace_dev, size_t workspace_nbytes, void *stream);

/* ---- MXFP4 weights and the mixture-of-experts layer -------------------------
 * No counterpart in the reference (it has no MXFP4 and no MoE op); built to its
 * conventions: exact dequantisation, then f32-accumulated matmul
 * (examples/llama/src/loader.rs:227-241), SwiGLU down(up(x) * swish(gate(x)))
 * (examples/llama/src/model.rs:24-32).
 *
 * Raw MXFP4 (OCP Microscaling / gpt-oss packing): blocks of 17 bytes = 16 bytes
 * of e2m1 nibbles (element 2i in the low nibble of byte i) + one e8m0 scale
 * (2^(e-127)).  A weight (N, K) is N*K/32 blocks, row-major.  Planar form:
 * nibble bytes uint8[N][K/2], padded to 256 B, then scales uint8[N][K/32]. */
size_t lhip_mxfp4_raw_nbytes(int64_t n, int64_t k);
size_t lhip_mxfp4_planar_nbytes(int64_t n, int64_t k);
size_t lhip_mxfp4_planar_scale_offset(int64_t n, int64_t k);
lhip_status lhip_mxfp4_repack(const void *raw_dev, void *planar_dev, int64_t n, int64_t k, void *stream);
lhip_status lhip_mxfp4_unpack(const void *planar_dev, void *raw_dev, int64_t n, int64_t k, void *stream);
/* Exact dequantisation to f32[N][K] (every e8m0 code, 0xff gives NaN). */
lhip_status lhip_mxfp4_dequant_f32(const void *planar_dev, float *out_dev, int64_t n, int64_t k, void *stream);
/* Dequantisation to bf16[N][K] (out 16-byte aligned) with the conversion instruction the expert GEMMs use
 * (v_cvt_scalef32_pk_bf16_fp4): e2m1 * 2^(e-127) has two significant bits and bf16 has f32's exponent range, so the
 * result equals lhip_mxfp4_dequant_f32's wherever that is a normal number (e8m0 codes 2..252 for every e2m1 value).
 * No counterpart in the reference; it is what pins the matrix path's weight values bit for bit. */
lhip_status lhip_mxfp4_dequant_bf16(const void *planar_dev, void *out_bf16_dev, int64_t n, int64_t k, void *stream);

/* Router: for each of t tokens, the topk largest of its e logits (ties to the
 * lower index) into sel[t][topk], and softmax over those k into wts[t][topk]. */
lhip_status lhip_moe_route_topk(const float *logits_dev, int32_t *sel_dev, float *wts_dev, int64_t t, int64_t e,
                                int64_t topk, void *stream);

/* Expert layer: y[t] = sum_s wts[t][s] * down_e( up_e(x[t]) * swish(gate_e(x[t])) ), e = sel[t][s].
 *   w_gate_up_planar : planar MXFP4 of shape (e*2*i, h): expert-major, rows [0,i) of an expert = gate, [i,2i) = up
 *   w_down_planar    : planar MXFP4 of shape (e*h, i)
 *   x, y             : bf16 (t, h); accumulation in f32; the SwiGLU result is rounded to bf16 between the two matmuls
 *   sel, wts         : routing as produced by lhip_moe_route_topk (an id outside [0,e) drops that term)
 *   workspace_dev    : lhip_mxfp4_moe_workspace_nbytes(...) bytes, 256-byte aligned; contents are scratch
 * h and i must be multiples of 32, e <= 1024.  e8m0 codes 0xff (NaN) in the weights are not supported here.
 *
 * Two forms of the matmuls (lhip_mxfp4_moe_bf16 is LHIP_MOE_EXACT):
 *   LHIP_MOE_EXACT  weights expanded exactly to bf16 in registers (lhip_mxfp4_dequant_bf16's values), bf16 matrix
 *                   instruction, f32 accumulation: every product is exact and every matmul output lies within the
 *                   f32 accumulation error of the exact product of its inputs (the reference's "dequantise exactly,
 *                   then multiply", examples/llama/src/loader.rs:227-241).
 *   LHIP_MOE_FAST   the block-scaled f8f6f4 matrix instruction on the raw fp4 codes, each bf16 activation split
 *                   exactly into two fp8 numbers.  The instruction aligns the 128 products of a step to the largest
 *                   and drops what lies 2^-13 below it, so an output carries an absolute error of up to about
 *                   2^-11 * sum over 128-wide chunks of max |a_k w_k|: small against typical outputs, unbounded
 *                   relative to outputs that cancel. */
#define LHIP_MOE_EXACT 0
#define LHIP_MOE_FAST 1
size_t lhip_mxfp4_moe_workspace_nbytes(int64_t t, int64_t h, int64_t i, int64_t e, int64_t topk);
lhip_status lhip_mxfp4_moe_bf16(const void *w_gate_up_planar, const void *w_down_planar, const void *x_dev,
                                const int32_t *sel_dev, const float *wts_dev, void *y_dev, int64_t t, int64_t h,
                                int64_t i, int64_t e, int64_t topk, void *workspace_dev, void *stream);
lhip_status lhip_mxfp4_moe_bf16_mode(const void *w_gate_up_planar, const void *w_down_planar, const void *x_dev,
                                     const int32_t *sel_dev, const float *wts_dev, void *y_dev, int64_t t, int64_t h,
                                     int64_t i, int64_t e, int64_t topk, int32_t mode, void *workspace_dev, void *stream);

/* lhip_mxfp4_moe_bf16 for callers that cannot allocate a workspace (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc): no counterpart in the reference.  The workspace is a scratch array inside the
 * library (a __device__ array of 8 MiB per device, held until the process ends); the call allocates and frees
 * nothing.  LHIP_ERR_UNSUPPORTED when lhip_mxfp4_moe_workspace_nbytes(t, h, i, e, topk) exceeds 8 MiB (the
 * benchmark layer, h = i = 2880 with 32 experts and top-4, fits up to t = 84).  Every call on a device shares
 * that device's array: calls that overlap in time on one device (two streams, two host threads) race for it and must
 * be ordered by the caller; the array keeps the last call's contents, and no call depends on them.  Same results,
 * bit for bit, as lhip_mxfp4_moe_bf16.  lhip_init looks the array's address up for its device; otherwise the first
 * call on a device does. */
lhip_status lhip_mxfp4_moe_bf16_static(const void *w_gate_up_planar, const void *w_down_planar, const void *x_dev,
                                       const int32_t *sel_dev, const float *wts_dev, void *y_dev, int64_t t, int64_t h,
                                       int64_t i, int64_t e, int64_t topk, void *stream);

/* The intermediates of the last layer call that used this workspace with the same (t, h, i, e, topk) and mode
 * (lhip_mxfp4_moe_read_intermediates: LHIP_MOE_EXACT, the mode of lhip_mxfp4_moe_bf16 and _static),
 * per routed entry r = t*topk + s: act_dev (t*topk, i) f32 = up * swish(gate) as the down projection consumed it
 * (a bf16 value; the fast form holds it as two fp8 numbers and a block scale, decoded exactly), down_dev (t*topk, h)
 * f32 = that entry's down projection before the weighted sum.  Either pointer may be NULL.  No counterpart in the
 * reference; it lets a caller check each of the layer's two matmuls against its own inputs, since the rounding of
 * the activations to bf16 between them makes the end-to-end result a discontinuous function of the first one. */
lhip_status lhip_mxfp4_moe_read_intermediates(const void *workspace_dev, float *act_dev, float *down_dev, int64_t t,
                                              int64_t h, int64_t i, int64_t e, int64_t topk, void *stream);
lhip_status lhip_mxfp4_moe_read_intermediates_mode(const void *workspace_dev, float *act_dev, float *down_dev, int64_t t,
                                                   int64_t h, int64_t i, int64_t e, int64_t topk, int32_t mode,
                                                   void *stream);

/* ---- the operators around the matmuls in the Llama-3 decode loop (f32) --------
 * What the reference assembles from primitive ops in examples/llama/src/model.rs,
 * as single kernels.  Positions live in device memory (pos_dev) so that a decode
 * step can be captured in a HIP graph and replayed. */

/* out[t][:] = table[(int)idx[t]][:]; fp32 embedding lookup with ids carried as f32
 * (crates/luminal_nn/src/embedding.rs:40-58, crates/luminal_cpu/src/binary.rs:175-191).
 * dim % 4 == 0; an id outside [0, n_rows) gives a zero row. */
lhip_status lhip_gather_rows_f32(const float *table_dev, const float *idx_dev, float *out_dev, int64_t n_idx,
                                 int64_t n_rows, int64_t dim, void *stream);
/* RMS norm as luminal's LayerNorm(mean_norm = false): y = v * 1/sqrt(mean(v^2) + eps) * w
 * (crates/luminal_nn/src/norm.rs:56-71, src/hl_ops/unary.rs:93-104).  With residual_dev
 * given, v = x + residual and v is also written to x_out_dev (the residual adds of
 * model.rs:173-187 fused into the norm that follows them; x_out may be x itself); otherwise
 * v = x.  dim % 4 == 0, dim <= 16384, 16-byte aligned pointers. */
lhip_status lhip_rms_norm_f32(const float *x_dev, const float *residual_dev, float *x_out_dev, const float *w_dev,
                              float *y_dev, int64_t rows, int64_t dim, float eps, void *stream);
/* Rotary embedding (adjacent pairs, model.rs:52-72) applied in place to the q and k heads
 * of fused rows qkv[tokens][(q_heads + 2*kv_heads)*head_dim] at positions *pos_dev + t, then
 * k and v appended to the caches [kv_heads][max_seq][head_dim] (model.rs:108-110).  The caches do not grow: a
 * position at or beyond max_seq is not appended (and the attention operators read at most max_seq rows), so the
 * caller keeps *pos_dev + tokens <= max_seq. */
lhip_status lhip_rope_kv_append_f32(float *qkv_dev, float *k_cache_dev, float *v_cache_dev, const int32_t *pos_dev,
                                    int64_t tokens, int64_t q_heads, int64_t kv_heads, int64_t head_dim,
                                    int64_t max_seq, float theta, void *stream);
/* Causal grouped-query attention of the q heads in qkv over the caches (model.rs:112-139):
 * out[tokens][q_heads*head_dim].  head_dim in {64, 128, 192, 256}, max_seq <= 12000;
 * qkv, caches and out 16-byte aligned. */
lhip_status lhip_attention_f32(const float *qkv_dev, const float *k_cache_dev, const float *v_cache_dev,
                               float *out_dev, const int32_t *pos_dev, int64_t tokens, int64_t q_heads,
                               int64_t kv_heads, int64_t head_dim, int64_t max_seq, void *stream);
/* Batch-1 decode: rotary + cache append + attention of the previous two operators as one call, for one new
 * token at position *pos_dev (model.rs:52-72, :108-139).  qkv_dev holds the un-rotated fused row
 * [(q_heads + 2*kv_heads)*head_dim] and is not modified; out_dev [q_heads*head_dim].  The keys of every KV head
 * are split over several workgroups whose partial softmax states meet in workspace_dev
 * (lhip_attention_decode_workspace_nbytes bytes, 256-byte aligned, contents irrelevant on entry; calls sharing a
 * workspace must be ordered on one stream) and are merged by a second small kernel.  Built for head_dim 64 or 128 and
 * q_heads / kv_heads in {1, 2, 4, 8}: LHIP_ERR_UNSUPPORTED otherwise (the workspace size is then 0). */
size_t lhip_attention_decode_workspace_nbytes(int64_t q_heads, int64_t kv_heads, int64_t head_dim);
lhip_status lhip_attention_decode_f32(const float *qkv_dev, float *k_cache_dev, float *v_cache_dev, float *out_dev,
                                      const int32_t *pos_dev, int64_t q_heads, int64_t kv_heads, int64_t head_dim,
                                      int64_t max_seq, float theta, void *workspace_dev, void *stream);
/* The same operator over FEW key ranges (one per 64-key tile up to eight for contexts of at most 2048 keys, sixteen
 * beyond) instead of all the workspace has room for: with its merge launch (_few_ranges_f32; same semantics, other
 * partial sums, so last bits differ from lhip_attention_decode_f32), and without it (_partial_f32: the ranges' partial
 * states stay in workspace_dev for lhip_q8_0_matvec_attn_merge_f32, which merges them while it stages its
 * activations).  Measured on MI355X at 512-768 keys: 9.5 us against 6.6 us for the many-range kernel - a range is
 * then two tiles of dependent trips to memory instead of one. */
lhip_status lhip_attention_decode_few_ranges_f32(const float *qkv_dev, float *k_cache_dev, float *v_cache_dev,
                                                 float *out_dev, const int32_t *pos_dev, int64_t q_heads, int64_t kv_heads,
                                                 int64_t head_dim, int64_t max_seq, float theta, void *workspace_dev,
                                                 void *stream);
lhip_status lhip_attention_decode_partial_f32(const float *qkv_dev, float *k_cache_dev, float *v_cache_dev,
                                              const int32_t *pos_dev, int64_t q_heads, int64_t kv_heads, int64_t head_dim,
                                              int64_t max_seq, float theta, void *workspace_dev, void *stream);
/* y = W att (+ residual), att = the attention output that lhip_attention_decode_few_ranges_f32 would have written for
 * the partial states lhip_attention_decode_partial_f32 left in attn_workspace_dev at position *pos_dev: the output
 * projection of model.rs:137-139 with the merge of the key ranges folded into its staging prologue (every workgroup
 * forms the q_heads * head_dim activations itself, with the merge kernel's arithmetic in the merge kernel's order, so
 * y equals lhip_attention_decode_few_ranges_f32 followed by lhip_q8_0_matvec_fused_f32 bit for bit), which takes one
 * launch out of a decoder layer.  k must equal q_heads * head_dim and be a multiple of 2048; residual_dev may be NULL
 * or equal y_dev.  Contexts beyond 2048 keys (more than eight ranges) are merged correctly but with a dependent trip
 * to memory per further range.  A measured alternative, not what the Llama engine uses by default: on MI355X the
 * pair (few-range attention 9.5 us, this call 11.5 us) takes 21.0 us per layer where many-range attention, its merge
 * launch and the plain output projection take 6.6 + 4.7 + 6.3 = 17.6 us. */
lhip_status lhip_q8_0_matvec_attn_merge_f32(const void *planar_dev, float *y_dev, int64_t n, int64_t k,
                                            const void *attn_workspace_dev, const int32_t *pos_dev, int64_t q_heads,
                                            int64_t kv_heads, int64_t head_dim, int64_t max_seq, const float *residual_dev,
                                            void *stream);
/* out[r][j] = up * swish(gate) (model.rs:24-32) with gate = gate_up[r][j], up = gate_up[r][f + j], or, with
 * interleaved != 0, gate = gate_up[r][2j], up = gate_up[r][2j + 1] (the row order the fused matvec epilogue uses). */
lhip_status lhip_swiglu_f32(const float *gate_up_dev, float *out_dev, int64_t rows, int64_t f, int interleaved,
                            void *stream);
/* The three operators that feed a bf16 GEMM, writing bf16 (round to nearest even) instead of f32, so a prompt pass
 * needs no cast kernels: same arguments and arithmetic as their f32 forms, y / out are bf16 buffers (8-byte
 * aligned).  lhip_attention_f32_bf16out runs the matrix-core kernel only (head_dim 64 or 128, q_heads / kv_heads in
 * {1, 2, 4, 8}): LHIP_ERR_UNSUPPORTED otherwise. */
lhip_status lhip_rms_norm_f32_bf16out(const float *x_dev, const float *residual_dev, float *x_out_dev,
                                      const float *w_dev, void *y_bf16_dev, int64_t rows, int64_t dim, float eps,
                                      void *stream);
lhip_status lhip_swiglu_f32_bf16out(const float *gate_up_dev, void *out_bf16_dev, int64_t rows, int64_t f,
                                    int interleaved, void *stream);
lhip_status lhip_attention_f32_bf16out(const float *qkv_dev, const float *k_cache_dev, const float *v_cache_dev,
                                       void *out_bf16_dev, const int32_t *pos_dev, int64_t tokens, int64_t q_heads,
                                       int64_t kv_heads, int64_t head_dim, int64_t max_seq, void *stream);
/* Prompt attention with bf16 matrix-core operands: Q / sqrt(head_dim), K, V and the soft-max weights are rounded to
 * bf16 for the matrix instructions, scores, soft-max and sums stay f32, output bf16 — for a prompt pass whose
 * attention output feeds a bf16 GEMM.  Five roundings of unit roundoff 2^-8 enter, one of them through the soft-max:
 * every output is within 2e-2 * sum_j p_j |v_j| of the exact softmax(QK)V (the sum before cancellation), against 1e-5
 * for the f32-operand kernel behind lhip_attention_f32_bf16out.
 * No counterpart in the reference (model.rs:112-139 builds attention from f16 primitives).  Built for head_dim 64 or
 * 128 and q_heads / kv_heads in {2, 4, 8}: LHIP_ERR_UNSUPPORTED otherwise (use lhip_attention_f32_bf16out). */
lhip_status lhip_attention_bf16(const float *qkv_dev, const float *k_cache_dev, const float *v_cache_dev,
                                void *out_bf16_dev, const int32_t *pos_dev, int64_t tokens, int64_t q_heads,
                                int64_t kv_heads, int64_t head_dim, int64_t max_seq, void *stream);
/* ---- persistent decode program --------------------------------------------
 * A batch-1 decode step as ONE launch: a list of operations that a resident grid (one workgroup
 * per compute unit) walks in order, the weight stream running on from one operation to the next.
 * No counterpart in the reference, whose graph executor runs one operator per kernel launch
 * (src/graph.rs execute loop); the operations are those of examples/llama/src/model.rs:95-139,150-160
 * in the fused forms of lhip_q8_0_matvec_fused_f32 and lhip_attention_decode_f32, with the same
 * arithmetic and reduction orders: the results equal those calls bit for bit.
 *
 * On MI355X this form is SLOWER than the per-operator launches replayed from a graph (Llama-3-8B:
 * 2.9 against 2.2 ms per token): what a launch boundary costs there (~7 us) is less than what the
 * exchange of an activation vector between 256 resident workgroups costs here.  It is kept as a
 * measured alternative, for parts and shapes where that balance differs.
 *
 * Operations:
 *   LHIP_DECODE_MATVEC     y = epilogue(W norm(x)): planar (n, k) weight, x (k floats), y (n floats; n / 2 for
 *                          SwiGLU, whose weight holds gate and up rows interleaved), norm_weight NULL or the k
 *                          gains of an RMS norm with eps, epilogue one of LHIP_FUSE_*, residual (n floats, may
 *                          be y) for LHIP_FUSE_ADD.  k % 1024 == 0 and k <= 14336 (LHIP_ERR_UNSUPPORTED beyond).
 *   LHIP_DECODE_ATTENTION  rotary + cache append + attention for the new token at *pos_dev: x = fused qkv row
 *                          (must be the output of an earlier operation), y = attention output rows, k_cache /
 *                          v_cache of the layer.  Head geometry is that of the create call: head_dim 64 or 128,
 *                          q_heads / kv_heads in {1, 2, 4, 8}.
 * Buffers are told apart by their base address and must not overlap otherwise.  x != y.  Workgroups are not
 * held back by a barrier: each waits only for the values it reads, which travel with the tag of the operation
 * that produced them.  An operation may therefore overwrite a buffer only if its own input x was produced at
 * or after the last operation that read, and the operation that wrote, the buffer's previous contents (y ==
 * residual of the same operation is fine); a list that breaks this is refused with LHIP_ERR_UNSUPPORTED.  The
 * decode loop of a transformer (h -> qkv -> attention -> h -> act -> h ...) satisfies it.  After a run every y
 * holds its operation's result.  Pointers are captured at creation; *pos_dev is read at every run.
 *
 * lhip_decode_program_run queues two kernels on the stream (a one-thread kernel that starts a new tag range,
 * then the program) and allocates nothing, so it can be captured into a graph.  Runs of one program must not
 * overlap in time.  The program kernel needs every compute unit of the device to itself while it runs: all of
 * its workgroups must be resident together, which holds when nothing else occupies the device (kernels queued
 * before it simply finish first).  Every wait inside is bounded (about a second): if values fail to arrive,
 * the kernel still ends, the step's results are meaningless, and lhip_decode_program_status (which waits for
 * the device) reports *timed_out = 1 from then on. */
enum { LHIP_DECODE_MATVEC = 0, LHIP_DECODE_ATTENTION = 1 };
enum { LHIP_FUSE_NONE = 0, LHIP_FUSE_ADD = 1, LHIP_FUSE_SWIGLU = 2 };
typedef struct lhip_decode_op {
    int32_t type;
    int32_t epilogue;
    const void *planar;
    int64_t n, k;
    const float *x;
    float *y;
    const float *norm_weight;
    float eps;
    const float *residual;
    float *k_cache, *v_cache;
} lhip_decode_op;
lhip_status lhip_decode_program_create(const lhip_decode_op *ops, int n_ops, int64_t q_heads, int64_t kv_heads,
                                       int64_t head_dim, int64_t max_seq, float theta, const int32_t *pos_dev,
                                       void **program);
lhip_status lhip_decode_program_run(void *program, void *stream);
lhip_status lhip_decode_program_status(void *program, int32_t *timed_out);
/* Per-phase clock of later runs (a profiler sees the program as one kernel): with ticks_dev != NULL, workgroup 0
 * writes the 100 MHz wall clock when it enters phase p to ticks_dev[2 p] and when it has finished its own share of
 * the phase (the wait for the phase's input included) to ticks_dev[2 p + 1].  *n_phases (if
 * given) receives the number of phases: an attention operation is two (attention, merge of the key ranges).
 * ticks_dev holds 2 * n_phases values, 8-byte aligned; NULL switches the trace off.  Takes effect at the next run
 * (not in runs already captured into a graph). */
lhip_status lhip_decode_program_trace(void *program, uint64_t *ticks_dev, int32_t *n_phases);
lhip_status lhip_decode_program_destroy(void *program);

/* Element-wise casts between f32 and bf16 (round to nearest even), for feeding f32
 * activations to the bf16 prefill GEMM. */
lhip_status lhip_cast_f32_to_bf16(const float *x_dev, void *y_dev, int64_t n, void *stream);
lhip_status lhip_cast_bf16_to_f32(const void *x_dev, float *y_dev, int64_t n, void *stream);
/* x += y */
lhip_status lhip_add_f32(float *x_dev, const float *y_dev, int64_t n, void *stream);
/* Greedy pick (examples/llama/src/main.rs:194-198; the last index wins exact ties): the index
 * goes to *id_f32_dev and/or *id_i32_dev, and *pos_dev (if given) is advanced by `advance`.
 * Rows of 16384 entries or more (16-byte aligned) take two launches whose partial picks pass through a small
 * array the library owns, one per device: picks that overlap in time on one device (two streams) race for it. */
lhip_status lhip_argmax_f32(const float *x_dev, int64_t n, float *id_f32_dev, int32_t *id_i32_dev, int32_t *pos_dev,
                            int32_t advance, void *stream);
/* lhip_argmax_f32 with the caller's workspace (512 bytes, 8-byte aligned) in place of the library's per-device array
 * of partial picks: re-entrant across streams.  Same result. */
lhip_status lhip_argmax_f32_ws(const float *x_dev, int64_t n, float *id_f32_dev, int32_t *id_i32_dev, int32_t *pos_dev,
                               int32_t advance, void *workspace_dev, void *stream);

/* ---- calibration kernels ---------------------------------------------------
 * No counterpart in the reference.  A plain device-to-device copy and a
 * read-only pass with known byte counts, used to calibrate hardware counters
 * and to measure the HBM rate a streaming kernel can reach on this part.
 * src/dst 16-byte aligned, nbytes a multiple of 16. */
lhip_status lhip_copy_bytes(void *dst_dev, const void *src_dev, size_t nbytes, void *stream);
/* Reads nbytes; each wavefront leaves the XOR of what it read in one of the
 * 1024 words of out_dev (4096 bytes, 4-byte aligned). */
lhip_status lhip_read_bytes(const void *src_dev, size_t nbytes, uint32_t *out_dev, void *stream);

/* Issue-rate probe (calibration, no counterpart in the reference): a register-only loop of `iters` x 8 independent
 * instructions of one kind on every SIMD of the device, `waves_per_simd` waves on each (256 * waves_per_simd
 * workgroups of four waves).  Lane 0 of wave w leaves out_dev[2w] = shader-clock cycles and out_dev[2w + 1] = ticks
 * of the 100 MHz wall clock that its loop took (out_dev: 2 * 1024 * waves_per_simd words of 64 bits).  Cycles per
 * instruction and SIMD = cycles * waves_per_simd / (8 * iters); the shader clock under that load = cycles / ticks *
 * 100 MHz.  These are the measured ceilings the matrix-pipe rooflines are read against. */
#define LHIP_RATE_MFMA_BF16_32X32X16 0  /* v_mfma_f32_32x32x16_bf16 (4 accumulators of 16 registers per wave) */
#define LHIP_RATE_MFMA_BF16_16X16X32 1  /* v_mfma_f32_16x16x32_bf16 */
#define LHIP_RATE_MFMA_SCALE_FP8_FP8 2  /* v_mfma_scale_f32_16x16x128_f8f6f4, both operands fp8 (e4m3) */
#define LHIP_RATE_MFMA_SCALE_FP8_FP4 3  /* ... fp8 x fp4 (e2m1) */
#define LHIP_RATE_MFMA_SCALE_FP4_FP4 4  /* ... fp4 x fp4 */
#define LHIP_RATE_MFMA_SCALE_FP6_FP4 5  /* ... fp6 (e2m3) x fp4 */
#define LHIP_RATE_CVT_BF16_FP4 6        /* v_cvt_scalef32_pk_bf16_fp4 */
lhip_status lhip_issue_rate_probe(int32_t kind, int32_t iters, int32_t waves_per_simd, uint64_t *out_dev, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* LUMINAL_HIP_H */
