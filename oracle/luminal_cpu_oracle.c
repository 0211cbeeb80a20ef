/*
 * CPU oracle for the quantized-matmul path of luminal (Q8_0 / MXFP4).
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, what the
 * reference's CPU path computes, so the HIP kernels can be checked against
 * it.  Nothing in the shipped library links, loads or calls it: only the
 * test-suite, the smoke check and the benchmark's cpu_baseline leg do.
 *
 * Compile with -ffp-contract=off: the reference rounds every product to f32
 * before it is added (src/op.rs:310-323 materialises the products, :361-382
 * adds them), so a fused multiply-add would change the bits.
 *
 * Pinning status of each function (what fixes its answer besides this file):
 *   lo_f16_to_f32 / lo_f32_to_f16   exhaustive comparison with numpy's
 *                                   IEEE binary16 over all 65536 codes
 *   lo_q8_0_dequant                 closed form int8*f16 exact in f32; byte
 *                                   layout pinned by three agreeing struct
 *                                   definitions in the reference and the
 *                                   n + n/16 size law
 *   lo_matmul_seq_f32 / _f64        the reference's literal matmul tests
 *                                   (crates/luminal_cpu/src/lib.rs:177-192,
 *                                   src/tests/mod.rs:38-54), integer-exact
 *                                   cases, numpy float64 on random data
 *   lo_q8_0_gather                  equals dequant of the selected rows
 *   lo_mxfp4_dequant, lo_moe_*      NOT in the reference: parity unpinned by
 *                                   the reference; pinned by the OCP MX
 *                                   value table and closed forms only
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ */
/* binary16 <-> binary32                                               */
/* ------------------------------------------------------------------ */

/* IEEE-754 binary16 -> binary32 widening (exact, subnormals included).
 * The reference calls half::f16::to_f32 at examples/llama/src/loader.rs:239. */
float lo_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: value = man * 2^-24 */
            int e = -1;
            do {
                man <<= 1;
                e++;
            } while (!(man & 0x400u));
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 112u) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* binary32 -> binary16, round to nearest even (half::f16::from_f32, used by
 * the reference's tests to build blocks:
 * crates/luminal_metal/src/quantized.rs:907). */
uint16_t lo_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t ax = x & 0x7fffffffu;
    if (ax >= 0x7f800000u) { /* inf / nan */
        return (uint16_t)(sign | 0x7c00u | ((ax > 0x7f800000u) ? (0x200u | ((ax >> 13) & 0x3ffu)) : 0u));
    }
    if (ax >= 0x477ff000u) { /* rounds to >= 65520 -> inf */
        return (uint16_t)(sign | 0x7c00u);
    }
    if (ax < 0x38800000u) { /* subnormal or zero in half */
        if (ax < 0x33000000u) return (uint16_t)sign; /* < 2^-25 -> 0 */
        int e = (int)(ax >> 23);
        uint32_t man = (ax & 0x7fffffu) | 0x800000u;
        int shift = 126 - e; /* value = man * 2^(e-150); half sub ulp = 2^-24 */
        uint32_t q = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (q & 1u))) q++;
        return (uint16_t)(sign | q);
    }
    uint32_t e = (ax >> 23) - 112u;
    uint32_t man = ax & 0x7fffffu;
    uint32_t q = (e << 10) | (man >> 13);
    uint32_t rem = man & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;
    return (uint16_t)(sign | q);
}

/* binary32 -> bfloat16 round to nearest even, and back (exact). */
uint16_t lo_f32_to_bf16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
    x += 0x7fffu + ((x >> 16) & 1u);
    return (uint16_t)(x >> 16);
}
float lo_bf16_to_f32(uint16_t h) {
    uint32_t x = (uint32_t)h << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

/* ------------------------------------------------------------------ */
/* Q8_0                                                                */
/* ------------------------------------------------------------------ */

/* Bytes of n Q8_0 weights: n + n/16 (examples/llama/src/loader.rs:126-129). */
size_t lo_q8_0_nbytes(size_t n_elements) { return n_elements + n_elements / 16; }

/* Dequantise raw GGUF Q8_0 blocks (34 B: little-endian f16 delta, then 32
 * int8) to f32: w = (q as f32) * delta.to_f32()
 * (examples/llama/src/loader.rs:227-241; block struct :173-178). */
void lo_q8_0_dequant(const uint8_t *blocks, size_t n_elements, float *out) {
    size_t nb = n_elements / 32;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *p = blocks + b * 34;
        float d = lo_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
        for (int i = 0; i < 32; i++) out[b * 32 + i] = (float)(int8_t)p[2 + i] * d;
    }
}

/* Pack int8 quants + f16 scale codes into raw 34-byte blocks. */
void lo_q8_0_pack(const int8_t *qs, const uint16_t *d, size_t n_elements, uint8_t *blocks) {
    size_t nb = n_elements / 32;
    for (size_t b = 0; b < nb; b++) {
        uint8_t *p = blocks + b * 34;
        p[0] = (uint8_t)(d[b] & 0xff);
        p[1] = (uint8_t)(d[b] >> 8);
        memcpy(p + 2, qs + b * 32, 32);
    }
}

/* Row gather over a Q8_0 table: out[t][j] = dequant(table[idx[t]][j]); the
 * indices are carried as f32 and truncated
 * (crates/luminal_cuda/src/quantized.rs:191-198; CPU Gather
 * crates/luminal_cpu/src/binary.rs:175-191). */
void lo_q8_0_gather(const uint8_t *blocks, const float *idx, size_t n_idx, size_t dim, float *out) {
    for (size_t t = 0; t < n_idx; t++) {
        size_t e = (size_t)idx[t];
        lo_q8_0_dequant(blocks + (e * dim / 32) * 34, dim, out + t * dim);
    }
}

/* ------------------------------------------------------------------ */
/* f32 matmul y = x . W^T, W stored (N,K) row-major                    */
/* ------------------------------------------------------------------ */

/* The un-fused core path: Mul materialises a[m,k]*w[n,k] rounded to f32
 * (src/op.rs:310-323), SumReduce adds them in increasing k into an f32
 * (src/op.rs:361-382).  Operand orientation: src/hl_ops/matmul.rs:4-33. */
void lo_matmul_seq_f32(const float *a, const float *w, float *c, size_t M, size_t N, size_t K) {
    for (size_t m = 0; m < M; m++)
        for (size_t n = 0; n < N; n++) {
            float acc = 0.0f;
            const float *ar = a + m * K, *wr = w + n * K;
            for (size_t k = 0; k < K; k++) {
                float p = ar[k] * wr[k];
                acc += p;
            }
            c[m * N + n] = acc;
        }
}

/* Same sum in binary64: the "truth" tolerance checks are made against. */
void lo_matmul_f64(const float *a, const float *w, double *c, size_t M, size_t N, size_t K) {
    for (size_t m = 0; m < M; m++)
        for (size_t n = 0; n < N; n++) {
            double acc = 0.0;
            const float *ar = a + m * K, *wr = w + n * K;
            for (size_t k = 0; k < K; k++) acc += (double)ar[k] * (double)wr[k];
            c[m * N + n] = acc;
        }
}

/* Throughput-shaped restatement of luminal_cpu::MatMul2D
 * (crates/luminal_cpu/src/matmul.rs:64-92): the reference hands the f32
 * operands to matrixmultiply::sgemm, single-threaded as configured
 * (crates/luminal_cpu/Cargo.toml has no "threading" feature).  sgemm's
 * summation order is its own; this version keeps 8 independent partial sums
 * per output so the compiler can vectorise, and is used as the CPU baseline
 * of the benchmark (threads = 1) and, with OpenMP over rows, as the
 * all-cores variant.  It is not a bit-exact model of sgemm. */
void lo_matmul_fast_f32(const float *a, const float *w, float *c, size_t M, size_t N, size_t K, int threads) {
#if defined(_OPENMP)
#pragma omp parallel for num_threads(threads) schedule(static) if (threads > 1)
#endif
    for (long n = 0; n < (long)N; n++) {
        const float *wr = w + (size_t)n * K;
        for (size_t m = 0; m < M; m++) {
            const float *ar = a + m * K;
            float acc[16] = {0};
            size_t k = 0;
            for (; k + 16 <= K; k += 16)
                for (int j = 0; j < 16; j++) acc[j] += ar[k + j] * wr[k + j];
            float s = 0.0f;
            for (int j = 0; j < 16; j++) s += acc[j];
            for (; k < K; k++) s += ar[k] * wr[k];
            c[m * N + (size_t)n] = s;
        }
    }
}

/* ------------------------------------------------------------------ */
/* MXFP4 (OCP Microscaling: 32 x e2m1 + one e8m0 scale)                */
/* Not in the reference.  Convention follows the Q8_0 path: dequantise  */
/* exactly to f32, then f32 matmul.                                    */
/* ------------------------------------------------------------------ */

static const float LO_E2M1[16] = {0.0f, 0.5f, 1.0f, 1.5f, 2.0f, 3.0f, 4.0f, 6.0f,
                                  -0.0f, -0.5f, -1.0f, -1.5f, -2.0f, -3.0f, -4.0f, -6.0f};

/* e8m0 scale byte -> 2^(e-127); 0xff is NaN per the OCP MX spec. */
float lo_e8m0_to_f32(uint8_t e) {
    if (e == 0xff) return NAN;
    return ldexpf(1.0f, (int)e - 127);
}

/* Block = 16 bytes of nibbles (element 2i in the low nibble of byte i,
 * element 2i+1 in the high nibble) followed by one e8m0 byte: 17 B / 32
 * weights. */
void lo_mxfp4_dequant(const uint8_t *blocks, size_t n_elements, float *out) {
    size_t nb = n_elements / 32;
    for (size_t b = 0; b < nb; b++) {
        const uint8_t *p = blocks + b * 17;
        float s = lo_e8m0_to_f32(p[16]);
        for (int i = 0; i < 16; i++) {
            out[b * 32 + 2 * i] = LO_E2M1[p[i] & 0xf] * s;
            out[b * 32 + 2 * i + 1] = LO_E2M1[p[i] >> 4] * s;
        }
    }
}

/* swish(t) = t * 1/(1+exp(-t))  (src/hl_ops/unary.rs:169-177). */
static float lo_swish(float t) { return t * (1.0f / (1.0f + expf(-t))); }

/* One MoE expert layer over T tokens, luminal's SwiGLU convention
 * (examples/llama/src/model.rs:24-32): out = down( up(x) * swish(gate(x)) ).
 *   x        T x H   f32 (bf16-representable values when checking bf16 paths)
 *   w_gu     E x (2I) x H  f32, rows [0,I) = gate, rows [I,2I) = up
 *   w_down   E x H x I     f32
 *   sel      T x topk expert ids, wts T x topk routing weights
 *   act_bf16 round the SwiGLU activations to bf16 before the down projection
 *            (what a bf16 kernel pipeline does between its two GEMMs)
 * Accumulation in f64 so the result is "truth" for tolerance checks. */
void lo_moe_forward(const float *x, const float *w_gu, const float *w_down, const int32_t *sel, const float *wts,
                    size_t T, size_t H, size_t I, size_t topk, int act_bf16, float *out) {
    float *act = (float *)malloc(I * sizeof(float));
    for (size_t t = 0; t < T; t++) {
        for (size_t h = 0; h < H; h++) out[t * H + h] = 0.0f;
        double *acc = (double *)calloc(H, sizeof(double));
        for (size_t s = 0; s < topk; s++) {
            size_t e = (size_t)sel[t * topk + s];
            const float *gu = w_gu + e * 2 * I * H;
            const float *dn = w_down + e * H * I;
            for (size_t i = 0; i < I; i++) {
                double g = 0.0, u = 0.0;
                for (size_t h = 0; h < H; h++) {
                    g += (double)x[t * H + h] * gu[i * H + h];
                    u += (double)x[t * H + h] * gu[(I + i) * H + h];
                }
                float a = (float)u * lo_swish((float)g);
                act[i] = act_bf16 ? lo_bf16_to_f32(lo_f32_to_bf16(a)) : a;
            }
            for (size_t h = 0; h < H; h++) {
                double d = 0.0;
                for (size_t i = 0; i < I; i++) d += (double)act[i] * dn[h * I + i];
                acc[h] += (double)wts[t * topk + s] * d;
            }
        }
        for (size_t h = 0; h < H; h++) out[t * H + h] = (float)acc[h];
        free(acc);
    }
    free(act);
}

/* Router: top-k of the logits (ties -> lower index), softmax over the
 * selected k (gpt-oss style routing; exp/sum as src/hl_ops/unary.rs:126-130). */
void lo_moe_route(const float *logits, size_t T, size_t E, size_t topk, int32_t *sel, float *wts) {
    for (size_t t = 0; t < T; t++) {
        const float *l = logits + t * E;
        for (size_t s = 0; s < topk; s++) {
            int best = -1;
            for (size_t e = 0; e < E; e++) {
                int taken = 0;
                for (size_t r = 0; r < s; r++) taken |= (sel[t * topk + r] == (int32_t)e);
                if (taken) continue;
                if (best < 0 || l[e] > l[best]) best = (int)e;
            }
            sel[t * topk + s] = best;
        }
        float mx = l[sel[t * topk]];
        float sum = 0.0f;
        for (size_t s = 0; s < topk; s++) {
            wts[t * topk + s] = expf(l[sel[t * topk + s]] - mx);
            sum += wts[t * topk + s];
        }
        for (size_t s = 0; s < topk; s++) wts[t * topk + s] *= 1.0f / sum;
    }
}
