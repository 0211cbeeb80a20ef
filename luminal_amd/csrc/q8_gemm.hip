// Q8_0 GEMM for prefill:  Y[M][N] = X[M][K] . W[N][K]^T, bf16 activations,
// f32 accumulation on the matrix cores, bf16 output.
//
// The reference has no such kernel on CUDA (its QuantizedMatmul re-runs the
// matvec once per activation row, crates/luminal_cuda/src/quantized.rs:146-164);
// the design precedent is the Metal backend's GEMM, which dequantises a weight
// tile into threadgroup memory (q * d rounded to the activation type) and feeds
// the matrix unit (crates/luminal_metal/src/quantized.rs:54-61,63-199).  This
// kernel does the same for gfx950:
//   * a workgroup owns a BM x BN output tile and walks K in steps of 64 (two
//     Q8_0 blocks);
//   * activations go global -> registers -> LDS as bf16; weights go global
//     (planar int8, 16-byte loads) -> registers -> dequantised q*d, rounded to
//     bf16 (v_cvt_pk_bf16_f32, round-to-nearest-even) -> LDS;
//   * LDS is double-buffered and the global loads run D = 4 tiles ahead in
//     rotating register sets, so HBM/L2 latency is covered by three tiles of
//     MFMA work; one barrier per tile separates LDS writers from readers;
//   * each wavefront computes a (BM/WM) x (BN/WN) sub-tile with
//     v_mfma_f32_32x32x16_bf16; LDS rows are padded by 16 bytes so the 16-byte
//     operand reads of 8 consecutive lanes hit all banks once;
//   * workgroups that share a weight tile (same N tile, different M tiles) get
//     consecutive slots on the same XCD (block id modulo 8), so the weight tile
//     is fetched from HBM once and re-read from that XCD's L2.
#include <hip/hip_fp16.h>

#include "common.h"

namespace lhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t gu32x4 __attribute__((ext_vector_type(4)));

constexpr int kBK = 64;             // K per tile: two Q8_0 blocks
constexpr int kRowBytes = 144;      // 64 bf16 + 16 bytes of padding

__device__ __forceinline__ float sbyte(uint32_t w, int i) {
    return static_cast<float>(static_cast<int8_t>((w >> (8 * i)) & 0xff));
}

// 4 packed int8 -> 4 bf16 (q * d, rounded to nearest even), as two dwords.
__device__ __forceinline__ uint2 dequant4_bf16(uint32_t q4, float d) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    bf16x2 lo = {static_cast<__bf16>(sbyte(q4, 0) * d), static_cast<__bf16>(sbyte(q4, 1) * d)};
    bf16x2 hi = {static_cast<__bf16>(sbyte(q4, 2) * d), static_cast<__bf16>(sbyte(q4, 3) * d)};
    return make_uint2(__builtin_bit_cast(uint32_t, lo), __builtin_bit_cast(uint32_t, hi));
}

// D = register prefetch depth in K tiles (D > 1 needs K % (64*D) == 0 and D even).
// OutT = __bf16 (rounded to nearest even) or float (the accumulators as they are).
template <int BM, int BN, int WM, int WN, int D, bool PIPE = false, typename OutT = __bf16>
__global__ __launch_bounds__(WM *WN * 64) void q8_gemm_bf16_kernel(const int8_t *__restrict__ qs,
                                                                   const __half *__restrict__ ds,
                                                                   const __bf16 *__restrict__ x,
                                                                   OutT *__restrict__ y_all, int M, int N, int K,
                                                                   int m_tiles, int n_tiles, int swiglu, int kt_slice) {
    constexpr int T = WM * WN * 64;
    constexpr int TM = BM / WM, TN = BN / WN;  // wave tile
    constexpr int FM = TM / 32, FN = TN / 32;  // 32x32 MFMA tiles per wave
    constexpr int A_CHUNKS = BM * 8 / T;       // 16-byte chunks (8 bf16) per thread per tile
    constexpr int B_CHUNKS = BN * 4 / T;       // 16-byte chunks (16 int8) per thread per tile
    static_assert(A_CHUNKS >= 1 && B_CHUNKS >= 1 && BM * 8 % T == 0 && BN * 4 % T == 0, "tile/thread mismatch");
    constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // 2 x (A tile, B tile)

    // Block id -> (m tile, n tile): ids that differ by 8 run on the same XCD;
    // the m tiles of one n tile take consecutive such ids.
    int mt, nt;
    {
        const int id = blockIdx.x;
        const int xcd = id & 7, slot = id >> 3;
        const int n_hi = slot / m_tiles;
        mt = slot - n_hi * m_tiles;
        nt = n_hi * 8 + xcd;
        if (nt >= n_tiles) return;  // grid is padded to a multiple of 8 n tiles
    }
    const int m0 = mt * BM, n0 = nt * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int nblk = K >> 5;
    // kt_slice > 0: blockIdx.y takes K tiles [kt0, kt0 + KT) and writes its f32 partial result to plane blockIdx.y
    // of y (the caller adds the planes); 0: all of K.
    const int kt0 = kt_slice > 0 ? static_cast<int>(blockIdx.y) * kt_slice : 0;
    const int KT = kt_slice > 0 ? min(kt_slice, K / kBK - kt0) : K / kBK;
    OutT *__restrict__ y = y_all + (kt_slice > 0 ? static_cast<size_t>(blockIdx.y) * M * N : 0);

    // Per-thread global sources (rows past the edge re-read the last row; their results are not stored).
    const __bf16 *a_src[A_CHUNKS];
    int a_dst[A_CHUNKS];
#pragma unroll
    for (int i = 0; i < A_CHUNKS; ++i) {
        const int c = tid + i * T;
        const int row = c >> 3, col = (c & 7) * 8;
        a_src[i] = x + static_cast<size_t>(min(m0 + row, M - 1)) * K + col + kt0 * kBK;
        a_dst[i] = row * kRowBytes + col * 2;
    }
    const int8_t *b_src[B_CHUNKS];
    const uint32_t *d_src[B_CHUNKS];  // the two scales of a K tile are one aligned dword (K/32 is even)
    int d_shift[B_CHUNKS];
    int b_dst[B_CHUNKS];
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
        const int c = tid + i * T;
        const int row = c >> 2, q16 = c & 3;
        const int grow = min(n0 + row, N - 1);
        b_src[i] = qs + static_cast<size_t>(grow) * K + q16 * 16 + kt0 * kBK;
        d_src[i] = reinterpret_cast<const uint32_t *>(ds + static_cast<size_t>(grow) * nblk) + kt0;
        d_shift[i] = (q16 >> 1) * 16;
        b_dst[i] = row * kRowBytes + q16 * 32;
    }

    // D register sets: tile t lives in set t % D from its load until it is written to LDS.
    gu32x4 a_reg[D][A_CHUNKS], b_reg[D][B_CHUNKS];
    uint32_t d_reg[D][B_CHUNKS];  // both f16 scale codes of the tile
    // part p of P: the p-th share of the thread's chunks (P = 1: everything), the same split as store_tile's.
    auto load_tile = [&](int set, int kt, int p = 0, int P = 1) {
        const int k0 = min(kt, KT - 1) * kBK;  // tiles past the end re-read the last one (never used)
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i)
            if (i * P / A_CHUNKS == p) a_reg[set][i] = *reinterpret_cast<const gu32x4 *>(a_src[i] + k0);
#pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i) {
            if (i * P / B_CHUNKS != p) continue;
            b_reg[set][i] = __builtin_nontemporal_load(reinterpret_cast<const gu32x4 *>(b_src[i] + k0));
            d_reg[set][i] = d_src[i][k0 >> 6];
        }
    };
    // part p of P: the p-th share of the thread's chunks (P = 1: everything).  A weight chunk (16 quants -> two
    // 16-byte halves of bf16) counts as two units, so its unpacking can be spread over two parts.
    auto store_tile = [&](int set, int buf, int p = 0, int P = 1) {
        unsigned char *A = lds + buf * (A_BYTES + B_BYTES);
        unsigned char *B = A + A_BYTES;
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i)
            if (i * P / A_CHUNKS == p) *reinterpret_cast<gu32x4 *>(A + a_dst[i]) = a_reg[set][i];
#pragma unroll
        for (int u = 0; u < 2 * B_CHUNKS; ++u) {
            if (u * P / (2 * B_CHUNKS) != p) continue;
            const int i = u >> 1;
            // Opaque to the optimiser: keeps the unpacking of this set here, at its use,
            // instead of next to its loads (where it would wait for data just requested).
            asm volatile("" : "+v"(b_reg[set][i]), "+v"(d_reg[set][i]));
            const float d = __half2float(__ushort_as_half(static_cast<unsigned short>(d_reg[set][i] >> d_shift[i])));
            if ((u & 1) == 0) {
                const uint2 w0 = dequant4_bf16(b_reg[set][i].x, d), w1 = dequant4_bf16(b_reg[set][i].y, d);
                gu32x4 lo = {w0.x, w0.y, w1.x, w1.y};
                *reinterpret_cast<gu32x4 *>(B + b_dst[i]) = lo;
            } else {
                const uint2 w2 = dequant4_bf16(b_reg[set][i].z, d), w3 = dequant4_bf16(b_reg[set][i].w, d);
                gu32x4 hi = {w2.x, w2.y, w3.x, w3.y};
                *reinterpret_cast<gu32x4 *>(B + b_dst[i] + 16) = hi;
            }
        }
    };

    f32x16 acc[FM][FN];
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

    // MFMA operand addresses inside a tile: lane l reads 8 consecutive k of row (l % 32), k group (l / 32).
    const int frag_off = (lane & 31) * kRowBytes + (lane >> 5) * 16;
    auto compute_tile = [&](int buf) {
        const unsigned char *A = lds + buf * (A_BYTES + B_BYTES) + (wm * TM) * kRowBytes + frag_off;
        const unsigned char *B = lds + buf * (A_BYTES + B_BYTES) + A_BYTES + (wn * TN) * kRowBytes + frag_off;
#pragma unroll
        for (int kk = 0; kk < kBK / 16; ++kk) {
            bf16x8 af[FM], bfr[FN];
#pragma unroll
            for (int i = 0; i < FM; ++i) af[i] = *reinterpret_cast<const bf16x8 *>(A + i * 32 * kRowBytes + kk * 32);
#pragma unroll
            for (int j = 0; j < FN; ++j) bfr[j] = *reinterpret_cast<const bf16x8 *>(B + j * 32 * kRowBytes + kk * 32);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        }
    };

    // Pipelined form of compute_tile + store_tile: the operand fragments of step kk+1 are requested before the
    // MFMAs of step kk, and the dequantise-and-store of the next tile is dealt out over the four steps so its VALU
    // and LDS-write work sits between the MFMAs instead of after them (measured: +10 % on the large shapes).
    // The global loads of the tile after next are dealt out the same way: issued all at once at the top of a step
    // by all eight waves, they fill the memory pipeline's queue (48 KiB per K tile at 64 B/clk is ~770 cycles) and
    // the later waves sit in their load instructions for ~1000 cycles while the first wave of each SIMD runs its
    // MFMAs alone; the two waves of a SIMD then work one after the other instead of side by side.
    auto compute_and_store = [&](int buf, int set, int next_buf, int load_set, int load_kt) {
        const unsigned char *A = lds + buf * (A_BYTES + B_BYTES) + (wm * TM) * kRowBytes + frag_off;
        const unsigned char *B = lds + buf * (A_BYTES + B_BYTES) + A_BYTES + (wn * TN) * kRowBytes + frag_off;
        bf16x8 af[2][FM], bfr[2][FN];
        auto load_frags = [&](int kk, int to) {
#pragma unroll
            for (int i = 0; i < FM; ++i) af[to][i] = *reinterpret_cast<const bf16x8 *>(A + i * 32 * kRowBytes + kk * 32);
#pragma unroll
            for (int j = 0; j < FN; ++j) bfr[to][j] = *reinterpret_cast<const bf16x8 *>(B + j * 32 * kRowBytes + kk * 32);
        };
        load_frags(0, 0);
#pragma unroll
        for (int kk = 0; kk < kBK / 16; ++kk) {
            if (kk + 1 < kBK / 16) load_frags(kk + 1, (kk + 1) & 1);
            store_tile(set, next_buf, kk, kBK / 16);
            load_tile(load_set, load_kt, kk, kBK / 16);
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[kk & 1][i], bfr[kk & 1][j], acc[i][j], 0, 0, 0);
        }
    };

#pragma unroll
    for (int j = 0; j < D; ++j) load_tile(j, j);
    store_tile(0, 0);
    __syncthreads();

    if constexpr (D == 1) {
        for (int kt = 0; kt < KT; ++kt) {
            load_tile(0, kt + 1);
            compute_tile(kt & 1);
            store_tile(0, (kt + 1) & 1);
            __syncthreads();
        }
    } else {
        static_assert(D % 2 == 0, "LDS buffer parity must follow the register set");
        for (int kt = 0; kt < KT; kt += D) {
#pragma unroll
            for (int j = 0; j < D; ++j) {
                // set j held tile kt+j, already in LDS: refill it with tile kt+j+D
                if constexpr (PIPE) {
                    compute_and_store(j & 1, (j + 1) % D, (j + 1) & 1, j, kt + j + D);
                } else {
                    load_tile(j, kt + j + D);
                    // Keep the loads here, at the top of the step: if they sink towards the
                    // LDS stores below, the wait for the tile loaded D-1 steps ago also
                    // waits for them and the prefetch distance collapses.
                    __builtin_amdgcn_sched_barrier(0);
                    compute_tile(j & 1);
                    store_tile((j + 1) % D, (j + 1) & 1);  // tile kt+j+1, loaded D-1 iterations ago
                }
                __syncthreads();
            }
        }
    }

    // Epilogue: acc element v of lane l is row 8*(v/4) + 4*(l/32) + v%4, column l%32 of its 32x32 tile.
    if constexpr (sizeof(OutT) == 2) {
        if (swiglu) {
            // Columns are (gate, up) pairs (weight rows interleaved at load): y[row][c/2] = up * swish(gate), N/2
            // columns of bf16.  A pair sits in neighbouring lanes; two pairs are packed into one 4-byte store.
#pragma unroll
            for (int i = 0; i < FM; ++i)
#pragma unroll
                for (int j = 0; j < FN; ++j) {
                    const int col = n0 + wn * TN + j * 32 + (lane & 31);
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int row = m0 + wm * TM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                        const float mine = acc[i][j][v], other = __shfl_xor(mine, 1);
                        const float act = (lane & 1) ? swiglu_value(other, mine) : swiglu_value(mine, other);
                        const float act2 = __shfl_xor(act, 2);
                        if ((lane & 3) == 0 && row < M && col < N) {
                            typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
                            const bf16x2 pk = {static_cast<__bf16>(act), static_cast<__bf16>(act2)};
                            *reinterpret_cast<bf16x2 *>(reinterpret_cast<__bf16 *>(y) +
                                                        static_cast<size_t>(row) * (N >> 1) + (col >> 1)) = pk;
                        }
                    }
                }
            return;
        }
    }
#pragma unroll
    for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) {
            const int col = n0 + wn * TN + j * 32 + (lane & 31);
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = m0 + wm * TM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
                if (row < M && col < N) y[static_cast<size_t>(row) * N + col] = static_cast<OutT>(acc[i][j][v]);
            }
        }
}

// What the epilogue writes: bf16 (m, N), f32 (m, N), or bf16 (m, N/2) = up * swish(gate) of (gate, up) column pairs.
enum { kOutBf16 = 0, kOutF32 = 1, kOutSwiglu = 2 };

// q8_gemm_skinny.hip: the weight-streaming kernel for at most 128 activation rows.
bool q8_gemm_skinny_supports(int m, int n, int k, int out, const void *y);
lhip_status q8_gemm_skinny_launch(const int8_t *qs, const __half *ds, const void *x_bf16, void *y, int m, int n, int k,
                                  int out, int splits, hipStream_t s);
float *q8_gemm_scratch(size_t *floats);  // the library's partial-sum array on the current device
lhip_status q8_gemm_reduce_launch(const float *part, void *y, int m, int n, int slices, int out, hipStream_t s);
constexpr int kTileSkinny = 5;        // K slices chosen by the library
constexpr int kTileSkinnySplit = 50;  // + number of K slices
constexpr int kTileSliced = 120;      // + number of K slices: the 256x128 tile over slices of K, then a reduction

template <int BM, int BN, int WM, int WN, int D, bool PIPE, typename OutT>
static lhip_status launch_gemm_t(const int8_t *qs, const __half *ds, const void *x, void *y, int m, int n, int k,
                                 int swiglu, hipStream_t s, int slices = 1) {
    const int m_tiles = (m + BM - 1) / BM, n_tiles = (n + BN - 1) / BN;
    const int n_tiles_pad = (n_tiles + 7) / 8 * 8;
    const size_t lds_bytes = 2 * static_cast<size_t>(BM + BN) * kRowBytes;
    auto kern = q8_gemm_bf16_kernel<BM, BN, WM, WN, D, PIPE, OutT>;
    if (lds_bytes > 64 * 1024) {
        // Opting in to more than 64 KiB of dynamic LDS is a per-function attribute.
        LHIP_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    }
    const int kt_slice = slices > 1 ? (k / kBK + slices - 1) / slices : 0;
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(m_tiles * n_tiles_pad), static_cast<unsigned>(slices)),
                       dim3(WM * WN * 64), lds_bytes, s, qs, ds, static_cast<const __bf16 *>(x), static_cast<OutT *>(y), m,
                       n, k, m_tiles, n_tiles, swiglu, kt_slice);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

template <int BM, int BN, int WM, int WN, int D, bool PIPE = false>
static lhip_status launch_gemm(int out, const int8_t *qs, const __half *ds, const void *x, void *y, int m, int n,
                               int k, hipStream_t s) {
    return out == kOutF32 ? launch_gemm_t<BM, BN, WM, WN, D, PIPE, float>(qs, ds, x, y, m, n, k, 0, s)
                          : launch_gemm_t<BM, BN, WM, WN, D, PIPE, __bf16>(qs, ds, x, y, m, n, k, out == kOutSwiglu, s);
}

static lhip_status gemm_dispatch(const void *planar_dev, const void *x_dev, void *y_dev, int64_t m, int64_t n, int64_t k,
                                 int tile, int out, void *stream) {
    if (!planar_dev || !x_dev || !y_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (m <= 0 || m > kMaxDim) return LHIP_ERR_INVALID_SHAPE;
    if (k % kBK != 0) return LHIP_ERR_UNSUPPORTED;
    if (out == kOutSwiglu && n % 4 != 0) return LHIP_ERR_INVALID_SHAPE;  // pairs, stored two at a time
    if (!aligned(planar_dev, 256) || !aligned(x_dev, 16) || !aligned(y_dev, out == kOutBf16 ? 2 : 4)) return LHIP_ERR_MISALIGNED;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    auto *qs = reinterpret_cast<const int8_t *>(base);
    auto *ds = reinterpret_cast<const __half *>(base + q8_scale_offset(n, k));
    const int mi = static_cast<int>(m), ni = static_cast<int>(n), ki = static_cast<int>(k);
    hipStream_t s = as_stream(stream);
    // Deep register prefetch (4 K tiles ahead) needs K to be a whole number of 4-tile rounds.
    const bool deep = (k % (kBK * 4)) == 0;
#define LHIP_TILE(BM, BN, WM, WN)                                                                  \
    return deep ? launch_gemm<BM, BN, WM, WN, 4, true>(out, qs, ds, x_dev, y_dev, mi, ni, ki, s) \
                : launch_gemm<BM, BN, WM, WN, 1>(out, qs, ds, x_dev, y_dev, mi, ni, ki, s)
    if (tile == kTileSkinny || (tile > kTileSkinnySplit && tile <= kTileSkinnySplit + 64)) {
        if (!q8_gemm_skinny_supports(mi, ni, ki, out, y_dev)) return LHIP_ERR_UNSUPPORTED;
        return q8_gemm_skinny_launch(qs, ds, x_dev, y_dev, mi, ni, ki, out, tile == kTileSkinny ? 0 : tile - kTileSkinnySplit, s);
    }
    if (tile > kTileSliced && tile <= kTileSliced + 16) {
        // Few output tiles and a long K (the down projection of a 512-token prompt: 64 tiles of 256x128): slices of K
        // fill the chip, f32 partial planes go to the scratch array and are added in slice order.
        const int slices = tile - kTileSliced;
        const int kt = ki / kBK;
        size_t cap = 0;
        float *part = q8_gemm_scratch(&cap);
        if (!part) return LHIP_ERR_HIP;
        if (slices < 2 || kt % slices != 0 || (kt / slices) % 4 != 0 || static_cast<size_t>(slices) * mi * ni > cap ||
            ni % 4 != 0 || !aligned(y_dev, out == kOutF32 ? 16 : (out == kOutBf16 ? 8 : 4)))
            return LHIP_ERR_UNSUPPORTED;
        if (lhip_status st = launch_gemm_t<256, 128, 4, 2, 4, true, float>(qs, ds, x_dev, part, mi, ni, ki, 0, s, slices))
            return st;
        return q8_gemm_reduce_launch(part, y_dev, mi, ni, slices, out, s);
    }
    switch (tile) {
        case 0: LHIP_TILE(256, 128, 4, 2);
        case 1: LHIP_TILE(128, 128, 2, 2);
        case 2: LHIP_TILE(128, 64, 2, 2);
        case 3: LHIP_TILE(64, 64, 2, 2);
        case 4:  // 256x256 by eight 64x128 waves: 0.75 KiB of LDS operand reads per MFMA instead of 1; both
                 // LDS buffers together are 144 KiB, which leaves registers for a prefetch depth of two K tiles
            if (k % (kBK * 2) != 0) return LHIP_ERR_UNSUPPORTED;
            return launch_gemm<256, 256, 4, 2, 2, true>(out, qs, ds, x_dev, y_dev, mi, ni, ki, s);
        default: return LHIP_ERR_UNSUPPORTED;
    }
#undef LHIP_TILE
}

static int gemm_auto_tile(int64_t m, int64_t n, int64_t k, int out, const void *y) {
    // Few activation rows: the product is bound by the weight stream
    if (m <= 128 && n <= kMaxDim && k <= kMaxDim &&
        q8_gemm_skinny_supports(static_cast<int>(m), static_cast<int>(n), static_cast<int>(k), out, y))
        return kTileSkinny;
    // Largest tile that still gives at least three quarters of the 256 CUs a
    // workgroup (measured: 224 workgroups of 256x256 beat 448 of 256x128, which
    // beat 896 of 128x128); a 256-row tile is skipped when it would be half padding.
    auto blocks = [&](int bm, int bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    // Long K and few 256x128 tiles: slices of K until the chip is full, when the partial planes (written and read
    // once more: 4 * slices / K bytes per flop) stay small next to the product.  Measured for 4096 x 14336: 102 -> 55 us
    // at 256 rows (8 slices), 115 -> 83 us at 512 (4), 236 -> 142 us at 1024 (2); no gain for K = 4096.
    if (m > 128 && k >= 8192 && n % 4 == 0 && aligned(y, out == kOutF32 ? 16 : (out == kOutBf16 ? 8 : 4))) {
        const int64_t b0 = blocks(256, 128), kt = k / kBK;
        for (int slices = 8; slices >= 2; slices >>= 1)
            if (b0 * slices <= 256 && kt % slices == 0 && (kt / slices) % 4 == 0 &&
                static_cast<size_t>(slices) * m * n <= (size_t{8} << 20))
                return kTileSliced + slices;
    }
    int tile = 3;
    if (m > 128 && k % (kBK * 2) == 0 && blocks(256, 256) >= 192) tile = 4;
    else if (m > 128 && blocks(256, 128) >= 192) tile = 0;
    else if (blocks(128, 128) >= 192) tile = 1;
    else if (blocks(128, 64) >= 192) tile = 2;
    return tile;
}

}  // namespace lhip

using namespace lhip;

extern "C" {

lhip_status lhip_q8_0_matmul_bf16_cfg(const void *planar_dev, const void *x_dev, void *y_dev, int64_t m, int64_t n,
                                      int64_t k, int tile, void *stream) {
    return gemm_dispatch(planar_dev, x_dev, y_dev, m, n, k, tile, kOutBf16, stream);
}

lhip_status lhip_q8_0_matmul_bf16(const void *planar_dev, const void *x_dev, void *y_dev, int64_t m, int64_t n,
                                  int64_t k, void *stream) {
    return gemm_dispatch(planar_dev, x_dev, y_dev, m, n, k, gemm_auto_tile(m, n, k, kOutBf16, y_dev), kOutBf16, stream);
}

lhip_status lhip_q8_0_matmul_bf16_f32out(const void *planar_dev, const void *x_dev, float *y_dev, int64_t m, int64_t n,
                                         int64_t k, void *stream) {
    return gemm_dispatch(planar_dev, x_dev, y_dev, m, n, k, gemm_auto_tile(m, n, k, kOutF32, y_dev), kOutF32, stream);
}

lhip_status lhip_q8_0_matmul_bf16_swiglu(const void *planar_dev, const void *x_dev, void *out_dev, int64_t m, int64_t n,
                                         int64_t k, void *stream) {
    return gemm_dispatch(planar_dev, x_dev, out_dev, m, n, k, gemm_auto_tile(m, n, k, kOutSwiglu, out_dev), kOutSwiglu, stream);
}

}  // extern "C"
