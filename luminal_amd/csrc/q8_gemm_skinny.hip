// Q8_0 weights x activations for few activation rows (short prompts, small batches; up to 128 rows per pass).
//
// With so few activation rows the product is bound by streaming the weights, not by the matrix cores, and the
// 128/256-row tiles of q8_gemm.hip leave most of the chip idle.  Here a workgroup owns a strip of 128 weight rows
// (and, when the strips alone would not fill the chip, a slice of K) and streams it from HBM straight into
// registers in matrix-core operand order:
//
//   * eight compute waves of 16 weight rows each (seven, i.e. strips of 112 rows, where that cuts N into a number
//     of workgroups that fills the 256 CUs better: sk_plan).  The int8 codes go to the matrix cores as they are (an int8 is
//     exact in bf16); an MFMA step (v_mfma_f32_16x16x32_bf16) is one Q8_0 block, a lane supplies eight of its
//     codes, and the block's scale multiplies the f32 block sum: acc += d * sum, the arithmetic of the matvec
//     kernels (crates/luminal_cuda/src/quantized.rs:93-96).  Eight groups of 64 k per row block are in flight per
//     wave, reloaded in place as they are consumed.
//   * four more waves ("loaders") stage the activations for all the compute waves: (16*MT) x (64*G) tiles of x go
//     through their registers into one of three LDS buffers, two tiles ahead, one barrier per tile.  The compute
//     waves never wait for an activation load, so their in-order load counter only ever sees the weight stream.
//     In LDS a tile is G panels of 64 k, a row of a panel 128 bytes at pitch 160 (free of bank conflicts for the
//     16-lane x 4-group operand reads).
//   * activations are bf16 (the prefill GEMM: one plane per tile), or f32 / f16 held as three / two bf16 limbs
//     whose sum is the value exactly (the f32 / f16 matmul operators for several rows: one plane and one chained
//     MFMA per limb).  Every product is exact; the only roundings are those of the f32 additions.
//
// K slices write f32 partial tiles to a scratch array owned by the library (one per device, shared by every
// call on it) and a second kernel adds them in slice order and applies the output form, so results do not depend
// on timing.
#include <hip/hip_fp16.h>

#include <type_traits>
#include <utility>

#include <algorithm>

#include "common.h"

namespace lhip {

typedef __bf16 sk_bf16x8 __attribute__((ext_vector_type(8)));
typedef float sk_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t sk_u32x4 __attribute__((ext_vector_type(4)));

enum { kSkOutBf16 = 0, kSkOutF32 = 1, kSkOutSwiglu = 2, kSkOutPartial = 3, kSkOutF16 = 4 };  // first three as in q8_gemm.hip

constexpr int kSkRows = 128;    // weight rows per workgroup of eight compute waves (seven: 112)
constexpr int kSkPitch = 160;   // bytes per activation row of a panel in LDS
constexpr int kSkStages = 3;    // LDS buffers
constexpr int kSkUnit = 512;     // K slices are whole multiples of this (eight groups of 64 k)
constexpr size_t kSkScratchFloats = size_t{8} << 20;  // 32 MiB of partial sums

static __device__ __align__(256) float sk_scratch[kSkScratchFloats];

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), expanded at compile time (a pragma gives up on
// bodies this large, and register arrays indexed at run time land in scratch memory).
template <class F, int... Is>
__device__ __forceinline__ void sk_static_for_impl(F &&f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void sk_static_for(F &&f) {
    sk_static_for_impl(static_cast<F &&>(f), std::make_integer_sequence<int, N>{});
}

// NL = bf16 planes of an activation tile (1: bf16 activations, 2: f16, 3: f32).  64 k per panel row.
template <int MT, int NL>
struct SkShape {
    static_assert(NL >= 1 && NL <= 3 && (MT <= 4 || NL == 1), "three or two planes per tile: at most 64 activation rows");
    static constexpr int G = MT >= 4 ? 1 : (MT == 2 ? 2 : 4);  // groups per activation tile; a slice is an even number of tiles
    static constexpr int PANEL = 16 * MT * kSkPitch;
    static constexpr int PLANE = G * PANEL;
    static constexpr int STAGE = NL * PLANE;
    static constexpr int CHUNKS = 16 * MT * G * 8;             // pieces of 8 k per tile
    static constexpr int CH = CHUNKS / 256;                    // per loader thread
    static_assert(CHUNKS % 256 == 0 && 8 % G == 0, "tile split");
    static constexpr size_t LDS = static_cast<size_t>(kSkStages) * STAGE;
};

// Two f32 -> NL packed bf16 pairs whose sums are the two values exactly: limb[0] the bf16 roundings, limb[1]
// the roundings of what that left, limb[2] of what is left then (8 + 8 + 8 significant bits cover an f32, 8 + 8 the
// 11 of a widened f16).
template <int NL>
__device__ __forceinline__ void sk_split2(float a, float b, uint32_t (&limb)[NL]) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int l = 0; l < NL; ++l) {
        const bf16x2 h = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
        limb[l] = __builtin_bit_cast(uint32_t, h);
        a -= __uint_as_float(limb[l] << 16);
        b -= __uint_as_float(limb[l] & 0xffff0000u);
    }
}

// One output form for four consecutive weight rows n .. n+3 of activation row m.
template <int OUT>
__device__ __forceinline__ void sk_store4(void *y, float *part, int split, int M, int N, int m, int n, sk_f32x4 v) {
    if constexpr (OUT == kSkOutPartial) {
        *reinterpret_cast<sk_f32x4 *>(part + (static_cast<size_t>(split) * M + m) * N + n) = v;
    } else if constexpr (OUT == kSkOutF32) {
        *reinterpret_cast<sk_f32x4 *>(static_cast<float *>(y) + static_cast<size_t>(m) * N + n) = v;
    } else if constexpr (OUT == kSkOutBf16) {
        typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
        const bf16x4 w = {static_cast<__bf16>(v[0]), static_cast<__bf16>(v[1]), static_cast<__bf16>(v[2]),
                          static_cast<__bf16>(v[3])};
        *reinterpret_cast<bf16x4 *>(static_cast<__bf16 *>(y) + static_cast<size_t>(m) * N + n) = w;
    } else if constexpr (OUT == kSkOutF16) {
        typedef _Float16 f16x4 __attribute__((ext_vector_type(4)));
        const f16x4 w = {static_cast<_Float16>(v[0]), static_cast<_Float16>(v[1]), static_cast<_Float16>(v[2]),
                         static_cast<_Float16>(v[3])};
        *reinterpret_cast<f16x4 *>(static_cast<_Float16 *>(y) + static_cast<size_t>(m) * N + n) = w;
    } else {  // rows are (gate, up) pairs
        typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
        const bf16x2 w = {static_cast<__bf16>(swiglu_value(v[0], v[1])), static_cast<__bf16>(swiglu_value(v[2], v[3]))};
        *reinterpret_cast<bf16x2 *>(static_cast<__bf16 *>(y) + static_cast<size_t>(m) * (N >> 1) + (n >> 1)) = w;
    }
}

// grid (strips of 16 * CW weight rows, K slices, passes of 16 * MT activation rows); CW compute waves of 16 weight
// rows and four loader waves.  K % 512 == 0, N % 4 == 0.
// A slice is `slice_groups` groups of 64 k (a multiple of 8); the last may be shorter (also a multiple of 8).
// RING = groups in flight per wave; a slice is a multiple of RING groups.
// XT = __bf16, __half or float: the loaders write x as NL = 1, 2 or 3 bf16 planes per tile whose sum is the value
// exactly (an f16 has 11 significant bits, which two limbs hold; an f32's 24 take three).
// CW = compute waves: 8, or 7 where strips of 112 weight rows cut N into a number of workgroups that fills the chip
// (14336 rows are 112 strips of 128 but 128 of 112: with two K slices 224 or 256 workgroups for the 256 CUs).
template <int MT, int OUT, int RING, typename XT, int CW = 8>
__global__ __launch_bounds__((CW + 4) * 64) void q8_gemm_skinny_kernel(const int8_t *__restrict__ qs, const __half *__restrict__ ds,
                                                             const XT *__restrict__ x, void *__restrict__ y,
                                                             float *__restrict__ part, int M, int N, int K,
                                                             int slice_groups) {
    constexpr int NL = sizeof(XT) == 4 ? 3 : (std::is_same<XT, __bf16>::value ? 1 : 2);  // bf16 limbs of an activation
    using S = SkShape<MT, NL>;
    constexpr int G = S::G;
    static_assert(CW == 8 || CW == 7, "compute waves");
    extern __shared__ __attribute__((aligned(16))) unsigned char sk_lds[];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int strip = blockIdx.x, split = blockIdx.y;
    const int g_begin = split * slice_groups;
    const int n_groups = min(slice_groups, (K >> 6) - g_begin);
    const int n_tiles = n_groups / G;
    // blockIdx.z takes 16 * MT activation rows of the M in all (one launch streams the weights once per pass)
    const int m_base = static_cast<int>(blockIdx.z) * (16 * MT);
    // With few activation rows every strip starts its walk over K at a different place (a whole number of rings):
    // the strips advance at the same pace and would otherwise all ask the same memory channels for the same k at
    // the same time (measured: 39 -> 36 us for 28672 x 4096 at 16 rows).  With many rows the strips reading the
    // same activation tile at the same time is worth more (57 against 64 us at 128 rows).
    const int rot = MT <= 2 ? (strip % (n_groups / RING)) * RING : 0;

    if (wave >= CW) {
        // ---------------- loaders: x tiles -> LDS, two tiles ahead of the compute waves
        const int lt = tid - CW * 64;
        const XT *src[S::CH];
        int dst[S::CH];
#pragma unroll
        for (int i = 0; i < S::CH; ++i) {
            const int c = lt + i * 256;
            const int m = c / (G * 8), j = c % (G * 8);
            const int panel = j >> 3, jj = j & 7;
            src[i] = x + static_cast<size_t>(min(m_base + m, M - 1)) * K + (static_cast<size_t>(g_begin) + panel) * 64 + jj * 8;
            dst[i] = panel * S::PANEL + m * kSkPitch + jj * 16;  // pieces in natural order: an MFMA step is one Q8_0 block
        }
        constexpr int XL = sizeof(XT) == 4 ? 2 : 1;  // 16-byte loads per piece of 8 k
        sk_u32x4 xr[2][S::CH][XL];
        auto load_x = [&](int slot, int t) __attribute__((always_inline)) {
            int tt = min(t, n_tiles - 1) + rot / G;  // past the end: re-read, never used
            if (tt >= n_tiles) tt -= n_tiles;
            const size_t off = static_cast<size_t>(tt) * (G * 64);
#pragma unroll
            for (int i = 0; i < S::CH; ++i)
#pragma unroll
                for (int l = 0; l < XL; ++l)
                    xr[slot][i][l] = reinterpret_cast<const sk_u32x4 *>(src[i] + off)[l];
        };
        auto store_x = [&](int slot, int stage) __attribute__((always_inline)) {
            unsigned char *base = sk_lds + stage * S::STAGE;
#pragma unroll
            for (int i = 0; i < S::CH; ++i) {
                if constexpr (NL == 1) {
                    *reinterpret_cast<sk_u32x4 *>(base + dst[i]) = xr[slot][i][0];
                } else {
                    float v[8];
                    if constexpr (sizeof(XT) == 4) {
#pragma unroll
                        for (int e = 0; e < 8; ++e) v[e] = __uint_as_float(xr[slot][i][e >> 2][e & 3]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 8; ++e)
                            v[e] = __half2float(__ushort_as_half(static_cast<unsigned short>(xr[slot][i][0][e >> 1] >> (16 * (e & 1)))));
                    }
                    constexpr int NLS = NL;
                    sk_u32x4 limbs[NLS];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        uint32_t l3[NLS];
                        sk_split2<NLS>(v[2 * e], v[2 * e + 1], l3);
#pragma unroll
                        for (int l = 0; l < NLS; ++l) limbs[l][e] = l3[l];
                    }
#pragma unroll
                    for (int l = 0; l < NLS; ++l) *reinterpret_cast<sk_u32x4 *>(base + l * S::PLANE + dst[i]) = limbs[l];
                }
            }
        };
        load_x(0, 0);
        load_x(1, 1);
        store_x(0, 0);
        load_x(0, 2);
        store_x(1, 1);
        load_x(1, 3);
        __syncthreads();
        int stage = 2;  // buffer of tile t + 2
        for (int t = 0; t < n_tiles; t += 2) {  // two tiles per trip: no branch between them, so the counted waits
                                                // are exact (the loads of a slot are two tiles old when it is stored)
            // The fences keep the arithmetic on one slot's values (the limb split) behind the barrier before it:
            // moved up, it waits for loads that are only one tile old instead of two.
            store_x(0, stage);  // tile t + 2 (a buffer last read for tile t - 1)
            load_x(0, t + 4);
            stage = stage == 2 ? 0 : stage + 1;
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
            store_x(1, stage);  // tile t + 3
            load_x(1, t + 5);
            stage = stage == 2 ? 0 : stage + 1;
            __syncthreads();
            __builtin_amdgcn_sched_barrier(0);
        }
        return;
    }

    // ---------------- compute waves
    const int r = lane & 15, g = lane >> 4;
    const int n0 = strip * (CW * 16) + wave * 16;

    {
        // The codes go to the matrix cores as they are (an int8 is exact in bf16) and the block scale is applied to
        // the f32 sum of each block, as the matvec kernels do; only an f32 / f16 x is split, into NL bf16 limbs.
        // An MFMA step is one Q8_0 block and a lane supplies eight of its codes; the x pieces lie in natural
        // order in LDS and a lane reads the one that matches its codes.  Two ways to get the codes:
        //  - WIDE (few activation rows, where the weight stream is what bounds the kernel): lane (r, g) requests the
        //    16 codes 16g .. 16g+15 of a group of two blocks (one 16-byte load: a row's 64 bytes are contiguous over
        //    its four lanes) and a swap between the wave's halves (lanes l and l + 32, i.e. g and g + 2) leaves it
        //    with eight codes of each block: codes 0-7, 16-23, 8-15, 24-31 for g = 0 .. 3;
        //  - otherwise two 8-byte loads, codes 8g .. 8g+7 of each block (from 64 rows on: measured 3-8 % faster
        //    there for f32 activations than the wide loads, 3-5 % slower for f16; one choice for both types keeps
        //    the order of additions, and so the f16 result, equal to the f32 form's).
        // Per block and column block NL chained MFMAs (x2, x1, x0 for f32; exact products, 96 f32 additions; an
        // f16's x2 is zero and has no MFMA, which leaves every sum as it is) and four fmas acc += d * sum.
        constexpr bool WIDE = MT <= 2;
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        const int n_rounds = n_groups >> 2;
        const int8_t *a_ptr = qs + static_cast<size_t>(min(n0 + r, N - 1)) * K + static_cast<size_t>(g_begin) * 64 + (WIDE ? 16 : 8) * g;
        const int x_lane = r * kSkPitch + (WIDE ? (g & 1) * 32 + (g >> 1) * 16 : g * 16);  // the x piece of this lane's codes
        const __half *d_ptr[4];  // scales of the four weight rows this lane accumulates: n0 + 4g + v
#pragma unroll
        for (int v = 0; v < 4; ++v)
            d_ptr[v] = ds + static_cast<size_t>(min(n0 + 4 * g + v, N - 1)) * (K >> 5) + static_cast<size_t>(g_begin) * 2;
        sk_u32x4 a_reg[RING];
        sk_u32x4 d_reg[RING / 4][4];
        auto load_a = [&](int u, int group) __attribute__((always_inline)) {
            int gg = min(group, n_groups - 1) + rot;
            if (gg >= n_groups) gg -= n_groups;
            if constexpr (WIDE) {
                a_reg[u] = *reinterpret_cast<const sk_u32x4 *>(a_ptr + static_cast<size_t>(gg) * 64);
            } else {
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    const u32x2 v = *reinterpret_cast<const u32x2 *>(a_ptr + static_cast<size_t>(gg) * 64 + 32 * b);
                    a_reg[u][2 * b] = v[0];
                    a_reg[u][2 * b + 1] = v[1];
                }
            }
        };
        auto load_d = [&](int set, int round) __attribute__((always_inline)) {
            int rr = min(round, n_rounds - 1) + rot / 4;
            if (rr >= n_rounds) rr -= n_rounds;
#pragma unroll
            for (int v = 0; v < 4; ++v) d_reg[set][v] = *reinterpret_cast<const sk_u32x4 *>(d_ptr[v] + static_cast<size_t>(rr) * 8);
        };
        // same order of requests in the prologue as in the loop: a0 .. a3, d0, a4 .. a7, d1
#pragma unroll
        for (int u = 0; u < RING; ++u) {
            load_a(u, u);
            if ((u & 3) == 3) load_d(u >> 2, u >> 2);
            __builtin_amdgcn_sched_barrier(0);  // or the requests are regrouped and the loop's counted waits follow
        }
        sk_f32x4 acc[MT];
#pragma unroll
        for (int cb = 0; cb < MT; ++cb) acc[cb] = sk_f32x4{0.f, 0.f, 0.f, 0.f};

        constexpr int UNITS = 2 * MT;  // (block, column block) pairs of a group
        auto b_read = [&](const unsigned char *xb, int i, int limb) __attribute__((always_inline)) {
            return *reinterpret_cast<const sk_bf16x8 *>(xb + limb * S::PLANE + (i % MT) * 16 * kSkPitch + (i / MT) * 64);
        };
        const unsigned char *xb_cur = sk_lds + x_lane;
        __syncthreads();  // tiles 0 and 1 are staged
        // The x operands of a unit are requested two units ahead (into the next group's tile too, which is staged
        // by then) in four rotating register sets, three of them live at a time; the fence keeps the request where
        // it is, or the reads sink to their use and every unit waits a full LDS round trip.
        sk_bf16x8 bq[4][NL];
#pragma unroll
        for (int l = 0; l < NL; ++l) {
            bq[0][l] = b_read(xb_cur, 0, l);
            bq[1][l] = UNITS > 1 ? b_read(xb_cur, 1 % UNITS, l) : b_read(xb_cur, 0, l);
        }
        int stage = 0;
        int R = 0;
        do {  // a slice is never empty: no guard, so the requests above stay where the fences put them
            sk_static_for<RING>([&](auto uc) __attribute__((always_inline)) {
                constexpr int u = decltype(uc)::value;
                constexpr bool tile_ends = (u + 1) % G == 0;
                const int gl = R * 4 + u;
                const int stage_next = tile_ends ? (stage == 2 ? 0 : stage + 1) : stage;
                const unsigned char *xb_next = sk_lds + stage_next * S::STAGE + ((u + 1) % G) * S::PANEL + x_lane;
                // the eight codes of each block as bf16
                asm volatile("" : "+v"(a_reg[u]));
                u32x2 a_blk[2];  // after the swap: dwords 0, 1 are codes of the group's first block, 2, 3 of its second
                if constexpr (WIDE) {
                    const auto s02 = __builtin_amdgcn_permlane32_swap(a_reg[u][0], a_reg[u][2], false, false);
                    const auto s13 = __builtin_amdgcn_permlane32_swap(a_reg[u][1], a_reg[u][3], false, false);
                    a_blk[0] = u32x2{s02[0], s13[0]};
                    a_blk[1] = u32x2{s02[1], s13[1]};
                } else {
                    a_blk[0] = u32x2{a_reg[u][0], a_reg[u][1]};
                    a_blk[1] = u32x2{a_reg[u][2], a_reg[u][3]};
                }
                sk_u32x4 a_bf[2];
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const uint32_t w = a_blk[b][e >> 1];
                        const float lo = static_cast<float>(static_cast<signed char>(w >> (16 * (e & 1))));
                        const float hi = static_cast<float>(static_cast<signed char>(w >> (16 * (e & 1) + 8)));
                        a_bf[b][e] = (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
                    }
                float dv[2][4];
#pragma unroll
                for (int b = 0; b < 2; ++b)
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        dv[b][v] = __half2float(__ushort_as_half(static_cast<unsigned short>(d_reg[u >> 2][v][u & 3] >> (16 * b))));
                load_a(u, gl + RING);
                sk_static_for<UNITS>([&](auto ic) __attribute__((always_inline)) {
                    constexpr int i = decltype(ic)::value;
                    constexpr int U = u * UNITS + i;  // RING * UNITS is a multiple of four: the sets rotate statically
                    constexpr int ahead = i + 2;
#pragma unroll
                    for (int l = 0; l < NL; ++l)
                        bq[(U + 2) % 4][l] = ahead < UNITS ? b_read(xb_cur, ahead, l) : b_read(xb_next, ahead - UNITS, l);
                    __builtin_amdgcn_sched_barrier(0);
                    const sk_bf16x8 a = __builtin_bit_cast(sk_bf16x8, a_bf[i / MT]);
                    sk_f32x4 t = sk_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                    for (int l = NL - 1; l >= 0; --l)
                        t = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, bq[U % 4][l], t, 0, 0, 0);
#pragma unroll
                    for (int v = 0; v < 4; ++v) acc[i % MT][v] = fmaf(dv[i / MT][v], t[v], acc[i % MT][v]);
                });
                // a set of scales is requested again once its last group has read it (requested earlier, the load
                // gets other registers and a copy at the end of the trip that waits for every load in flight)
                if constexpr ((u & 3) == 3) load_d(u >> 2, R + RING / 4 + (u >> 2));
                xb_cur = xb_next;
                if constexpr (tile_ends) {
                    stage = stage_next;
                    __syncthreads();
                }
            });
        } while ((R += RING / 4) < n_rounds);
        const int n = n0 + 4 * g;
        if (n < N) {
#pragma unroll
            for (int cb = 0; cb < MT; ++cb) {
                const int m = m_base + cb * 16 + r;
                if (m < M) sk_store4<OUT>(y, part, split, M, N, m, n, acc[cb]);
            }
        }
        return;
    }

}

// Sum of the K slices in slice order, then the output form.  One thread per four weight rows.  ldy = row pitch of y
// in weight rows (N, or more when the planes are the trailing columns of a wider output).
template <int OUT>
__global__ __launch_bounds__(256) void q8_gemm_skinny_reduce_kernel(const float *__restrict__ part, void *__restrict__ y,
                                                                    int M, int N, int splits, int ldy) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    const size_t quads = static_cast<size_t>(M) * (N >> 2);
    if (i >= quads) return;
    const size_t plane = static_cast<size_t>(M) * N;
    sk_f32x4 v = *reinterpret_cast<const sk_f32x4 *>(part + 4 * i);
    for (int s = 1; s < splits; ++s) v += *reinterpret_cast<const sk_f32x4 *>(part + s * plane + 4 * i);
    const int m = static_cast<int>(i / (N >> 2)), n = static_cast<int>(i % (N >> 2)) * 4;
    sk_store4<OUT>(y, nullptr, 0, M, ldy, m, n, v);
}

// Scratch address per device (a __device__ array has one copy, at its own address, on every device).
static float *sk_scratch_ptr() {
    static float *ptrs[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
    float *p = __atomic_load_n(&ptrs[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        if (hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(sk_scratch)) != hipSuccess) return nullptr;
        __atomic_store_n(&ptrs[dev], p, __ATOMIC_RELEASE);
    }
    return p;
}

float *q8_gemm_scratch(size_t *floats) {
    *floats = kSkScratchFloats;
    return sk_scratch_ptr();
}

// Adds `slices` f32 planes of (m, n) in order and writes the output form (as the GEMM epilogues: bf16, f32, f16, SwiGLU).
lhip_status q8_gemm_reduce_launch(const float *part, void *y, int m, int n, int slices, int out, hipStream_t s, int ldy = 0) {
    if (ldy <= 0) ldy = n;
    const size_t quads = static_cast<size_t>(m) * (n >> 2);
    const dim3 grid(static_cast<unsigned>((quads + 255) / 256));
    switch (out) {
        case kSkOutBf16: hipLaunchKernelGGL(q8_gemm_skinny_reduce_kernel<kSkOutBf16>, grid, dim3(256), 0, s, part, y, m, n, slices, ldy); break;
        case kSkOutF32: hipLaunchKernelGGL(q8_gemm_skinny_reduce_kernel<kSkOutF32>, grid, dim3(256), 0, s, part, y, m, n, slices, ldy); break;
        case kSkOutF16: hipLaunchKernelGGL(q8_gemm_skinny_reduce_kernel<kSkOutF16>, grid, dim3(256), 0, s, part, y, m, n, slices, ldy); break;
        default: hipLaunchKernelGGL(q8_gemm_skinny_reduce_kernel<kSkOutSwiglu>, grid, dim3(256), 0, s, part, y, m, n, slices, ldy); break;
    }
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

// K slices for a product: enough workgroups for the 256 CUs, slices of whole 512-k units, partial sums within the
// scratch array.
static int sk_splits_for(int strips, int m, int n, int k, size_t room) {
    const int units = k / kSkUnit, passes = (m + 127) / 128;
    int s = 256 / (strips * passes);
    if (s < 1) s = 1;
    if (s > units) s = units;
    while (s > 1 && static_cast<size_t>(s) * m * n > room) --s;
    const int per = (units + s - 1) / s;
    return (units + per - 1) / per;
}

// Compute waves per workgroup (strips of 16 rows each) for `splits` K slices (0: the slices are chosen with them).
// A workgroup's time goes with the weights it streams (rows x its share of K) and the launch takes as many rounds of
// 256 workgroups as it has workgroups: eight waves unless seven make that product smaller.
struct SkPlan {
    int cw, splits;
};
static SkPlan sk_plan(int m, int n, int k, size_t room, int splits = 0) {
    const int units = k / kSkUnit, passes = (m + 127) / 128;
    SkPlan best{8, 1};
    long best_cost = -1;
    for (int cw = 8; cw >= 7; --cw) {
        const int strips = (n + cw * 16 - 1) / (cw * 16);
        int s = splits > 0 ? (splits > units ? units : splits) : sk_splits_for(strips, m, n, k, room);
        const int per = (units + s - 1) / s;
        s = (units + per - 1) / per;  // no empty slice
        const long rounds = (static_cast<long>(strips) * s * passes + 255) / 256;
        const long cost = rounds * cw * per;
        if (best_cost < 0 || cost < best_cost) {
            best_cost = cost;
            best = SkPlan{cw, s};
        }
    }
    return best;
}

// The plan for `room` floats of partial planes: the one the library's own array allows wherever it fits (so that a
// caller's workspace of the recommended size gets the plain call's plan and bits), else the best within `room`.
static SkPlan sk_plan_within(int m, int n, int k, size_t room, int splits = 0) {
    const SkPlan plan = sk_plan(m, n, k, kSkScratchFloats, splits);
    if (plan.splits == 1 || static_cast<size_t>(plan.splits) * m * n <= room) return plan;
    return sk_plan(m, n, k, room, splits);
}

int q8_gemm_skinny_splits(int m, int n, int k, size_t room) { return sk_plan_within(m, n, k, room).splits; }

constexpr int kSkMaxRows = 128 * 64;  // passes are the grid's z extent

bool q8_gemm_skinny_supports(int m, int n, int k, int out, const void *y) {
    return m >= 1 && m <= kSkMaxRows && k % kSkUnit == 0 && n % 4 == 0 && aligned(y, out == kSkOutF32 ? 16 : (out == kSkOutBf16 ? 8 : 4));
}

template <typename XT>
constexpr int sk_limbs() { return sizeof(XT) == 4 ? 3 : (std::is_same<XT, __bf16>::value ? 1 : 2); }

template <int MT, int OUT, typename XT, int CW = 8>
static lhip_status sk_launch_t(const int8_t *qs, const __half *ds, const XT *x, void *y, float *part, int m, int n,
                               int k, int splits, int passes, hipStream_t s) {
    auto kern = q8_gemm_skinny_kernel<MT, OUT, 8, XT, CW>;
    constexpr size_t lds_bytes = SkShape<MT, sk_limbs<XT>()>::LDS;
    static LdsOptIn opt;  // opting in to more than 64 KiB of dynamic LDS is a per-function attribute
    if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(kern), lds_bytes)) return st;
    const int units = k / kSkUnit, per = (units + splits - 1) / splits;
    hipLaunchKernelGGL(kern,
                       dim3(static_cast<unsigned>((n + CW * 16 - 1) / (CW * 16)), static_cast<unsigned>(splits),
                            static_cast<unsigned>(passes)),
                       dim3((CW + 4) * 64), lds_bytes, s, qs, ds, x, y, part, m, n, k, per * 8);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

// bf16 activations: passes of 16 * MT rows (one plane per tile leaves room for 128-row tiles)
template <int MT, int CW>
static lhip_status sk_launch_mt(int out, const int8_t *qs, const __half *ds, const __bf16 *x, void *y, float *part, int m,
                                int n, int k, int splits, hipStream_t s) {
    const int passes = (m + 16 * MT - 1) / (16 * MT);
    if (splits > 1) return sk_launch_t<MT, kSkOutPartial, __bf16, CW>(qs, ds, x, y, part, m, n, k, splits, passes, s);
    switch (out) {
        case kSkOutBf16: return sk_launch_t<MT, kSkOutBf16, __bf16, CW>(qs, ds, x, y, part, m, n, k, 1, passes, s);
        case kSkOutF32: return sk_launch_t<MT, kSkOutF32, __bf16, CW>(qs, ds, x, y, part, m, n, k, 1, passes, s);
        default: return sk_launch_t<MT, kSkOutSwiglu, __bf16, CW>(qs, ds, x, y, part, m, n, k, 1, passes, s);
    }
}
template <int CW>
static lhip_status sk_launch_rows(int out, const int8_t *qs, const __half *ds, const __bf16 *x, void *y, float *part, int m,
                                  int n, int k, int splits, hipStream_t s) {
    if (m <= 16) return sk_launch_mt<1, CW>(out, qs, ds, x, y, part, m, n, k, splits, s);
    if (m <= 32) return sk_launch_mt<2, CW>(out, qs, ds, x, y, part, m, n, k, splits, s);
    if (m <= 64) return sk_launch_mt<4, CW>(out, qs, ds, x, y, part, m, n, k, splits, s);
    return sk_launch_mt<8, CW>(out, qs, ds, x, y, part, m, n, k, splits, s);
}

// `splits` = 0: chosen here.  The caller has checked q8_gemm_skinny_supports.
// `own_workspace`: partial planes go to `ws` (ws_floats floats; none: no K slices) and the library's scratch array is
// not touched.
lhip_status q8_gemm_skinny_launch(const int8_t *qs, const __half *ds, const void *x_bf16, void *y, int m, int n, int k,
                                  int out, int splits, hipStream_t s, bool own_workspace, float *ws, size_t ws_floats) {
    const size_t room = own_workspace ? (ws ? std::min(ws_floats, kSkScratchFloats) : 0) : kSkScratchFloats;
    const SkPlan plan = sk_plan_within(m, n, k, room, splits);
    splits = plan.splits;
    float *part = nullptr;
    if (splits > 1) {
        if (static_cast<size_t>(splits) * m * n > room) return LHIP_ERR_UNSUPPORTED;
        part = own_workspace ? ws : sk_scratch_ptr();
        if (!part) return LHIP_ERR_HIP;
    }
    const __bf16 *x = static_cast<const __bf16 *>(x_bf16);
    const lhip_status st = plan.cw == 7 ? sk_launch_rows<7>(out, qs, ds, x, y, part, m, n, k, splits, s)
                                        : sk_launch_rows<8>(out, qs, ds, x, y, part, m, n, k, splits, s);
    if (st != LHIP_OK || splits == 1) return st;
    return q8_gemm_reduce_launch(part, y, m, n, splits, out, s);
}

// ---- the f32-accurate ("split") form behind the f32 / f16 operators

// m rows in all; passes of 64 rows (one: the tile height follows m).
template <typename XT, int OUT>
static lhip_status sk_launch_split_rows(const int8_t *qs, const __half *ds, const XT *x, void *y, float *part, int m, int n,
                                        int k, int splits, int passes, hipStream_t s) {
    if (splits > 1) {
        if (passes == 1 && m <= 16) return sk_launch_t<1, kSkOutPartial, XT>(qs, ds, x, y, part, m, n, k, splits, 1, s);
        if (passes == 1 && m <= 32) return sk_launch_t<2, kSkOutPartial, XT>(qs, ds, x, y, part, m, n, k, splits, 1, s);
        return sk_launch_t<4, kSkOutPartial, XT>(qs, ds, x, y, part, m, n, k, splits, passes, s);
    }
    if (passes == 1 && m <= 16) return sk_launch_t<1, OUT, XT>(qs, ds, x, y, part, m, n, k, 1, 1, s);
    if (passes == 1 && m <= 32) return sk_launch_t<2, OUT, XT>(qs, ds, x, y, part, m, n, k, 1, 1, s);
    return sk_launch_t<4, OUT, XT>(qs, ds, x, y, part, m, n, k, 1, passes, s);
}

bool q8_gemm_split_supports(int n, int k, const void *x, const void *y, bool f16) {
    return k % kSkUnit == 0 && n % 4 == 0 && aligned(x, 16) && aligned(y, f16 ? 8 : 16);
}

// y (m, N) = x (m, K) W^T for f32 or f16 activations and results, any m: passes of 64 rows, each streaming the
// weights once, as blockIdx.z of one launch; K is sliced only while strips x passes leave the chip unfilled.  At most
// kSkMaxPasses passes per launch (the grid's z extent).  `splits` = 0: chosen here.  The caller has checked
// q8_gemm_split_supports.
constexpr int64_t kSkMaxPasses = 1024;

// K slices of one chunk of mc rows: as many as fill the chip, within `room` floats of partial planes.
static int split_slices(int mc, int n, int k, int splits_arg, size_t room) {
    const int units = k / kSkUnit, strips = (n + kSkRows - 1) / kSkRows, passes = (mc + 63) / 64;
    int splits = splits_arg > 0 ? splits_arg : 256 / (strips * passes);
    if (splits < 1) splits = 1;
    if (splits > units) splits = units;
    while (splits > 1 && static_cast<size_t>(splits) * mc * n > room) --splits;
    const int per = (units + splits - 1) / splits;
    return (units + per - 1) / per;  // no empty slice
}

// Floats of partial planes the plan of q8_gemm_split_launch uses for (m, n, k) when it has the library's own
// scratch array to itself: what a caller's workspace must hold for the same plan (and the same bits).
size_t q8_gemm_split_workspace_floats(int64_t m, int n, int k) {
    size_t most = 0;
    for (int64_t m0 = 0; m0 < m; m0 += 64 * kSkMaxPasses) {
        const int mc = static_cast<int>(m - m0 < 64 * kSkMaxPasses ? m - m0 : 64 * kSkMaxPasses);
        const int splits = split_slices(mc, n, k, 0, kSkScratchFloats);
        if (splits > 1) most = std::max(most, static_cast<size_t>(splits) * mc * n);
    }
    return most;
}

// `own_workspace`: partial planes go to `ws` (ws_floats floats; none: no K slices) and the library's scratch array
// is not touched, so calls may overlap in time.
lhip_status q8_gemm_split_launch(const int8_t *qs, const __half *ds, const void *x, void *y, int64_t m, int n, int k,
                                 bool f16, int splits_arg, hipStream_t s, bool own_workspace, float *ws, size_t ws_floats) {
    const size_t esz = f16 ? 2 : 4;
    for (int64_t m0 = 0; m0 < m; m0 += 64 * kSkMaxPasses) {
        const int mc = static_cast<int>(m - m0 < 64 * kSkMaxPasses ? m - m0 : 64 * kSkMaxPasses);
        const int passes = (mc + 63) / 64;
        const size_t room = own_workspace ? (ws ? std::min(ws_floats, kSkScratchFloats) : 0) : kSkScratchFloats;
        const int splits = split_slices(mc, n, k, splits_arg, room);
        float *part = nullptr;
        if (splits > 1) {
            part = own_workspace ? ws : sk_scratch_ptr();
            if (!part) return LHIP_ERR_HIP;
        }
        const auto *xc = static_cast<const unsigned char *>(x) + static_cast<size_t>(m0) * k * esz;
        auto *yc = static_cast<unsigned char *>(y) + static_cast<size_t>(m0) * n * esz;
        lhip_status st = f16 ? sk_launch_split_rows<__half, kSkOutF16>(qs, ds, reinterpret_cast<const __half *>(xc), yc, part,
                                                                       mc, n, k, splits, passes, s)
                             : sk_launch_split_rows<float, kSkOutF32>(qs, ds, reinterpret_cast<const float *>(xc), yc, part,
                                                                      mc, n, k, splits, passes, s);
        if (st != LHIP_OK) return st;
        if (splits > 1)
            if (lhip_status r = q8_gemm_reduce_launch(part, yc, mc, n, splits, f16 ? kSkOutF16 : kSkOutF32, s)) return r;
    }
    return LHIP_OK;
}

}  // namespace lhip
