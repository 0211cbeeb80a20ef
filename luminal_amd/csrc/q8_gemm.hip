// Q8_0 GEMM for prefill:  Y[M][N] = X[M][K] . W[N][K]^T, bf16 activations,
// f32 accumulation on the matrix cores, bf16 output.
//
// The reference has no such kernel on CUDA (its QuantizedMatmul re-runs the
// matvec once per activation row, crates/luminal_cuda/src/quantized.rs:146-164);
// the design precedent is the Metal backend's GEMM, which dequantises a weight
// tile into threadgroup memory and feeds the matrix unit
// (crates/luminal_metal/src/quantized.rs:54-61,63-199).  That kernel rounds
// q * d to the activation type first; this one keeps the weights exact:
//   * a workgroup owns a BM x BN output tile and walks K in steps of 64 (two
//     Q8_0 blocks);
//   * activations go global -> registers -> LDS as bf16; weight codes go global
//     (planar int8, 16-byte loads) -> registers -> bf16 (an int8 is exact in
//     bf16: one sign-extending byte conversion and a pack) -> LDS, and the two
//     block scales of the K tile go to LDS as f32;
//   * LDS is double-buffered and the global loads run D tiles ahead in
//     rotating register sets; one barrier per tile separates LDS writers from
//     readers;
//   * each wavefront computes a 64 x 64 sub-tile with v_mfma_f32_32x32x16_bf16:
//     a Q8_0 block is two chained steps into a zeroed accumulator, and the
//     block's scale multiplies that f32 block sum, acc += d * sum, the
//     arithmetic of the matvec kernels (quantized.rs:93-96: sumf += sumq * d);
//     LDS rows are padded by 16 bytes so the 16-byte operand reads of 8
//     consecutive lanes hit all banks once;
//   * workgroups that share a weight tile (same N tile, different M tiles) get
//     consecutive slots on the same XCD (block id modulo 8), so the weight tile
//     is fetched from HBM once and re-read from that XCD's L2; the M tiles are
//     walked in groups of 8, so that the activation tiles of a group stay in
//     that L2 while the XCD's N tiles pass.  What the counters show fetched
//     beyond the algorithmic bytes is activations (every XCD reads all of X for
//     each round of its N tiles), not weights.
// With bf16 activations every product is exact, so the only roundings are those
// of the f32 additions (and the one of the bf16 store).  Rounding q * d to bf16
// instead leaves a relative error of 2^-9 per weight, proportional to the sum
// of |w x| and therefore large on every output that cancels: measured 3.5 to
// 5.1 under max |y - t| / max(|t|, 1e-3 rms(t)) on the Llama-3-8B shapes, where
// this kernel scores 3.9e-3 (the bf16 store alone) and 1e-4 to 5e-4 on its f32 output.
#include <hip/hip_fp16.h>

#include <type_traits>
#include <utility>

#include "common.h"

namespace lhip {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t gu32x4 __attribute__((ext_vector_type(4)));

// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), expanded at compile time (register arrays
// indexed at run time land in scratch memory).
template <class F, int... Is>
__device__ __forceinline__ void gm_static_for_impl(F &&f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void gm_static_for(F &&f) {
    gm_static_for_impl(static_cast<F &&>(f), std::make_integer_sequence<int, N>{});
}

constexpr int kBK = 64;             // K per tile: two Q8_0 blocks
constexpr int kRowBytes = 144;      // 64 bf16 + 16 bytes of padding

// Tile BM x BN by WM x WN waves of at most 64 x 64 each.  LDS per buffer: activations BM x 64 bf16, codes BN x 64 as
// bf16 (rows of 144 bytes), and the BN x 2 block scales of the K tile as f32.  The lane that owns column n of a
// 32 x 32 accumulator tile needs one scale per block: it reads both scales of the K tile with one 8-byte LDS read.
// The per-block fma costs one v_fma per output element and block on the vector ALU, the same number of cycles the
// block's two MFMAs take on the matrix pipe.
// D = register prefetch depth in K tiles (D > 1 needs K % (64*D) == 0 and D even).
// N = weight rows of this launch; ldy = row pitch of y in weight rows (N, or more when the launch writes the leading
// columns of a wider output; the SwiGLU form stores pairs at half that pitch).
// OutT = __bf16 (rounded to nearest even) or float (the accumulators as they are).
template <int BM, int BN, int WM, int WN, int D, typename OutT>
__global__ __launch_bounds__(WM *WN * 64) void q8_gemm_bf16_kernel(const int8_t *__restrict__ qs,
                                                                 const __half *__restrict__ ds,
                                                                 const __bf16 *__restrict__ x, OutT *__restrict__ y_all,
                                                                 int M, int N, int K, int m_tiles, int n_tiles,
                                                                 int swiglu, int kt_slice, int m_group, int ldy) {
    constexpr int T = WM * WN * 64;
    constexpr int TM = BM / WM, TN = BN / WN;
    constexpr int FM = TM / 32, FN = TN / 32;  // 32x32 accumulator tiles per wave
    static_assert(FM >= 1 && FN >= 1 && FM <= 2 && FN <= 2, "wave tiles of at most 64 x 64");
    constexpr int A_CHUNKS = BM * 8 / T;
    constexpr int B_CHUNKS = BN * 4 / T;
    static_assert(A_CHUNKS >= 1 && B_CHUNKS >= 1 && BM * 8 % T == 0 && BN * 4 % T == 0, "tile/thread mismatch");
    constexpr int A_BYTES = BM * kRowBytes, B_BYTES = BN * kRowBytes, S_BYTES = BN * 8;
    constexpr int BUF = A_BYTES + B_BYTES + S_BYTES;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // 2 x (A tile, B tile, scales)

    int mt, nt;
    {
        // Workgroups are dealt to the eight XCDs in turn (id modulo 8) and an XCD runs its slots in order, 32 at a
        // time.  The XCD owns the N tiles xcd, xcd + 8, ...; its slots walk the M tiles in groups of m_group: within
        // a group N tile by N tile, the group's M tiles innermost.  The 32 workgroups in flight on an XCD are then
        // m_group M tiles x 32 / m_group N tiles: each of their weight tiles is fetched once and shared by m_group
        // workgroups out of the XCD's L2, each activation tile by 32 / m_group.
        const int id = blockIdx.x;
        const int xcd = id & 7, slot = id >> 3;
        const int npx = (n_tiles + 7) >> 3;                      // N tiles per XCD (the grid is padded to whole eights)
        const int full = m_tiles / m_group;                      // whole groups of M tiles
        const int in_full = full * m_group * npx;
        const int g0 = slot < in_full ? slot / (m_group * npx) : full;
        const int cur = slot < in_full ? m_group : m_tiles - full * m_group;
        const int rem = slot - g0 * m_group * npx;
        const int n_idx = rem / cur;
        mt = g0 * m_group + (rem - n_idx * cur);
        nt = n_idx * 8 + xcd;
        if (nt >= n_tiles) return;
    }
    const int m0 = mt * BM, n0 = nt * BN;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WN, wn = wave % WN;
    const int nblk = K >> 5;
    const int kt0 = kt_slice > 0 ? static_cast<int>(blockIdx.y) * kt_slice : 0;
    const int KT = kt_slice > 0 ? min(kt_slice, K / kBK - kt0) : K / kBK;
    OutT *__restrict__ y = y_all + (kt_slice > 0 ? static_cast<size_t>(blockIdx.y) * M * N : 0);

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
    int b_dst[B_CHUNKS];
    int s_dst[B_CHUNKS];              // where this thread leaves the row's scales, or -1: one thread in four does
#pragma unroll
    for (int i = 0; i < B_CHUNKS; ++i) {
        const int c = tid + i * T;
        const int row = c >> 2, q16 = c & 3;
        const int grow = min(n0 + row, N - 1);
        b_src[i] = qs + static_cast<size_t>(grow) * K + q16 * 16 + kt0 * kBK;
        d_src[i] = reinterpret_cast<const uint32_t *>(ds + static_cast<size_t>(grow) * nblk) + kt0;
        b_dst[i] = row * kRowBytes + q16 * 32;
        s_dst[i] = q16 == 0 ? row * 8 : -1;
    }

    gu32x4 a_reg[D][A_CHUNKS], b_reg[D][B_CHUNKS];
    uint32_t d_reg[D][B_CHUNKS];
    auto load_tile = [&](int set, int kt, int p = 0, int P = 1) {
        const int k0 = min(kt, KT - 1) * kBK;  // tiles past the end re-read the last one (never used)
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i)
            if (i * P / A_CHUNKS == p) a_reg[set][i] = *reinterpret_cast<const gu32x4 *>(a_src[i] + k0);
#pragma unroll
        for (int i = 0; i < B_CHUNKS; ++i) {
            if (i * P / B_CHUNKS != p) continue;
            b_reg[set][i] = *reinterpret_cast<const gu32x4 *>(b_src[i] + k0);
            d_reg[set][i] = d_src[i][k0 >> 6];
        }
    };
    // two int8 of a dword (bytes 2h, 2h+1) -> two bf16, exactly: the sign-extending byte conversion gives an f32
    // whose upper half is the bf16 code
    auto codes2 = [](uint32_t w, int h) {
        const float lo = static_cast<float>(static_cast<signed char>(w >> (16 * h)));
        const float hi = static_cast<float>(static_cast<signed char>(w >> (16 * h + 8)));
        return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
    };
    auto store_tile = [&](int set, int buf, int p = 0, int P = 1) {
        unsigned char *A = lds + buf * BUF;
        unsigned char *B = A + A_BYTES;
        unsigned char *S = B + B_BYTES;
#pragma unroll
        for (int i = 0; i < A_CHUNKS; ++i)
            if (i * P / A_CHUNKS == p) *reinterpret_cast<gu32x4 *>(A + a_dst[i]) = a_reg[set][i];
#pragma unroll
        for (int u = 0; u < 2 * B_CHUNKS; ++u) {
            if (u * P / (2 * B_CHUNKS) != p) continue;
            const int i = u >> 1;
            // Opaque to the optimiser: keeps the unpacking of this set here, at its use, instead of next to its loads
            asm volatile("" : "+v"(b_reg[set][i]), "+v"(d_reg[set][i]));
            if ((u & 1) == 0) {
                const gu32x4 lo = {codes2(b_reg[set][i].x, 0), codes2(b_reg[set][i].x, 1), codes2(b_reg[set][i].y, 0),
                                   codes2(b_reg[set][i].y, 1)};
                *reinterpret_cast<gu32x4 *>(B + b_dst[i]) = lo;
                if (s_dst[i] >= 0) {
                    const float d0 = __half2float(__ushort_as_half(static_cast<unsigned short>(d_reg[set][i] & 0xffffu)));
                    const float d1 = __half2float(__ushort_as_half(static_cast<unsigned short>(d_reg[set][i] >> 16)));
                    *reinterpret_cast<float2 *>(S + s_dst[i]) = make_float2(d0, d1);
                }
            } else {
                const gu32x4 hi = {codes2(b_reg[set][i].z, 0), codes2(b_reg[set][i].z, 1), codes2(b_reg[set][i].w, 0),
                                   codes2(b_reg[set][i].w, 1)};
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

    const int frag_off = (lane & 31) * kRowBytes + (lane >> 5) * 16;
    // One K tile: two blocks of FM x FN slots; a slot is the two chained MFMAs of one accumulator tile's block sum.
    // The scheduler, left alone, issues every MFMA of the K tile first and every fma after (eight block sums live:
    // spills), so the order is fixed with scheduling fences: the sixteen fmas of the previous slot's block sum are
    // issued in two halves behind the two MFMAs of this slot and run on the vector ALU while the matrix pipe
    // works; the last slot's sum of a K tile is carried into the next tile (`pend`, zero before the first).  With STAGE the
    // dequantise-and-store of the next tile and the global loads of the tile after that are dealt out over the
    // slots.  The operand fragments of block 1 are requested during block 0 as their registers fall free (row i's
    // A fragments after its last column, column j's B fragments after its last row).
    f32x16 pend = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};  // block sum whose fmas are still to be issued
    float pend_d = 0.f;                                                                              // and its scale
    // Opaque to the optimiser, or it peels the first K tile off the loop (its fmas fold away) and schedules that
    // copy with all eight block sums live.
    asm volatile("" : "+v"(pend), "+v"(pend_d));
    auto k_tile = [&](int buf, bool stage, int set, int next_buf, int load_set, int load_kt) {
        const unsigned char *A = lds + buf * BUF + (wm * TM) * kRowBytes + frag_off;
        const unsigned char *B = lds + buf * BUF + A_BYTES + (wn * TN) * kRowBytes + frag_off;
        const unsigned char *S = lds + buf * BUF + A_BYTES + B_BYTES + (wn * TN + (lane & 31)) * 8;
        bf16x8 af[2][2][FM], bfr[2][2][FN];  // [block][k step][tile]
        auto load_a = [&](int b, int i) {
#pragma unroll
            for (int s = 0; s < 2; ++s)
                af[b][s][i] = *reinterpret_cast<const bf16x8 *>(A + i * 32 * kRowBytes + (2 * b + s) * 32);
        };
        auto load_b = [&](int b, int j) {
#pragma unroll
            for (int s = 0; s < 2; ++s)
                bfr[b][s][j] = *reinterpret_cast<const bf16x8 *>(B + j * 32 * kRowBytes + (2 * b + s) * 32);
        };
        float2 sc[FN];
#pragma unroll
        for (int j = 0; j < FN; ++j) sc[j] = *reinterpret_cast<const float2 *>(S + j * 32 * 8);
#pragma unroll
        for (int i = 0; i < FM; ++i) load_a(0, i);
#pragma unroll
        for (int j = 0; j < FN; ++j) load_b(0, j);
        gm_static_for<2 * FM * FN>([&](auto qc) __attribute__((always_inline)) {
            constexpr int q = decltype(qc)::value;
            constexpr int b = q / (FM * FN), r = q % (FM * FN), i = r / FN, j = r % FN;
            constexpr int rp = (r + FM * FN - 1) % (FM * FN), ip = rp / FN, jp = rp % FN;  // the slot before this one
            if (stage) {
                store_tile(set, next_buf, q, 2 * FM * FN);
                load_tile(load_set, load_kt, q, 2 * FM * FN);
            }
            __builtin_amdgcn_sched_barrier(0);
            f32x16 sum = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
            sum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[b][0][i], bfr[b][0][j], sum, 0, 0, 0);
            // (the empty asm statements tie each result to its place between the fences: the fences hold the machine
            // scheduler, but arithmetic without side effects is moved past them before it ever gets there)
            asm volatile("" : "+v"(sum));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int v = 0; v < 8; ++v) acc[ip][jp][v] = fmaf(pend_d, pend[v], acc[ip][jp][v]);
            asm volatile("" : "+v"(acc[ip][jp]));
            __builtin_amdgcn_sched_barrier(0);
            sum = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[b][1][i], bfr[b][1][j], sum, 0, 0, 0);
            asm volatile("" : "+v"(sum));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int v = 8; v < 16; ++v) acc[ip][jp][v] = fmaf(pend_d, pend[v], acc[ip][jp][v]);
            asm volatile("" : "+v"(acc[ip][jp]));
            if constexpr (b == 0) {  // this slot's MFMAs are issued: block 1's fragments into the registers that fell free
                if constexpr (j == FN - 1) load_a(1, i);
                if constexpr (i == FM - 1) load_b(1, j);
            }
            __builtin_amdgcn_sched_barrier(0);
            pend = sum;
            pend_d = b ? sc[j].y : sc[j].x;
        });
    };

#pragma unroll
    for (int j = 0; j < D; ++j) load_tile(j, j);
    store_tile(0, 0);
    __syncthreads();

    if constexpr (D == 1) {
        for (int kt = 0; kt < KT; ++kt) {
            load_tile(0, kt + 1);
            k_tile(kt & 1, false, 0, 0, 0, 0);
            store_tile(0, (kt + 1) & 1);
            __syncthreads();
        }
    } else {
        static_assert(D % 2 == 0, "LDS buffer parity must follow the register set");
        for (int kt = 0; kt < KT; kt += D) {
#pragma unroll
            for (int j = 0; j < D; ++j) {
                // set j held tile kt+j, already in LDS: refill it with tile kt+j+D
                k_tile(j & 1, true, (j + 1) % D, (j + 1) & 1, j, kt + j + D);
                __syncthreads();
            }
        }
    }

#pragma unroll
    for (int v = 0; v < 16; ++v) acc[FM - 1][FN - 1][v] = fmaf(pend_d, pend[v], acc[FM - 1][FN - 1][v]);

    // Epilogue: acc element v of lane l is row 8*(v/4) + 4*(l/32) + v%4, column l%32 of its 32x32 tile.
    if constexpr (sizeof(OutT) == 2) {
        if (swiglu) {
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
                                                        static_cast<size_t>(row) * (ldy >> 1) + (col >> 1)) = pk;
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
                if (row < M && col < N) y[static_cast<size_t>(row) * ldy + col] = static_cast<OutT>(acc[i][j][v]);
            }
        }
}

// What the epilogue writes: bf16 (m, N), f32 (m, N), or bf16 (m, N/2) = up * swish(gate) of (gate, up) column pairs.
enum { kOutBf16 = 0, kOutF32 = 1, kOutSwiglu = 2 };

// q8_gemm_skinny.hip: the weight-streaming kernel for at most 128 activation rows.
bool q8_gemm_skinny_supports(int m, int n, int k, int out, const void *y);
int q8_gemm_skinny_splits(int m, int n, int k, size_t room);
lhip_status q8_gemm_skinny_launch(const int8_t *qs, const __half *ds, const void *x_bf16, void *y, int m, int n, int k,
                                  int out, int splits, hipStream_t s, bool own_workspace = false, float *ws = nullptr,
                                  size_t ws_floats = 0);
float *q8_gemm_scratch(size_t *floats);  // the library's partial-sum array on the current device
constexpr size_t kGemmScratchFloats = size_t{8} << 20;  // its size (q8_gemm_skinny.hip: kSkScratchFloats)

// Where the partial planes of a K-sliced product go: the library's per-device scratch array (shared by every call on
// the device), or the caller's workspace (the re-entrant entry points).  A workspace smaller than the plan of the
// plain call needs means fewer or no slices.
struct GemmScratch {
    bool own = false;       // true: `ws` / `floats` below, never the library's array
    float *ws = nullptr;
    size_t floats = 0;
    size_t room() const { return own ? (ws ? (floats < kGemmScratchFloats ? floats : kGemmScratchFloats) : 0) : kGemmScratchFloats; }
};
lhip_status q8_gemm_reduce_launch(const float *part, void *y, int m, int n, int slices, int out, hipStream_t s, int ldy = 0);
constexpr int kTileSkinny = 5;        // K slices chosen by the library
constexpr int kTileSkinnySplit = 50;  // + number of K slices
constexpr int kTileSliced = 120;      // + number of K slices: the 256x128 tile over slices of K, then a reduction
constexpr int kTileTail = 200;        // the 256x128 tile in whole rounds of 256 workgroups, the last columns over K slices

// A product of more than 256 tiles of 256x128 runs in rounds of 256 workgroups (one per CU), and a last round that
// is partly filled takes as long as a full one: 896 tiles (gate/up at 2048 rows) are 3.5 rounds of work in the time
// of 4.  The plan below gives the whole rounds to the plain kernel and the remaining column tiles to the K-sliced
// form (f32 partial planes in the scratch array, added in slice order), so that the remainder fills the chip for
// 1 / slices of a round: `n_main` leading weight rows in whole rounds, `slices` K slices for the rest (0: no such
// plan).  Needs the M tiles to divide 256, a remainder of at most half a round, K long enough for the saving to
// exceed the reduction launch, and room for the planes.
struct GemmTail {
    int n_main = 0, slices = 0;
};
static GemmTail gemm_tail_plan(int64_t m, int64_t n, int64_t k, int out, const void *y, size_t room) {
    GemmTail none;
    if (m <= 128 || k < 2048 || n % 4 != 0 || !aligned(y, out == kOutF32 ? 16 : (out == kOutBf16 ? 8 : 4))) return none;
    const int64_t m_tiles = (m + 255) / 256, n_tiles = (n + 127) / 128;
    if (m_tiles * n_tiles <= 256 || 256 % m_tiles != 0) return none;
    const int64_t per_round = 256 / m_tiles;                 // column tiles of one round
    const int64_t main_tiles = n_tiles / per_round * per_round;
    const int64_t tail_tiles = (n_tiles - main_tiles) * m_tiles;
    if (tail_tiles == 0) return none;
    const int64_t n_tail = n - main_tiles * 128, kt = k / kBK;
    for (int slices = 8; slices >= 2; slices >>= 1)
        if (tail_tiles * slices <= 256 && kt % slices == 0 && (kt / slices) % 4 == 0 &&
            static_cast<size_t>(slices) * m * n_tail <= room) {
            GemmTail t;
            t.n_main = static_cast<int>(main_tiles * 128);
            t.slices = slices;
            return t;
        }
    return none;
}

// M tiles per group of the raster (see the kernel).  Measured on the FFN, QKV and lm_head shapes: groups of 8 are
// 5 % faster than one group of all the M tiles at M = 8192 (32 M tiles), 1 % at 4096, and the same launch at or below
// 2048 (at most 8 M tiles); groups of 4 or 6 are within 1 % of 8.
constexpr int kGemmMGroup = 8;
static int gemm_m_group(int m_tiles) { return m_tiles < kGemmMGroup ? m_tiles : kGemmMGroup; }

template <int BM, int BN, int WM, int WN, int D, typename OutT>
static lhip_status launch_gemm_t(const int8_t *qs, const __half *ds, const void *x, void *y, int m, int n, int k,
                               int swiglu, hipStream_t s, int slices = 1, int ldy = 0) {
    const int m_tiles = (m + BM - 1) / BM, n_tiles = (n + BN - 1) / BN;
    const int n_tiles_pad = (n_tiles + 7) / 8 * 8;
    if (static_cast<int64_t>(m_tiles) * n_tiles_pad > 0x7fffffff) return LHIP_ERR_INVALID_SHAPE;  // the grid's x extent
    const size_t lds_bytes = 2 * (static_cast<size_t>(BM + BN) * kRowBytes + static_cast<size_t>(BN) * 8);
    auto kern = q8_gemm_bf16_kernel<BM, BN, WM, WN, D, OutT>;
    static LdsOptIn opt;
    if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(kern), lds_bytes)) return st;
    const int kt_slice = slices > 1 ? (k / kBK + slices - 1) / slices : 0;
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(m_tiles * n_tiles_pad), static_cast<unsigned>(slices)),
                       dim3(WM * WN * 64), lds_bytes, s, qs, ds, static_cast<const __bf16 *>(x), static_cast<OutT *>(y), m,
                       n, k, m_tiles, n_tiles, swiglu, kt_slice, gemm_m_group(m_tiles), ldy > 0 ? ldy : n);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

template <int BM, int BN, int WM, int WN, int D>
static lhip_status launch_gemm(int out, const int8_t *qs, const __half *ds, const void *x, void *y, int m, int n, int k,
                             hipStream_t s) {
    return out == kOutF32 ? launch_gemm_t<BM, BN, WM, WN, D, float>(qs, ds, x, y, m, n, k, 0, s)
                          : launch_gemm_t<BM, BN, WM, WN, D, __bf16>(qs, ds, x, y, m, n, k, out == kOutSwiglu, s);
}

static lhip_status gemm_dispatch(const void *planar_dev, const void *x_dev, void *y_dev, int64_t m, int64_t n, int64_t k,
                                 int tile, int out, void *stream, const GemmScratch &scratch = GemmScratch{}) {
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
    if (tile == kTileSkinny || (tile > kTileSkinnySplit && tile <= kTileSkinnySplit + 64)) {
        if (!q8_gemm_skinny_supports(mi, ni, ki, out, y_dev)) return LHIP_ERR_UNSUPPORTED;
        return q8_gemm_skinny_launch(qs, ds, x_dev, y_dev, mi, ni, ki, out, tile == kTileSkinny ? 0 : tile - kTileSkinnySplit, s,
                                     scratch.own, scratch.ws, scratch.floats);
    }
    if (tile > kTileSliced && tile <= kTileSliced + 16) {
        // Few output tiles and a long K (the down projection of a 512-token prompt: 64 tiles of 256x128): slices of K
        // fill the chip, f32 partial planes go to the scratch array and are added in slice order.
        const int slices = tile - kTileSliced;
        const int kt = ki / kBK;
        size_t cap = scratch.room();
        float *part = scratch.own ? scratch.ws : q8_gemm_scratch(&cap);
        if (!part) return scratch.own ? LHIP_ERR_UNSUPPORTED : LHIP_ERR_HIP;
        if (slices < 2 || kt % slices != 0 || (kt / slices) % 4 != 0 || static_cast<size_t>(slices) * mi * ni > cap ||
            ni % 4 != 0 || !aligned(y_dev, out == kOutF32 ? 16 : (out == kOutBf16 ? 8 : 4)))
            return LHIP_ERR_UNSUPPORTED;
        if (lhip_status st = launch_gemm_t<256, 128, 4, 2, 4, float>(qs, ds, x_dev, part, mi, ni, ki, 0, s, slices))
            return st;
        return q8_gemm_reduce_launch(part, y_dev, mi, ni, slices, out, s);
    }
    if (tile == kTileTail) {
        size_t cap = scratch.room();
        float *part = scratch.own ? scratch.ws : q8_gemm_scratch(&cap);
        if (!part) return scratch.own ? LHIP_ERR_UNSUPPORTED : LHIP_ERR_HIP;
        const GemmTail t = gemm_tail_plan(m, n, k, out, y_dev, cap);
        if (t.slices < 2) return LHIP_ERR_UNSUPPORTED;
        const int n_tail = ni - t.n_main;
        // whole rounds: the leading n_main weight rows, written into the full-width output
        if (lhip_status st = out == kOutF32
                                 ? launch_gemm_t<256, 128, 4, 2, 4, float>(qs, ds, x_dev, y_dev, mi, t.n_main, ki, 0, s, 1, ni)
                                 : launch_gemm_t<256, 128, 4, 2, 4, __bf16>(qs, ds, x_dev, y_dev, mi, t.n_main, ki,
                                                                            out == kOutSwiglu, s, 1, ni))
            return st;
        // the rest: K slices of the trailing weight rows into the planes, then their sum into the trailing columns
        const int8_t *qs_tail = qs + static_cast<size_t>(t.n_main) * ki;
        const __half *ds_tail = ds + static_cast<size_t>(t.n_main) * (ki / 32);
        if (lhip_status st = launch_gemm_t<256, 128, 4, 2, 4, float>(qs_tail, ds_tail, x_dev, part, mi, n_tail, ki, 0, s, t.slices))
            return st;
        const size_t col0 = out == kOutSwiglu ? t.n_main / 2 : t.n_main;
        void *y_tail = out == kOutF32 ? static_cast<void *>(static_cast<float *>(y_dev) + col0)
                                      : static_cast<void *>(static_cast<__bf16 *>(y_dev) + col0);
        return q8_gemm_reduce_launch(part, y_tail, mi, n_tail, t.slices, out, s, ni);
    }
    // Register prefetch four (two) K tiles ahead needs K to be a whole number of 4-tile (2-tile) rounds.
    const int depth = (k % (kBK * 4)) == 0 ? 4 : ((k % (kBK * 2)) == 0 ? 2 : 1);
#define LHIP_TILE(BM, BN, WM, WN)                                                                          \
    return depth == 4   ? launch_gemm<BM, BN, WM, WN, 4>(out, qs, ds, x_dev, y_dev, mi, ni, ki, s)      \
           : depth == 2 ? launch_gemm<BM, BN, WM, WN, 2>(out, qs, ds, x_dev, y_dev, mi, ni, ki, s)      \
                        : launch_gemm<BM, BN, WM, WN, 1>(out, qs, ds, x_dev, y_dev, mi, ni, ki, s)
    switch (tile) {
        case 0: LHIP_TILE(256, 128, 4, 2);
        case 1: LHIP_TILE(128, 128, 2, 2);
        case 2: LHIP_TILE(128, 64, 2, 2);
        case 3: LHIP_TILE(64, 64, 2, 2);
        default: return LHIP_ERR_UNSUPPORTED;
    }
#undef LHIP_TILE
}

static int gemm_auto_tile(int64_t m, int64_t n, int64_t k, int out, const void *y, size_t room = kGemmScratchFloats) {
    // Few activation rows: the product is bound by the weight stream
    if (m <= 128 && n <= kMaxDim && k <= kMaxDim &&
        q8_gemm_skinny_supports(static_cast<int>(m), static_cast<int>(n), static_cast<int>(k), out, y))
        return kTileSkinny;
    auto blocks = [&](int bm, int bn) { return ((m + bm - 1) / bm) * ((n + bn - 1) / bn); };
    // Few 256x128 tiles: slices of K until the chip is full, when the partial planes (written and read once more:
    // 4 * slices / K bytes per flop) fit the scratch array.  A workgroup walks K at about 1.2 us per 64-wide tile
    // whatever M is, so with fewer workgroups than CUs the K loop is the critical path and slicing it pays at every K
    // (measured, us, whole K -> sliced: 4096 x 4096 at 256 / 512 / 1024 rows 75 -> 30 / 75 -> 38 / 78 -> 58;
    // 1024 x 4096 at 512 rows 72 -> 23; 4096 x 14336 at 256 / 512 / 1024 rows 237 -> 56 / 240 -> 89 / 249 -> 163).
    if (m > 128 && n % 4 == 0 && aligned(y, out == kOutF32 ? 16 : (out == kOutBf16 ? 8 : 4))) {
        const int64_t b0 = blocks(256, 128), kt = k / kBK;
        for (int slices = 8; slices >= 2; slices >>= 1)
            if (b0 * slices <= 256 && kt % slices == 0 && (kt / slices) % 4 == 0 &&
                static_cast<size_t>(slices) * m * n <= room)
                return kTileSliced + slices;
    }
    // Otherwise the 256x128 tile from 64 workgroups on (measured faster than the smaller tiles there even with a
    // quarter of the CUs busy: its K loop is the shortest per flop), smaller tiles for small products.
    if (m > 128 && k % (kBK * 4) == 0 && gemm_tail_plan(m, n, k, out, y, room).slices >= 2) return kTileTail;
    if (m > 128 && blocks(256, 128) >= 64) return 0;
    return blocks(128, 64) >= 64 ? 2 : 3;
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

size_t lhip_q8_0_matmul_bf16_workspace_nbytes(int64_t m, int64_t n, int64_t k, int32_t out_form) {
    if (check_q8_shape(n, k) != LHIP_OK || m <= 0 || m > kMaxDim || k % kBK != 0) return 0;
    if (out_form < kOutBf16 || out_form > kOutSwiglu) return 0;
    // the plan of the plain call (an aligned output is assumed: the plain call slices K for aligned outputs only)
    const int tile = gemm_auto_tile(m, n, k, out_form, nullptr);
    size_t floats = 0;
    if (tile > kTileSliced && tile <= kTileSliced + 16)
        floats = static_cast<size_t>(tile - kTileSliced) * m * n;
    else if (tile == kTileTail) {
        const GemmTail t = gemm_tail_plan(m, n, k, out_form, nullptr, kGemmScratchFloats);
        floats = static_cast<size_t>(t.slices) * m * (n - t.n_main);
    }
    else if (tile == kTileSkinny) {
        const int splits = q8_gemm_skinny_splits(static_cast<int>(m), static_cast<int>(n), static_cast<int>(k), kGemmScratchFloats);
        if (splits > 1) floats = static_cast<size_t>(splits) * m * n;
    }
    return floats * sizeof(float);
}

lhip_status lhip_q8_0_matmul_bf16_ws(const void *planar_dev, const void *x_dev, void *y_dev, int64_t m, int64_t n, int64_t k,
                                     int32_t out_form, void *workspace_dev, size_t workspace_nbytes, void *stream) {
    if (out_form < kOutBf16 || out_form > kOutSwiglu) return LHIP_ERR_INVALID_SHAPE;
    if (workspace_dev && !aligned(workspace_dev, 256)) return LHIP_ERR_MISALIGNED;
    GemmScratch scratch;
    scratch.own = true;
    scratch.ws = static_cast<float *>(workspace_dev);
    scratch.floats = workspace_dev ? workspace_nbytes / sizeof(float) : 0;
    return gemm_dispatch(planar_dev, x_dev, y_dev, m, n, k, gemm_auto_tile(m, n, k, out_form, y_dev, scratch.room()), out_form,
                         stream, scratch);
}

}  // extern "C"
