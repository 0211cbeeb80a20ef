// MXFP4 mixture-of-experts layer, exact form: the weights are expanded to bf16 in registers and multiplied on the
// bf16 matrix instruction with f32 accumulation.
//
// Not in the reference (it has neither MXFP4 nor MoE).  Its convention for quantised weights is "dequantise exactly,
// then multiply in f32" (examples/llama/src/loader.rs:227-241) and its expert MLP is luminal's SwiGLU
// down( up(x) * swish(gate(x)) ) (examples/llama/src/model.rs:24-32, src/hl_ops/unary.rs:169-177).  This form keeps
// to that: an e2m1 value times 2^(e8m0 - 127) has at most two significant bits and bf16 has the exponent range of
// f32, so every weight is a bf16 number exactly; the activations are the bf16 numbers the caller passed; products of
// two bf16 numbers are exact in f32, and v_mfma_f32_16x16x32_bf16 adds them at f32 accuracy.  The only roundings of a
// matmul are those of its f32 accumulation (and one to bf16 where the output is bf16).
//
// The expansion is one instruction per two weights: v_cvt_scalef32_pk_bf16_fp4 takes a byte of two e2m1 codes and a
// scale (an f32 whose exponent field is the block's e8m0 code) and returns the two scaled values as a bf16 pair.
//
// Operands.  The planar weights are tiled for a wavefront (common.h: lane (r, g) of a 16-row panel and 128-wide
// chunk holds the 32 codes of block g of row r as four dwords).  Dword d of that piece is codes k = 32g + 8d .. + 7,
// eight bf16 numbers after expansion, which is a lane's share of the weight operand of one 16x16x32 step; the
// hardware's k slot (g, e) of step d therefore stands for k = 32g + 8d + e, and the activation operand of that step
// is x[row][chunk*128 + 32g + 8d .. + 7] for lane (row, g): one 16-byte LDS read.  Four steps cover the chunk.
// In LDS an activation row of a chunk lies in two planes of 128 bytes (steps 0-1, steps 2-3), piece (g, d) at
// byte 16 (g + 4 (d & 1)) of plane d >> 1, which gives the fragment reads the addresses r * pitch + 16 g + 64 (d & 1)
// that were measured free of bank conflicts at a pitch of 160 bytes.
#include "mxfp4_moe_device.h"

namespace lhip {

typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));

// The 32 codes of one block (four dwords, even k in the low nibble) times 2^(code - 127), as the four weight
// operands of the block's matrix steps.
__device__ __forceinline__ void mx_expand_block(const mu32x4 &q, uint32_t scale_code, v8bf (&w)[4]) {
    const float s = __uint_as_float(scale_code << 23);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const v2bf p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[d], s, 0);
        const v2bf p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[d], s, 1);
        const v2bf p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[d], s, 2);
        const v2bf p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q[d], s, 3);
        w[d] = v8bf{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
    }
}

// LDS byte offset, inside a row's two planes of `plane_bytes` each, of 16-byte piece j (k = 8j .. 8j+7) of a chunk.
__device__ __forceinline__ int exact_piece_offset(int j, int plane_bytes) {
    const int g = j >> 2, d = j & 3;
    return (d >> 1) * plane_bytes + (g + 4 * (d & 1)) * 16;
}

// up * swish(gate) with the hardware exp2 and reciprocal (1 ulp each), as the block-scaled form computes it.
__device__ __forceinline__ float exact_swiglu(float gate, float up) {
    return up * (gate * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * gate)));
}

// ---------------------------------------------------------------------------
// Planar MXFP4 -> bf16[N][K] through the expansion the GEMMs use.  One thread per block of 32 weights.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void mx_dequant_bf16_kernel(const uint8_t *__restrict__ nib, const uint8_t *__restrict__ sc,
                                                              __bf16 *__restrict__ out, size_t n_pieces, int n, int k,
                                                              int chunks) {
    const size_t piece = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (piece >= n_pieces) return;
    const size_t tile = piece >> 6;
    const int in_tile = static_cast<int>(piece & 63);
    const size_t panel = tile / chunks;
    const int chunk = static_cast<int>(tile - panel * chunks);
    const size_t row = panel * 16 + (in_tile & 15);
    const int kb = chunk * 4 + (in_tile >> 4);
    if (row >= static_cast<size_t>(n) || kb * 32 >= k) return;
    const mu32x4 q = *reinterpret_cast<const mu32x4 *>(nib + piece * 16);
    v8bf w[4];
    mx_expand_block(q, sc[piece], w);
    v8bf *o = reinterpret_cast<v8bf *>(out + row * k + kb * 32);
#pragma unroll
    for (int d = 0; d < 4; ++d) o[d] = w[d];
}

// ---------------------------------------------------------------------------
// Grouped expert GEMM.  grid = (column blocks, max tiles); a workgroup of 4 * WR waves owns one row tile (up to
// BM = 16 MT routed rows of one expert) and 4 NT column fragments of 16.  Wave (column group, row group) holds the
// activation fragments of its MT / WR row fragments in registers for a whole chunk and walks its NT weight
// fragments: expand one (16 conversions), multiply it with every row fragment (4 matrix steps each).  So a weight
// is expanded once per row tile whatever the tile's height, and an activation fragment is read from LDS once per
// chunk.  GATED: fragments come in pairs, gate rows and the matching up rows; output bf16 up * swish(gate), else f32.
// ---------------------------------------------------------------------------
struct MoeExactArgs {
    const __bf16 *a;      // activation rows, K elements each
    const int *a_index;   // slot -> routed entry (GEMM 1) or nullptr (rows are slots)
    int a_div;            // routed entry / a_div = activation row
    const uint8_t *w_nib, *w_sc;
    int rows_per_expert;
    int K, Kp;
    int N;
    const int *tile_expert, *tile_row0, *tile_rows, *n_tiles;
    const int *tile_run0, *tile_runlen;
    int tiles_per_xcd;
    void *out;            // bf16 [R][N] (gated) or f32 [R][N]
};

template <int MT, int NT, bool GATED, int WR, int D>
__global__ __launch_bounds__(256 * WR) void mx_moe_gemm_exact_kernel(MoeExactArgs g) {
    static_assert(!GATED || NT % 2 == 0, "gated tiles pair each gate fragment with its up fragment");
    static_assert(MT % WR == 0 && D % 2 == 0 && NT >= 2, "tile shape");
    constexpr int BM = 16 * MT;
    constexpr int MTW = MT / WR;  // row fragments per wave
    constexpr int THREADS = 256 * WR;
    constexpr int STG = MT / WR;  // 16-byte pieces of the activation tile staged per thread and chunk
    constexpr int A_PLANE = BM * kARow;
    constexpr int A_BUF = 2 * A_PLANE;

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // 3 x A_BUF

    // Tile and column block of this workgroup (see MoePlan::tiles_per_xcd for the per-XCD list).
    // Within a run of tiles of one expert the workgroups are ordered column block by column block: the tiles that
    // read the same weights are dispatched next to each other and share one fetch of them out of the XCD's L2.
    int tile = blockIdx.y, cb = blockIdx.x;
    int expert, row0, rows;
    if (g.tiles_per_xcd) {
        const int linear = blockIdx.y * gridDim.x + blockIdx.x;
        const int turn = linear >> 3, cols = static_cast<int>(gridDim.x);
        const int base = (linear & 7) * g.tiles_per_xcd;
        const int entry = turn / cols;
        cb = turn - entry * cols;
        tile = base + entry;
        // (the entry's own tile is read in the same trip to memory; only a workgroup inside a run pays a second one,
        // and not for the expert, which the run shares)
        expert = g.tile_expert[tile];
        row0 = g.tile_row0[tile];
        rows = g.tile_rows[tile];
        const int run0 = g.tile_run0[tile], runlen = g.tile_runlen[tile];
        if (runlen > 1) {
            const int local = turn - (run0 - base) * cols;  // position among the run's runlen * cols workgroups
            cb = local / runlen;
            tile = run0 + (local - cb * runlen);
            row0 = g.tile_row0[tile];
            rows = g.tile_rows[tile];
        }
    } else {
        expert = g.tile_expert[tile];
        row0 = g.tile_row0[tile];
        rows = g.tile_rows[tile];
    }
    if (rows == 0) return;


    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave_id = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave = wave_id & 3;
    const int wrow = WR == 1 ? 0 : wave_id >> 2;
    const int r = lane & 15, grp = lane >> 4;
    const int K = g.K, Kp = g.Kp;
    const int chunks = Kp / kChunk;
    const int steps = (chunks + D - 1) / D * D;
    const int frags = (rows + 15) >> 4;

    // ---- weight fragments: one contiguous KiB of codes and 64 scale bytes per fragment and chunk
    const uint8_t *w_tile[NT];
    const uint8_t *s_tile[NT];
    int col[NT];
#pragma unroll
    for (int f = 0; f < NT; ++f) {
        int n0, wrow0;
        if (GATED) {
            n0 = ((cb * 4 + wave) * (NT / 2) + (f >> 1)) * 16;
            wrow0 = ((f & 1) ? g.N : 0) + min(n0, g.N - 16);
        } else {
            n0 = ((cb * 4 + wave) * NT + f) * 16;
            wrow0 = min(n0, g.N - 16);
        }
        col[f] = n0 + r;
        const size_t panel = (static_cast<size_t>(expert) * g.rows_per_expert + wrow0) >> 4;
        w_tile[f] = g.w_nib + (panel * chunks * 64 + lane) * 16;
        s_tile[f] = g.w_sc + panel * chunks * 64 + lane;
    }
    BSet<MT, NT> bs[D];
    auto load_b = [&](int set, int c) __attribute__((always_inline)) {
        bs[set].valid = c < chunks;  // dead chunks (past the padded K; the refills of the last round) are not multiplied
        const int cc = min(c, chunks - 1);
#pragma unroll
        for (int f = 0; f < NT; ++f) {
            if (MT <= 2) {  // short tiles read every weight once: keep them out of the caches
                // (a dead chunk's request goes to one line for the whole wave: aimed at the last chunk it would pull
                // that kilobyte through the memory system again, D + 1 times per wave and fragment)
                const uint8_t *wq = c < chunks ? w_tile[f] + static_cast<size_t>(cc) * 1024 : g.w_nib;
                bs[set].q[f] = __builtin_nontemporal_load(reinterpret_cast<const mu32x4 *>(wq));
                bs[set].s[f] = s_tile[f][cc * 64];  // (cached: the 64 scale bytes of two consecutive chunks share a line)
            } else {
                bs[set].q[f] = *reinterpret_cast<const mu32x4 *>(w_tile[f] + static_cast<size_t>(cc) * 1024);
                bs[set].s[f] = s_tile[f][cc * 64];
            }
        }
    };

    // ---- activation tile: global (bf16 rows) -> registers -> LDS (three buffers), shared by all waves.
    // Threads take the tile's pieces in source order (16 consecutive threads = the 256 bytes of one row).
    const uint8_t *a_src[STG];
    int a_k[STG], a_dst[STG];
#pragma unroll
    for (int i = 0; i < STG; ++i) {
        const int q = tid + i * THREADS;
        const int row = q >> 4, j = q & 15;
        const int slot = row0 + min(row, rows - 1);  // rows past the tile re-read its last row (their results are not stored)
        const int arow = g.a_index ? g.a_index[slot] / g.a_div : slot;
        a_src[i] = reinterpret_cast<const uint8_t *>(g.a + static_cast<size_t>(arow) * K) + j * 16;
        a_k[i] = j * 8;
        a_dst[i] = row * kARow + exact_piece_offset(j, A_PLANE);
    }
    struct AStage {
        mu32x4 q[STG];
    };
    auto load_a = [&](AStage &st, int c) __attribute__((always_inline)) {
        const int cc = min(c, chunks - 1);
#pragma unroll
        for (int i = 0; i < STG; ++i) {
            // Pieces past K (the last chunk of a K that is no multiple of 128) are zeros: the padding weights are zero
            // too, but zero times whatever lies behind the row need not be.
            const bool in = cc * kChunk + a_k[i] < K;
            const uint8_t *p = in ? a_src[i] + cc * (kChunk * 2) : reinterpret_cast<const uint8_t *>(g.a);
            const mu32x4 v = *reinterpret_cast<const mu32x4 *>(p);
            const mu32x4 zero = {0, 0, 0, 0};
            st.q[i] = in ? v : zero;
        }
    };
    auto store_a = [&](AStage &st, unsigned char *base) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < STG; ++i) {
            asm volatile("" : "+v"(st.q[i]));
            *reinterpret_cast<mu32x4 *>(base + a_dst[i]) = st.q[i];
        }
    };

    v4f acc[MTW][NT];
#pragma unroll
    for (int i = 0; i < MTW; ++i)
#pragma unroll
        for (int f = 0; f < NT; ++f) acc[i][f] = v4f{0.f, 0.f, 0.f, 0.f};

    // Row fragment n of this wave's row group is tile fragment n * WR + wrow.
    const int frag_lane = (wrow * 16 + r) * kARow + grp * 16;
    v8bf afr[MTW][4];
    auto load_frag = [&](const unsigned char *base, auto ic) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        const unsigned char *p = base + frag_lane + i * (WR * 16 * kARow);
        afr[i][0] = *reinterpret_cast<const v8bf *>(p);
        afr[i][1] = *reinterpret_cast<const v8bf *>(p + 64);
        afr[i][2] = *reinterpret_cast<const v8bf *>(p + A_PLANE);
        afr[i][3] = *reinterpret_cast<const v8bf *>(p + A_PLANE + 64);
    };
    auto mfma_frag = [&](const v8bf (&wb)[4], auto ic, auto fc) __attribute__((always_inline)) {
        constexpr int i = decltype(ic)::value;
        constexpr int f = decltype(fc)::value;
#pragma unroll
        for (int d = 0; d < 4; ++d) acc[i][f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(afr[i][d], wb[d], acc[i][f], 0, 0, 0);
        // Pin the accumulation here: nothing else reads acc until the epilogue, and without this the optimiser
        // sinks the matrix steps of the unrolled pipeline to its end and keeps every operand alive.
        asm volatile("" : "+a"(acc[i][f]));
    };

    // ---- pipeline: three LDS buffers, one barrier per chunk.  Chunk c multiplies out of buffer c % 3 (its
    // fragments are already in registers).  After the first weight fragment every wave passes the barrier and then
    // writes chunk c+2 (requested during chunk c-1) into buffer (c+2) % 3, which was last read when the fragments of
    // chunk c-1 were fetched; chunk c+1's buffer is complete behind that barrier, so its fragments are fetched into
    // the registers of each row fragment as soon as the chunk's last weight fragment has used them.
    // The prologue issues its loads in the loop's order (see mx_moe_gemm_kernel).
    AStage stage, stage2;
#pragma unroll
    for (int j = 0; j + 1 < D; ++j) load_b(j, j);
    load_a(stage, 0);
    load_a(stage2, 1);
    store_a(stage, lds);
    store_a(stage2, lds + A_BUF);
    load_a(stage, 2);
    load_b(D - 1, D - 1);
    __syncthreads();
    unsigned char *cur = lds, *nxt = lds + A_BUF, *fill = lds + 2 * A_BUF;
    static_for_n<MTW>([&](auto ic) __attribute__((always_inline)) { load_frag(cur, ic); });
    for (int c0 = 0; c0 < steps; c0 += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            const int c = c0 + j;
            const bool live = bs[j].valid;
#pragma unroll
            for (int f = 0; f < NT; ++f) asm volatile("" : "+v"(bs[j].q[f]), "+v"(bs[j].s[f]));
            static_for_n<NT>([&](auto fc) __attribute__((always_inline)) {
                constexpr int f = decltype(fc)::value;
                v8bf wb[4];
                mx_expand_block(bs[j].q[f], bs[j].s[f], wb);
                static_for_n<MTW>([&](auto ic) __attribute__((always_inline)) {
                    constexpr int i = decltype(ic)::value;
                    if (live && i * WR + wrow < frags) mfma_frag(wb, ic, fc);  // wave-uniform
                    if (f == NT - 1) load_frag(nxt, ic);
                });
                if (f == 0) {
                    __builtin_amdgcn_sched_barrier(0);
                    __syncthreads();
                    store_a(stage, fill);
                    load_a(stage, c + 3);
                    __builtin_amdgcn_sched_barrier(0);
                }
            });
            load_b(j, c + D);  // refill the set just consumed
            unsigned char *t = cur;
            cur = nxt;
            nxt = fill;
            fill = t;
        }
    }

    // ---- epilogue: acc[i][f][v] is row (i * WR + wrow) * 16 + 4 * grp + v, column fragment f, column r
#pragma unroll
    for (int i = 0; i < MTW; ++i)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int m = (i * WR + wrow) * 16 + 4 * grp + v;
            if (m >= rows) continue;
            const size_t orow = static_cast<size_t>(row0 + m) * g.N;
            if (GATED) {
#pragma unroll
                for (int p = 0; p < NT / 2; ++p)
                    if (col[2 * p] < g.N)
                        static_cast<__bf16 *>(g.out)[orow + col[2 * p]] =
                            static_cast<__bf16>(exact_swiglu(acc[i][2 * p][v], acc[i][2 * p + 1][v]));
            } else {
#pragma unroll
                for (int f = 0; f < NT; ++f)
                    if (col[f] < g.N) static_cast<float *>(g.out)[orow + col[f]] = acc[i][f][v];
            }
        }
}

// ---------------------------------------------------------------------------
// Direct form for a handful of routed rows (at most 4: one token's top-4, batch-1 decode), two launches.
//
// Gate|up: row tile t is routed entry t (expert sel[t], no plan); the token's row of x is staged whole in LDS once,
// the K loop is nothing but the weight stream, D chunks of weights in flight per wave.
// ---------------------------------------------------------------------------
struct MoeDirectExactArgs {
    const __bf16 *x;      // [T][K]
    const int *sel;       // [R]
    int a_div;            // routed entry / a_div = token
    const uint8_t *w_nib, *w_sc;
    int rows_per_expert, K, Kp, N;
    int n_experts, direct_rows;
    int *slot_of;         // gets the identity (or -1 for an entry that names no expert)
    __bf16 *act;          // [R][N]
};

// Stage `rows` bf16 rows of K elements (row stride `stride` elements) into the two-plane layout, zeros past K.
__device__ __forceinline__ void exact_stage_rows(unsigned char *lds, const __bf16 *src, size_t stride, int rows, int K,
                                                 int Kp, int a_row, int a_plane, int tid) {
    const int per_row = Kp / 8;  // 16-byte pieces per row
    for (int q = tid; q < rows * per_row; q += 256) {
        const int row = q / per_row, piece = q - row * per_row;
        const int chunk = piece >> 4, j = piece & 15;
        mu32x4 v = {0, 0, 0, 0};
        if (piece * 8 < K) v = *reinterpret_cast<const mu32x4 *>(src + row * stride + piece * 8);
        *reinterpret_cast<mu32x4 *>(lds + row * a_row + chunk * kChunk + exact_piece_offset(j, a_plane)) = v;
    }
}

// The leading arguments are what stands between the launch and the first weight load (sel[tile] -> expert -> address):
// as scalars they reach the wave in registers, where a by-value struct is read from the argument buffer first.
template <int D>
__global__ __launch_bounds__(256) void mx_moe_gateup_direct_exact_kernel(const int *sel, const uint8_t *w_nib, const uint8_t *w_sc,
                                                                         const __bf16 *x, int rows_per_expert, int k_in,
                                                                         int k_padded, int n_out, int n_experts,
                                                                         int direct_rows, MoeDirectExactArgs rest) {
    MoeDirectExactArgs g = rest;
    g.sel = sel; g.w_nib = w_nib; g.w_sc = w_sc; g.x = x;
    g.rows_per_expert = rows_per_expert; g.K = k_in; g.Kp = k_padded; g.N = n_out; g.n_experts = n_experts; g.direct_rows = direct_rows;
    constexpr int NT = 2;  // a gate fragment and its up fragment
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tile = blockIdx.y;
    if (tile >= g.direct_rows) return;
    const int expert = g.sel[tile];
    const bool known = expert >= 0 && expert < g.n_experts;
    if (blockIdx.x == 0 && threadIdx.x == 0) g.slot_of[tile] = known ? tile : -1;
    if (!known) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, grp = lane >> 4;
    const int Kp = g.Kp;
    const int chunks = Kp / kChunk;
    const int steps = (chunks + D - 1) / D * D;
    const int a_row = moe_small_pitch(Kp);
    const int a_plane = 16 * a_row;

    const int n0 = (blockIdx.x * 4 + wave) * 16;
    const int col = n0 + r;
    const uint8_t *w_tile[NT];
    const uint8_t *s_tile[NT];
#pragma unroll
    for (int f = 0; f < NT; ++f) {
        const int wrow0 = (f ? g.N : 0) + min(n0, g.N - 16);
        const size_t panel = (static_cast<size_t>(expert) * g.rows_per_expert + wrow0) >> 4;
        w_tile[f] = g.w_nib + (panel * chunks * 64 + lane) * 16;
        s_tile[f] = g.w_sc + panel * chunks * 64 + (lane & ~3);  // the dword that holds this lane's scale byte
    }
    const int s_shift = 8 * (lane & 3);
    BSet<1, NT> bs[D];
    auto load_b = [&](int set, int c) {
        bs[set].valid = c < chunks;
        const int cc = min(c, chunks - 1);
#pragma unroll
        for (int f = 0; f < NT; ++f) {
            bs[set].q[f] = __builtin_nontemporal_load(reinterpret_cast<const mu32x4 *>(w_tile[f] + static_cast<size_t>(cc) * 1024));
            bs[set].s[f] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(s_tile[f] + cc * 64));
        }
    };
    // Weights first: their trip to memory overlaps the staging of the activations.
#pragma unroll
    for (int j = 0; j < D; ++j) load_b(j, j);
    exact_stage_rows(lds, g.x + static_cast<size_t>(tile / g.a_div) * g.K, 0, 1, g.K, Kp, a_row, a_plane, tid);
    __syncthreads();

    v4f acc[NT];
#pragma unroll
    for (int f = 0; f < NT; ++f) acc[f] = v4f{0.f, 0.f, 0.f, 0.f};
    // Rows 1..15 of the tile hold whatever LDS held before; a row's products stay in that row's results, which are
    // never stored.
    const unsigned char *ap = lds + r * a_row + grp * 16;
    auto compute = [&](int set, int c) {
        const int cc = min(c, chunks - 1);
        const unsigned char *p = ap + cc * kChunk;
        v8bf a[4];
        a[0] = *reinterpret_cast<const v8bf *>(p);
        a[1] = *reinterpret_cast<const v8bf *>(p + 64);
        a[2] = *reinterpret_cast<const v8bf *>(p + a_plane);
        a[3] = *reinterpret_cast<const v8bf *>(p + a_plane + 64);
#pragma unroll
        for (int f = 0; f < NT; ++f) {
            asm volatile("" : "+v"(bs[set].q[f]), "+v"(bs[set].s[f]));
            const mu32x4 zero = {0, 0, 0, 0};
            const mu32x4 q = bs[set].valid ? bs[set].q[f] : zero;  // a dead chunk adds zeros
            v8bf wb[4];
            mx_expand_block(q, (bs[set].s[f] >> s_shift) & 0xffu, wb);
#pragma unroll
            for (int d = 0; d < 4; ++d) acc[f] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[d], wb[d], acc[f], 0, 0, 0);
            asm volatile("" : "+a"(acc[f]));
        }
    };
    for (int c0 = 0; c0 < steps; c0 += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            compute(j, c0 + j);
            __builtin_amdgcn_sched_barrier(0);
            load_b(j, c0 + j + D);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // row 0 of the fragment is the routed row: element 0 of the lanes of group 0
    if (grp == 0 && col < g.N) g.act[static_cast<size_t>(tile) * g.N + col] = static_cast<__bf16>(exact_swiglu(acc[0][0], acc[1][0]));
}

// Down projection of the routed rows with the weighted sum over a token's experts folded in (see
// mx_moe_down_direct_kernel: a workgroup owns 16 output columns for all routed rows, the four waves split K and meet
// in LDS, every wave requests its whole share of the weights before anything else).
struct MoeDownDirectExactArgs {
    const __bf16 *act;    // [R][K]
    const uint8_t *w_nib, *w_sc;
    int rows_per_expert, K, Kp, N;
    const int *sel;
    const float *wts;
    int R, topk, n_experts;
    float *out;           // [R][N]
    __bf16 *y;            // [R / topk][N]
};

__global__ __launch_bounds__(256) void mx_moe_down_direct_exact_kernel(const int *sel, const uint8_t *w_nib, const uint8_t *w_sc,
                                                                       const __bf16 *act, int rows_per_expert, int k_in,
                                                                       int k_padded, int n_out, int n_experts, int n_rows,
                                                                       MoeDownDirectExactArgs rest) {
    MoeDownDirectExactArgs g = rest;  // (leading scalars as in the gate/up kernel)
    g.sel = sel; g.w_nib = w_nib; g.w_sc = w_sc; g.act = act;
    g.rows_per_expert = rows_per_expert; g.K = k_in; g.Kp = k_padded; g.N = n_out; g.n_experts = n_experts; g.R = n_rows;
    constexpr int D = 8;  // chunks of a routed row per wave: K up to 4 * D * kChunk
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, grp = lane >> 4;
    const int Kp = g.Kp, chunks = Kp / kChunk, R = g.R;
    const int a_row = moe_small_pitch(Kp), a_plane = 16 * a_row;
    const int n0 = blockIdx.x * 16;  // N is a multiple of 16
    const int col = n0 + r;

    unsigned off_lo, off_hi, known;
    {
        const int t = lane & (kDirectRows - 1);
        const int e = t < R ? g.sel[t] : -1;
        const bool ok = e >= 0 && e < g.n_experts;
        const size_t off = ((static_cast<size_t>(ok ? e : 0) * g.rows_per_expert + n0) >> 4) * chunks * 64;
        off_lo = static_cast<unsigned>(off);
        off_hi = static_cast<unsigned>(off >> 32);
        known = static_cast<unsigned>(__ballot(ok)) & ((1u << kDirectRows) - 1u);
    }
    const uint8_t *w_lane = g.w_nib + lane * 16;
    const uint8_t *s_lane = g.w_sc + (lane & ~3);
    const int s_shift = 8 * (lane & 3);
    static_assert(D * 4 * kChunk >= 4096, "K up to 4096");
    BSet<1, 1> bs[kDirectRows][D];
#pragma unroll
    for (int t = 0; t < kDirectRows; ++t) {
        const int tc = min(t, R - 1);
        const size_t off = static_cast<size_t>(__builtin_amdgcn_readlane(off_hi, tc)) << 32 | __builtin_amdgcn_readlane(off_lo, tc);
        const uint8_t *wb = w_lane + off * 16;
        const uint8_t *sb = s_lane + off;
#pragma unroll
        for (int j = 0; j < D; ++j) {
            const int cc = min(wave + 4 * j, chunks - 1);
            bs[t][j].q[0] = __builtin_nontemporal_load(reinterpret_cast<const mu32x4 *>(wb + static_cast<size_t>(cc) * 1024));
            bs[t][j].s[0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(sb + cc * 64));
        }
    }
    exact_stage_rows(lds, g.act, static_cast<size_t>(g.K), R, g.K, Kp, a_row, a_plane, tid);
    __syncthreads();

    const unsigned char *ap = lds + r * a_row + grp * 16;
    float vals[kDirectRows];
#pragma unroll
    for (int t = 0; t < kDirectRows; ++t) {
        v4f acc = v4f{0.f, 0.f, 0.f, 0.f};
        const bool live = (t < R) & ((known >> t) & 1u);
#pragma unroll
        for (int j = 0; j < D; ++j) {
            const int c = wave + 4 * j;
            asm volatile("" : "+v"(bs[t][j].q[0]), "+v"(bs[t][j].s[0]));
            if (live & (c < chunks)) {  // wave-uniform
                const unsigned char *p = ap + c * kChunk;
                v8bf a[4], wb[4];
                a[0] = *reinterpret_cast<const v8bf *>(p);
                a[1] = *reinterpret_cast<const v8bf *>(p + 64);
                a[2] = *reinterpret_cast<const v8bf *>(p + a_plane);
                a[3] = *reinterpret_cast<const v8bf *>(p + a_plane + 64);
                mx_expand_block(bs[t][j].q[0], (bs[t][j].s[0] >> s_shift) & 0xffu, wb);
#pragma unroll
                for (int d = 0; d < 4; ++d) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[d], wb[d], acc, 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        vals[t] = acc[t];  // routed row t is row t of the fragment: element t of the lanes of group 0
    }

    __syncthreads();
    float *part = reinterpret_cast<float *>(lds);  // [4 waves][kDirectRows][16 columns]
    if (grp == 0) {
#pragma unroll
        for (int t = 0; t < kDirectRows; ++t) part[(wave * kDirectRows + t) * 16 + r] = vals[t];
    }
    __syncthreads();
    if (wave != 0 || grp != 0 || col >= g.N) return;
    float down[kDirectRows];
#pragma unroll
    for (int t = 0; t < kDirectRows; ++t) {
        down[t] = ((part[t * 16 + r] + part[(kDirectRows + t) * 16 + r]) + part[(2 * kDirectRows + t) * 16 + r]) +
                  part[(3 * kDirectRows + t) * 16 + r];
        if (t < R) g.out[static_cast<size_t>(t) * g.N + col] = ((known >> t) & 1u) ? down[t] : 0.f;
    }
    for (int token = 0; token * g.topk < R; ++token) {
        float a = 0.f;
        for (int sidx = 0; sidx < g.topk; ++sidx) {
            const int t = token * g.topk + sidx;
            const float d = t == 0 ? down[0] : t == 1 ? down[1] : t == 2 ? down[2] : down[3];
            if ((known >> t) & 1u) a = fmaf(g.wts[t], d, a);
        }
        g.y[static_cast<size_t>(token) * g.N + col] = static_cast<__bf16>(a);
    }
}

__global__ __launch_bounds__(1024) void moe_plan_kernel(const int *__restrict__ sel, int R, int E, int BM, MoePlan p) {
    moe_plan_block(sel, R, E, BM, p);
}

// act[r][k] = the bf16 activation the down GEMM consumed, down[r][h] = its f32 row, per routed entry.
__global__ __launch_bounds__(256) void moe_read_intermediates_exact_kernel(const int *__restrict__ slot_of,
                                                                           const __bf16 *__restrict__ a,
                                                                           const float *__restrict__ out,
                                                                           float *__restrict__ act, float *__restrict__ down,
                                                                           int R, int I, int H) {
    const int r = blockIdx.x;
    if (r >= R) return;
    const int slot = slot_of[r];
    if (act)
        for (int k = threadIdx.x; k < I; k += 256)
            act[static_cast<size_t>(r) * I + k] = slot >= 0 ? static_cast<float>(a[static_cast<size_t>(slot) * I + k]) : 0.f;
    if (down)
        for (int h = threadIdx.x; h < H; h += 256)
            down[static_cast<size_t>(r) * H + h] = slot >= 0 ? out[static_cast<size_t>(slot) * H + h] : 0.f;
}

template <int MT, int NT, bool GATED, int WR, int D>
static lhip_status launch_exact_gemm(const MoeExactArgs &a, int col_blocks, int max_tiles, hipStream_t s) {
    constexpr int BM = 16 * MT;
    const size_t lds_bytes = 3 * (2 * static_cast<size_t>(BM) * kARow);
    auto kern = mx_moe_gemm_exact_kernel<MT, NT, GATED, WR, D>;
    static LdsOptIn opt;
    if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(kern), lds_bytes)) return st;
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(col_blocks), static_cast<unsigned>(max_tiles)), dim3(256 * WR),
                       lds_bytes, s, a);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

// Tile height of the exact form for R routed rows over E experts: the smallest of 16, 32, 64 rows that holds an
// expert with two standard deviations more rows than the average (so that nearly every expert is one tile and its
// weights are read and expanded once); experts with more than 64 rows are cut into equal tiles of at most 64, whose
// later reads of the weights come out of the XCD's L2.  Measured on the benchmark layer (us per layer, 64-row tiles as
// four-wave workgroups two to a CU / 128-row tiles as eight-wave workgroups): T = 256 134 / 194, T = 512 187 / 207,
// T = 1024 274 / 342, T = 2048 458 / 530; and 16- / 32- / 64-row tiles: T = 32 87 / 94 / 110, T = 64 90 / 95 / 110,
// T = 128 132 / 99 / 114.
static inline int exact_tile_fragments(int R, int E) {
    const int avg = (R + E - 1) / E;
    const int need = avg + 2 * static_cast<int>(sqrtf(static_cast<float>(avg)) + 0.5f);
    return need <= 16 ? 1 : need <= 32 ? 2 : 4;
}

lhip_status moe_exact_forward(const uint8_t *gu, const uint8_t *dn, const __bf16 *x, const int32_t *sel_dev,
                              const float *wts_dev, __bf16 *y, int T, int H, int I, int E, int topk, MoeWorkspace &w,
                              hipStream_t s) {
    const int R = T * topk;
    const int Hp = static_cast<int>(pad128(H)), Ip = static_cast<int>(pad128(I));
    const uint8_t *gu_sc = gu + mx_scale_offset(static_cast<int64_t>(E) * 2 * I, H);
    const uint8_t *dn_sc = dn + mx_scale_offset(static_cast<int64_t>(E) * H, I);

    if (R <= kDirectRows && moe_small_lds_bytes(Hp) <= 150 * 1024 && moe_small_lds_bytes(Ip) <= 150 * 1024 && Ip <= 4096) {
        MoeDirectExactArgs a1{};
        a1.x = x; a1.sel = sel_dev; a1.a_div = topk;
        a1.w_nib = gu; a1.w_sc = gu_sc;
        a1.rows_per_expert = 2 * I; a1.K = H; a1.Kp = Hp; a1.N = I;
        a1.n_experts = E; a1.direct_rows = R; a1.slot_of = w.plan.slot_of; a1.act = w.act;
        {
            const size_t lds_bytes = moe_small_lds_bytes(Hp);
            auto kern = mx_moe_gateup_direct_exact_kernel<8>;
            static LdsOptIn opt;
            if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(kern), lds_bytes)) return st;
            hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>((I + 63) / 64), static_cast<unsigned>(R)), dim3(256), lds_bytes, s,
                               a1.sel, a1.w_nib, a1.w_sc, a1.x, a1.rows_per_expert, a1.K, a1.Kp, a1.N, a1.n_experts, a1.direct_rows, a1);
            LHIP_CHECK_LAUNCH();
        }
        MoeDownDirectExactArgs a2{};
        a2.act = w.act; a2.w_nib = dn; a2.w_sc = dn_sc;
        a2.rows_per_expert = H; a2.K = I; a2.Kp = Ip; a2.N = H;
        a2.sel = sel_dev; a2.wts = wts_dev; a2.R = R; a2.topk = topk; a2.n_experts = E;
        a2.out = w.out; a2.y = y;
        {
            const size_t lds_bytes = moe_small_lds_bytes(Ip);
            static LdsOptIn opt;
            if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(mx_moe_down_direct_exact_kernel), lds_bytes)) return st;
            hipLaunchKernelGGL(mx_moe_down_direct_exact_kernel, dim3(static_cast<unsigned>(H / 16)), dim3(256), lds_bytes, s,
                               a2.sel, a2.w_nib, a2.w_sc, a2.act, a2.rows_per_expert, a2.K, a2.Kp, a2.N, a2.n_experts, a2.R, a2);
            LHIP_CHECK_LAUNCH();
        }
        return LHIP_OK;
    }

    const int mt = exact_tile_fragments(R, E);
    const int BM = 16 * mt;
    const int max_tiles = (R / BM + E + 7) / 8 * 8;
    w.plan.max_tiles = max_tiles;
    w.plan.tiles_per_xcd = max_tiles / 8;
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(1024), 0, s, sel_dev, R, E, BM, w.plan);
    LHIP_CHECK_LAUNCH();

    MoeExactArgs a1{};
    a1.a = x; a1.a_index = w.plan.slot_src; a1.a_div = topk;
    a1.w_nib = gu; a1.w_sc = gu_sc;
    a1.rows_per_expert = 2 * I; a1.K = H; a1.Kp = Hp; a1.N = I;
    a1.tile_expert = w.plan.tile_expert; a1.tile_row0 = w.plan.tile_row0; a1.tile_rows = w.plan.tile_rows;
    a1.n_tiles = w.plan.n_tiles; a1.tiles_per_xcd = w.plan.tiles_per_xcd; a1.out = w.act;
    a1.tile_run0 = w.plan.tile_run0; a1.tile_runlen = w.plan.tile_runlen;
    const int cb1 = (I + 127) / 128;  // 4 waves x two (gate, up) pairs of 16 columns
    lhip_status st;
    switch (mt) {
        case 1: st = launch_exact_gemm<1, 4, true, 1, 4>(a1, cb1, max_tiles, s); break;
        case 2: st = launch_exact_gemm<2, 4, true, 1, 4>(a1, cb1, max_tiles, s); break;
        default: st = launch_exact_gemm<4, 4, true, 1, 2>(a1, cb1, max_tiles, s); break;
    }
    if (st) return st;
    MoeExactArgs a2{};
    a2.a = w.act; a2.a_index = nullptr; a2.a_div = 1;
    a2.w_nib = dn; a2.w_sc = dn_sc;
    a2.rows_per_expert = H; a2.K = I; a2.Kp = Ip; a2.N = H;
    a2.tile_expert = w.plan.tile_expert; a2.tile_row0 = w.plan.tile_row0; a2.tile_rows = w.plan.tile_rows;
    a2.n_tiles = w.plan.n_tiles; a2.tiles_per_xcd = w.plan.tiles_per_xcd; a2.out = w.out;
    a2.tile_run0 = w.plan.tile_run0; a2.tile_runlen = w.plan.tile_runlen;
    const int cb2 = (H + 127) / 128, cb2w = (H + 255) / 256;
    switch (mt) {
        case 1: st = launch_exact_gemm<1, 2, false, 1, 4>(a2, cb2, max_tiles, s); break;
        case 2: st = launch_exact_gemm<2, 2, false, 1, 4>(a2, cb2, max_tiles, s); break;
        default: st = launch_exact_gemm<4, 4, false, 1, 2>(a2, cb2w, max_tiles, s); break;
    }
    if (st) return st;
    return moe_launch_combine(w.out, w.plan.slot_of, wts_dev, y, T, H, topk, s);
}

lhip_status moe_exact_read_intermediates(const MoeWorkspace &w, float *act_dev, float *down_dev, int R, int I, int H,
                                         hipStream_t s) {
    hipLaunchKernelGGL(moe_read_intermediates_exact_kernel, dim3(static_cast<unsigned>(R)), dim3(256), 0, s,
                       w.plan.slot_of, w.act, w.out, act_dev, down_dev, R, I, H);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

}  // namespace lhip

using namespace lhip;

extern "C" {

lhip_status lhip_mxfp4_dequant_bf16(const void *planar_dev, void *out_bf16_dev, int64_t n, int64_t k, void *stream) {
    if (!planar_dev || !out_bf16_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_q8_shape(n, k)) return s;
    if (!aligned(planar_dev, 256) || !aligned(out_bf16_dev, 16)) return LHIP_ERR_MISALIGNED;
    auto *base = static_cast<const uint8_t *>(planar_dev);
    const size_t n_pieces = mx_scale_offset(n, k) / 16;
    hipLaunchKernelGGL(mx_dequant_bf16_kernel, dim3(static_cast<unsigned>((n_pieces + 255) / 256)), dim3(256), 0,
                       as_stream(stream), base, base + mx_scale_offset(n, k), static_cast<__bf16 *>(out_bf16_dev), n_pieces,
                       static_cast<int>(n), static_cast<int>(k), static_cast<int>(mx_chunks(k)));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

}  // extern "C"
