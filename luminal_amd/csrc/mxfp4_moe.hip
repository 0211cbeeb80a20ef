// MXFP4 mixture-of-experts layer on gfx950's block-scaled matrix instruction.
//
// Not in the reference (it has neither MXFP4 nor MoE); semantics follow its
// conventions: weights dequantise exactly (e2m1 * 2^(e8m0-127)), the expert MLP is
// luminal's SwiGLU  down( up(x) * swish(gate(x)) )  (examples/llama/src/model.rs:24-32,
// src/hl_ops/unary.rs:169-177), routing is top-k of the logits with a softmax
// over the selected k.
//
// v_mfma_scale_f32_16x16x128_f8f6f4 multiplies an fp8 operand by an fp4 operand
// and applies one e8m0 scale per 32-element block to each — exactly the MXFP4
// block structure — so the weights go from HBM into the instruction's
// registers untouched: no dequantisation arithmetic, no LDS traffic for them.
// Operand layout (measured on the part; lane l = (r, g) with r = l % 16,
// g = l / 16; a K chunk is 128 elements):
//   fp4 operand, 4 dwords : the 32 nibbles of block g (k in [32g, 32g+32)), even k low
//   fp8 operand, 8 dwords : bytes 0-15 = k in [16g, 16g+16), bytes 16-31 = k in [64+16g, +16)
//   scale (byte 0 of a VGPR): the e8m0 of (row r, block g), for either operand
//   result, 4 floats      : C[4g + i][r], rows from the first operand, columns from the second
// bf16 activations are not an MFMA input format here, so each activation is
// split exactly into two fp8 numbers: per 32-block, scale 2^s with
// max|x|/2^s in [128, 256); hi = fp8(x/2^s) keeps the top 4 significant bits,
// lo = fp8(32 (x/2^s - hi)) the remaining 4 of bf16's 8, multiplied with the
// block scale 2^(s-5): the residual is at most 8, so 32 times it stays inside
// fp8's range while its last bit stays above fp8's smallest step for every
// element down to 2^-14 of the block maximum (smaller ones are off by at most
// 2^-22 of the maximum; without the gain of 32 the bounds were 2^-9 and 2^-17,
// which shows on elements far below the block's scale).  Two MFMAs (hi, lo) per
// weight fragment then give the exact sum of exact products in f32, which is
// closer to the f32 semantics than a bf16 MFMA over rounded weights would be.
#include "mxfp4_moe_device.h"

namespace lhip {
// ---------------------------------------------------------------------------
// Router: top-k of the logits (ties to the lower index), softmax over the k.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void moe_route_kernel(const float *__restrict__ logits, int T, int E, int topk,
                                                        int *__restrict__ sel, float *__restrict__ wts) {
    const int t = blockIdx.x * 256 + threadIdx.x;
    if (t >= T) return;
    const float *l = logits + static_cast<size_t>(t) * E;
    int *s = sel + static_cast<size_t>(t) * topk;
    float *w = wts + static_cast<size_t>(t) * topk;
    for (int j = 0; j < topk; ++j) {
        int best = -1;
        float bv = 0.f;
        for (int e = 0; e < E; ++e) {
            bool taken = false;
            for (int r = 0; r < j; ++r) taken |= (s[r] == e);
            if (taken) continue;
            const float v = l[e];
            if (best < 0 || v > bv) {
                best = e;
                bv = v;
            }
        }
        s[j] = best;
    }
    const float mx = l[s[0]];
    float sum = 0.f;
    for (int j = 0; j < topk; ++j) {
        w[j] = expf(l[s[j]] - mx);
        sum += w[j];
    }
    const float inv = 1.0f / sum;
    for (int j = 0; j < topk; ++j) w[j] *= inv;
}

// One wavefront per token for E <= 64: lane e holds logit e; k rounds of a
// wave-wide arg-max (larger value wins, ties to the lower index).
__global__ __launch_bounds__(256) void moe_route_wave_kernel(const float *__restrict__ logits, int T, int E, int topk,
                                                             int *__restrict__ sel, float *__restrict__ wts) {
    const int lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (t >= T) return;
    float v = lane < E ? logits[static_cast<size_t>(t) * E + lane] : 0.f;
    bool avail = lane < E;
    float mx = 0.f, sum = 0.f, mine = 0.f;
    for (int j = 0; j < topk; ++j) {
        float bv = v;
        int bi = avail ? lane : 64;  // 64 = nothing to offer
        for (int o = 32; o > 0; o >>= 1) {
            const float ov = __shfl_xor(bv, o);
            const int oi = __shfl_xor(bi, o);
            const bool take = (oi < 64) && (bi == 64 || ov > bv || (ov == bv && oi < bi));
            if (take) {
                bv = ov;
                bi = oi;
            }
        }
        if (j == 0) mx = bv;
        const float w = expf(bv - mx);
        sum += w;
        if (lane == j) {
            mine = w;
            sel[static_cast<size_t>(t) * topk + j] = bi;
        }
        if (lane == bi) avail = false;
    }
    if (lane < topk) wts[static_cast<size_t>(t) * topk + lane] = mine * (1.0f / sum);
}

// ---------------------------------------------------------------------------
// Activation quantisation: bf16 rows -> fp8 hi plane, fp8 lo plane, e8m0 scales.
// One thread per 8 elements; the 4 threads of a 32-block share the maximum.
// Planes have row stride Kp = K rounded up to 128, zero-filled past K; the scale
// plane has row stride Kp/32, filled with 127 (2^0) past K.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void mx_quantize_act_item(size_t idx, const __bf16 *__restrict__ x, uint8_t *__restrict__ hi,
                                                     uint8_t *__restrict__ lo, uint8_t *__restrict__ sc, int rows, int K,
                                                     int Kp) {
    const int per_row = Kp / 8;
    const size_t row = idx / per_row;
    const int c8 = static_cast<int>(idx - row * per_row);
    const bool live = row < static_cast<size_t>(rows);
    const int k = c8 * 8;
    float v[8];
    mu32x4 raw = {0, 0, 0, 0};
    if (live && k < K) raw = *reinterpret_cast<const mu32x4 *>(x + row * K + k);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        v[2 * j] = __uint_as_float(raw[j] << 16);
        v[2 * j + 1] = __uint_as_float(raw[j] & 0xffff0000u);
    }
    float amax = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(v[j]));
    amax = fmaxf(amax, __shfl_xor(amax, 1));
    amax = fmaxf(amax, __shfl_xor(amax, 2));
    // scale 2^s with amax / 2^s in [128, 256): s = floor(log2 amax) - 7
    int e = 127;
    float inv = 1.0f;
    if (amax > 0.f && amax < __uint_as_float(0x7f800000u)) {
        const int ex = static_cast<int>((__float_as_uint(amax) >> 23) & 0xff);  // biased exponent (0 = subnormal)
        e = max(ex - 7, kLoShift + 1);                                                       // e8m0 code of 2^s
        inv = __uint_as_float(static_cast<uint32_t>(254 - e) << 23);              // 2^-s, exact
    }
    uint32_t ph[2], pl[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const float a0 = v[4 * j] * inv, a1 = v[4 * j + 1] * inv, a2 = v[4 * j + 2] * inv, a3 = v[4 * j + 3] * inv;
        int h = __builtin_amdgcn_cvt_pk_fp8_f32(a0, a1, 0, false);
        h = __builtin_amdgcn_cvt_pk_fp8_f32(a2, a3, h, true);
        const float r0 = a0 - __builtin_amdgcn_cvt_f32_fp8(h, 0), r1 = a1 - __builtin_amdgcn_cvt_f32_fp8(h, 1);
        const float r2 = a2 - __builtin_amdgcn_cvt_f32_fp8(h, 2), r3 = a3 - __builtin_amdgcn_cvt_f32_fp8(h, 3);
        int l = __builtin_amdgcn_cvt_pk_fp8_f32(r0 * kLoGain, r1 * kLoGain, 0, false);
        l = __builtin_amdgcn_cvt_pk_fp8_f32(r2 * kLoGain, r3 * kLoGain, l, true);
        ph[j] = static_cast<uint32_t>(h);
        pl[j] = static_cast<uint32_t>(l);
    }
    if (!live) return;
    *reinterpret_cast<uint2 *>(hi + row * Kp + k) = make_uint2(ph[0], ph[1]);
    *reinterpret_cast<uint2 *>(lo + row * Kp + k) = make_uint2(pl[0], pl[1]);
    if ((c8 & 3) == 0) sc[row * (Kp / 32) + (c8 >> 2)] = static_cast<uint8_t>(k < K ? e : 127);
}

// The two independent first steps of a layer pass in one launch: workgroup 0 makes the plan, the others
// quantise the layer input (1024 items each).
__global__ __launch_bounds__(1024) void moe_prepare_kernel(const int *__restrict__ sel, int R, int E, int BM, MoePlan p,
                                                           const __bf16 *__restrict__ x, uint8_t *__restrict__ hi,
                                                           uint8_t *__restrict__ lo, uint8_t *__restrict__ sc, int rows,
                                                           int K, int Kp) {
    if (blockIdx.x == 0)
        moe_plan_block(sel, R, E, BM, p);
    else
        mx_quantize_act_item(static_cast<size_t>(blockIdx.x - 1) * 1024 + threadIdx.x, x, hi, lo, sc, rows, K, Kp);
}

// ---------------------------------------------------------------------------
// Grouped expert GEMM.  grid = (column blocks, max tiles); a workgroup of 4 waves
// owns one row tile (up to BM = 16*MT routed rows of one expert) and 4*NT column
// fragments of 16.  GATED: fragments come in pairs, gate rows and the matching
// up rows, output bf16 up*swish(gate).  Otherwise f32 output.
// ---------------------------------------------------------------------------
struct MoeGemmArgs {
    const uint8_t *a_hi, *a_lo, *a_sc;  // activation planes, row stride Kp / Kp/32
    const int *a_index;                 // slot -> routed entry (GEMM 1) or nullptr (rows are slots)
    int a_div;                          // routed entry / a_div = activation row
    const uint8_t *w_nib, *w_sc;        // planar weights of all experts, rows_per_expert rows each
    int rows_per_expert;
    int K, Kp;
    int N;                              // output columns per expert (I or H)
    const int *tile_expert, *tile_row0, *tile_rows, *n_tiles;
    const int *tile_run0, *tile_runlen; // runs of tiles of one expert (MoePlan)
    int tiles_per_xcd;                  // layout of the tile list (MoePlan::tiles_per_xcd)
    void *out;                          // bf16 [R][N] (gated) or f32 [R][N]
    // Gated GEMM with NT == 4 only: when q_hi is set, the epilogue quantises its bf16 result for the next GEMM
    // (planes of row stride q_kp, scales of row stride q_kp / 32) instead of writing `out`.
    uint8_t *q_hi, *q_lo, *q_sc;
    int q_kp;
    // Direct form (a handful of routed rows, no plan launch in front): row tile t is routed entry t, its expert
    // sel[t]; the activations are the bf16 rows of x, quantised by the workgroup itself; slot_of gets the identity.
    const int *sel;
    const __bf16 *x;
    int *slot_of;
    int n_experts, direct_rows;
};


// WR = 1: 4 waves, each all MT row fragments x its NT column fragments.  WR = 2: 8 waves, the upper four
// take the odd row fragments, so every SIMD holds two waves with half the accumulators each
// and one wave's waits (LDS, barrier, weight stream) are covered by the other's matrix work.
// D = weight prefetch distance in chunks (even).
template <int MT, int NT, bool GATED, int WR, int D>
__global__ __launch_bounds__(256 * WR) __attribute__((amdgpu_waves_per_eu(1, (MT >= 8 && WR == 1) ? 1 : 8)))
void mx_moe_gemm_kernel(MoeGemmArgs g) {
    static_assert(!GATED || NT % 2 == 0, "gated tiles pair each gate fragment with its up fragment");
    static_assert(MT % WR == 0 && D % 2 == 0, "tile shape");
    constexpr int BM = 16 * MT;
    constexpr int MTW = MT / WR;      // row fragments per wave
    constexpr int THREADS = 256 * WR;
    constexpr int STG = MT / WR;      // 16-byte pieces of the activation tile staged per thread and chunk
    constexpr int A_PLANE = BM * kARow;
    constexpr int A_BUF = 2 * A_PLANE + BM * 4;  // hi, lo, scales

    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];  // 3 x A_BUF

    // Which tile and which column block.  Workgroups are dispatched in the order of their linear number
    // (x fastest) and dealt to the eight XCDs in turn, so the workgroups with the same number modulo 8 share an L2.
    // With a tile list laid out per XCD, those take the entries of their XCD's range in order, all column blocks
    // of one tile after another: the tile's activation rows, which every column block reads, come out of that L2
    // after their first use.  Where an expert was cut into a run of several tiles, the run is walked column block
    // by column block instead (all tiles of the run for one block, then the next block): the workgroups that read
    // the same weights are dispatched next to each other and share one fetch of them.  Entries without a tile have
    // no rows.
    int tile = blockIdx.y, cb = blockIdx.x;
    int expert, row0, rows;
    if (g.tiles_per_xcd) {
        const int linear = blockIdx.y * gridDim.x + blockIdx.x;
        const int turn = linear >> 3, cols = static_cast<int>(gridDim.x);
        const int base = (linear & 7) * g.tiles_per_xcd;
        const int entry = turn / cols;  // < gridDim.y / 8 = tiles_per_xcd
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
    const int wave = wave_id & 3;    // column group
    const int wrow = WR == 1 ? 0 : wave_id >> 2;  // row group
    const int r = lane & 15, grp = lane >> 4;
    const int Kp = g.Kp;
    const int chunks = Kp / kChunk;
    const int steps = (chunks + D - 1) / D * D;  // padded with dead chunks that add zero
    const int frags = (rows + 15) >> 4;          // row fragments of this tile that hold rows

    // ---- weight fragments: straight from global memory into MFMA registers.
    // The planar weights are tiled so that the 64 pieces a wave needs for one
    // fragment and one chunk are one contiguous KiB (lane order).
    const uint8_t *w_tile[NT];
    const uint8_t *s_tile[NT];
    int col[NT];
#pragma unroll
    for (int f = 0; f < NT; ++f) {
        int n0, wrow0;  // first column of the fragment, first weight row inside the expert
        if (GATED) {  // fragments 2p / 2p+1 = gate / up rows of the same 16 intermediate columns
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
        // Dead chunks (past the padded K; the refills of the last round) are zeroed by compute(); their requests go to one
        // line for the whole wave (aimed at the last chunk, a short tile would pull that kilobyte through memory again).
        // (Masking here, next to the loads, would make the wave wait for data it has only just requested.)
        bs[set].valid = c < chunks;
        const int cc = min(c, chunks - 1);
#pragma unroll
        for (int f = 0; f < NT; ++f) {
            // Short tiles (few routed rows per expert) read every weight once: keep them out of the caches.
            // Tall tiles come several per expert, and the later ones find the weights in L2 / the last-level cache.
            if (MT <= 2) {
                const uint8_t *wq = c < chunks ? w_tile[f] + static_cast<size_t>(cc) * 1024 : g.w_nib;
                bs[set].q[f] = __builtin_nontemporal_load(reinterpret_cast<const mu32x4 *>(wq));
                bs[set].s[f] = s_tile[f][cc * 64];  // (cached: the 64 scale bytes of two consecutive chunks share a line)
            } else {
                bs[set].q[f] = *reinterpret_cast<const mu32x4 *>(w_tile[f] + static_cast<size_t>(cc) * 1024);
                bs[set].s[f] = s_tile[f][cc * 64];
            }
        }
    };

    // ---- activation tile: global -> registers -> LDS (three buffers), shared by all waves
    const uint8_t *a_src[STG];
    int a_dst[STG];
#pragma unroll
    for (int i = 0; i < STG; ++i) {
        const int q = tid + i * THREADS;  // chunk of 16 bytes: plane, row, 16-byte column
        const int plane = q / (BM * 8), rem = q - plane * (BM * 8);
        const int row = rem >> 3, c16 = rem & 7;
        const int slot = row0 + min(row, rows - 1);  // rows past the tile re-read its last row (not stored)
        const int arow = g.a_index ? g.a_index[slot] / g.a_div : slot;
        a_src[i] = (plane ? g.a_lo : g.a_hi) + static_cast<size_t>(arow) * Kp + c16 * 16;
        a_dst[i] = plane * A_PLANE + row * kARow + c16 * 16;
    }
    const uint8_t *as_src = nullptr;
    if (tid < BM) {
        const int slot = row0 + min(tid, rows - 1);
        const int arow = g.a_index ? g.a_index[slot] / g.a_div : slot;
        as_src = g.a_sc + static_cast<size_t>(arow) * (Kp / 32);
    }
    struct AStage {
        mu32x4 q[STG];
        uint32_t s;
    };
    auto load_a = [&](AStage &st, int c) __attribute__((always_inline)) {
        const int cc = min(c, chunks - 1);  // dead chunks re-read the last one; they are not multiplied
#pragma unroll
        for (int i = 0; i < STG; ++i) st.q[i] = *reinterpret_cast<const mu32x4 *>(a_src[i] + cc * kChunk);
        if (tid < BM) st.s = *reinterpret_cast<const uint32_t *>(as_src + cc * 4);
    };
    auto store_a = [&](AStage &st, unsigned char *base) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < STG; ++i) {
            asm volatile("" : "+v"(st.q[i]));
            *reinterpret_cast<mu32x4 *>(base + a_dst[i]) = st.q[i];
        }
        if (tid < BM) *reinterpret_cast<uint32_t *>(base + 2 * A_PLANE + tid * 4) = st.s;
    };

    v4f acc[MTW][NT];
#pragma unroll
    for (int i = 0; i < MTW; ++i)
#pragma unroll
        for (int f = 0; f < NT; ++f) acc[i][f] = v4f{0.f, 0.f, 0.f, 0.f};

    // One row fragment of activations: fp8 hi and lo operands and the scale byte.
    struct AFrag {
        mu32x4 h0, h1, l0, l1;
        uint32_t sw;
    };
    // Fragment `n` of this wave's row group (tile fragment n * WR + wrow): the lane's part of the address is
    // fixed, so every read of a chunk is one base register plus an immediate offset.
    const int frag_lane = (wrow * 16 + r) * kARow + grp * 16;
    const int scale_lane = 2 * A_PLANE + (wrow * 16 + r) * 4;
    auto load_frag = [&](const unsigned char *base, int n) __attribute__((always_inline)) {
        const unsigned char *p = base + frag_lane + n * (WR * 16 * kARow);
        AFrag a;
        a.h0 = *reinterpret_cast<const mu32x4 *>(p);
        a.h1 = *reinterpret_cast<const mu32x4 *>(p + 64);
        a.l0 = *reinterpret_cast<const mu32x4 *>(p + A_PLANE);
        a.l1 = *reinterpret_cast<const mu32x4 *>(p + A_PLANE + 64);
        a.sw = *reinterpret_cast<const uint32_t *>(base + scale_lane + n * (WR * 16 * 4));
        return a;
    };
    // The MFMAs of row fragment i against the NT weight fragments of a set.
    auto mfma_frag = [&](int set, const AFrag &cur, int i) __attribute__((always_inline)) {
        const int sa = static_cast<int>((cur.sw >> (8 * grp)) & 0xff);
        const v8i ah = {(int)cur.h0.x, (int)cur.h0.y, (int)cur.h0.z, (int)cur.h0.w,
                        (int)cur.h1.x, (int)cur.h1.y, (int)cur.h1.z, (int)cur.h1.w};
        const v8i al = {(int)cur.l0.x, (int)cur.l0.y, (int)cur.l0.z, (int)cur.l0.w,
                        (int)cur.l1.x, (int)cur.l1.y, (int)cur.l1.z, (int)cur.l1.w};
#pragma unroll
        for (int f = 0; f < NT; ++f) {
            const mu32x4 &q = bs[set].q[f];
            const v8i b = {(int)q.x, (int)q.y, (int)q.z, (int)q.w, 0, 0, 0, 0};
            const int sb = static_cast<int>(bs[set].s[f]);
            acc[i][f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ah, b, acc[i][f], 0, 4, 0, sa, 0, sb);
            acc[i][f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(al, b, acc[i][f], 0, 4, 0, sa - kLoShift, 0, sb);
            // Pin the accumulation here: nothing else reads acc until the epilogue, and
            // without this the optimiser sinks every MFMA of the unrolled pipeline to its
            // end, keeping the fragments of all its steps alive.
            asm volatile("" : "+a"(acc[i][f]));
        }
    };

    // ---- pipeline: three LDS buffers, one barrier per chunk, placed in the MIDDLE of the chunk's matrix work.
    // Chunk c multiplies out of buffer c % 3.  After the MFMAs of its first row fragment every wave passes the
    // barrier and then writes chunk c+2 (requested during chunk c-1) into buffer (c+2) % 3: that buffer was last
    // read in chunk c-1, which every wave has left by then; and chunk c+2 is first read after the barrier of
    // chunk c+1, by when every wave has written it.  So nothing waits at a chunk boundary (the first fragment of
    // chunk c+1 is read right after the barrier of chunk c), a wave arriving at the barrier has its own and its
    // SIMD neighbour's MFMAs in flight, and the staging traffic runs under matrix work.
    // A dead chunk (past the padded K, there only to keep the unrolled shape) skips its MFMAs (wave-uniform).
    // The prologue issues its loads in the loop's order (activation stage, then the youngest weight set):
    // the compiler's wait counts inside the loop are the stricter of what the prologue and the previous
    // trip leave outstanding, and with the stage requested last here the loop would wait for the weight
    // set it has only just requested every time it stores a stage.
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
    AFrag first = load_frag(cur, 0);
    for (int c0 = 0; c0 < steps; c0 += D) {
#pragma unroll
        for (int j = 0; j < D; ++j) {
            const int c = c0 + j;
            const bool live = bs[j].valid;
#pragma unroll
            for (int f = 0; f < NT; ++f) asm volatile("" : "+v"(bs[j].q[f]), "+v"(bs[j].s[f]));
            // Two fragment buffers used alternately besides `first` (compile-time parity, so no register
            // copies); the LDS reads of fragment i+1 are issued before the MFMAs of fragment i and fenced
            // there.  Reads ahead are unconditional (they stay inside the staged tile); the matrix work stops at
            // the tile's last fragment.  Row fragments are dealt round-robin to the WR row groups, so a short
            // tile still occupies all waves.
            AFrag fr[2];
            if (MTW > 1) fr[1] = load_frag(cur, 1);
            __builtin_amdgcn_sched_barrier(0);
            if (live && wrow < frags) mfma_frag(j, first, 0);
            __builtin_amdgcn_sched_barrier(0);
            __syncthreads();
            if (MTW > 2) fr[0] = load_frag(cur, 2);
            store_a(stage, fill);
            load_a(stage, c + 3);
            first = load_frag(nxt, 0);
            __builtin_amdgcn_sched_barrier(0);
            if (live) {
                // Unrolled by template expansion (a pragma gives up on ten fragments with an exit test each, and
                // the accumulators, then indexed at run time, land in scratch memory).
                static_for_from1<MTW>([&](auto ic) __attribute__((always_inline)) {
                    constexpr int i = decltype(ic)::value;
                    if (i * WR + wrow < frags) {  // wave-uniform: the tile has rows there
                        if (i >= 2 && i + 1 < MTW) fr[(i + 1) & 1] = load_frag(cur, i + 1);
                        __builtin_amdgcn_sched_barrier(0);
                        mfma_frag(j, fr[i & 1], i);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                });
            }
            __builtin_amdgcn_sched_barrier(0);
            load_b(j, c + D);  // refill the set just consumed
            unsigned char *t = cur;
            cur = nxt;
            nxt = fill;
            fill = t;
        }
    }

    // ---- epilogue: acc[i][f][v] is row i*16 + 4*grp + v, column fragment f, column r
    if constexpr (GATED && NT == 4) {
        if (g.q_hi) {
            // The wave's two (gate, up) pairs are the 32 intermediate columns [32 b, 32 b + 32), b = 4 cb +
            // wave: one quantisation block of the next GEMM's activations.  Same arithmetic as
            // mx_quantize_act_item on the bf16-rounded result (block maximum over the 16 lanes of a row group),
            // so the intermediate activations never go through memory as bf16.
            const int b = cb * 4 + wave;
#pragma unroll
            for (int i = 0; i < MTW; ++i)
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int m = (i * WR + wrow) * 16 + 4 * grp + v;
                    if (m >= rows) continue;  // uniform over the 16 lanes that exchange values below
                    float a[2];
#pragma unroll
                    for (int p = 0; p < 2; ++p) {
                        const float gate = acc[i][2 * p][v], up = acc[i][2 * p + 1][v];
                        const float act = up * (gate * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * gate)));
                        a[p] = col[2 * p] < g.N ? static_cast<float>(static_cast<__bf16>(act)) : 0.f;
                    }
                    const float amax = row16_max(fmaxf(fabsf(a[0]), fabsf(a[1])));
                    int e = 127;
                    float inv = 1.0f;
                    if (amax > 0.f && amax < __uint_as_float(0x7f800000u)) {
                        const int ex = static_cast<int>((__float_as_uint(amax) >> 23) & 0xff);
                        e = max(ex - 7, kLoShift + 1);
                        inv = __uint_as_float(static_cast<uint32_t>(254 - e) << 23);
                    }
                    const float s0 = a[0] * inv, s1 = a[1] * inv;
                    const int h = __builtin_amdgcn_cvt_pk_fp8_f32(s0, s1, 0, false);
                    const float r0 = s0 - __builtin_amdgcn_cvt_f32_fp8(h, 0), r1 = s1 - __builtin_amdgcn_cvt_f32_fp8(h, 1);
                    const int l = __builtin_amdgcn_cvt_pk_fp8_f32(r0 * kLoGain, r1 * kLoGain, 0, false);
                    const size_t at = static_cast<size_t>(row0 + m) * g.q_kp + b * 32 + r;
                    g.q_hi[at] = static_cast<uint8_t>(h);
                    g.q_hi[at + 16] = static_cast<uint8_t>(h >> 8);
                    g.q_lo[at] = static_cast<uint8_t>(l);
                    g.q_lo[at + 16] = static_cast<uint8_t>(l >> 8);
                    if (r == 0)
                        g.q_sc[static_cast<size_t>(row0 + m) * (g.q_kp / 32) + b] = static_cast<uint8_t>(b * 32 < g.N ? e : 127);
                }
            return;
        }
    }
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
                    if (col[2 * p] < g.N) {
                        const float gate = acc[i][2 * p][v], up = acc[i][2 * p + 1][v];
                        // Hardware exp2 and reciprocal (1 ulp each): the result is rounded to bf16 right away,
                        // and the library forms cost more than the tile's matrix work is worth.
                        const float act = up * (gate * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * gate)));
                        static_cast<__bf16 *>(g.out)[orow + col[2 * p]] = static_cast<__bf16>(act);
                    }
            } else {
#pragma unroll
                for (int f = 0; f < NT; ++f)
                    if (col[f] < g.N) static_cast<float *>(g.out)[orow + col[f]] = acc[i][f][v];
            }
        }
}

// ---------------------------------------------------------------------------
// Decode-sized variant: row tiles of at most 16 routed rows (one row fragment).
// The tile's whole quantised activation rows (all of K) are staged in LDS once,
// so the K loop is nothing but the weight stream — no activation loads, no
// barriers — with D = 8 chunks of weights in flight per wave.  Needs
// 2 * 16 * pitch + 16 * Kp/32 bytes of LDS (K up to ~4.6k).
// ---------------------------------------------------------------------------
template <int NT, bool GATED, bool DIRECT = false, int D = 8>
__global__ __launch_bounds__(256) void mx_moe_gemm_small_kernel(MoeGemmArgs g) {
    static_assert(!GATED || NT % 2 == 0, "gated tiles pair each gate fragment with its up fragment");
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

    const int tile = blockIdx.y;
    int expert, row0, rows;
    if (DIRECT) {
        if (tile >= g.direct_rows) return;
        expert = g.sel[tile];
        const bool known = expert >= 0 && expert < g.n_experts;
        if (blockIdx.x == 0 && threadIdx.x == 0) g.slot_of[tile] = known ? tile : -1;
        if (!known) return;
        row0 = tile;
        rows = 1;
    } else {
        if (tile >= *g.n_tiles) return;
        expert = g.tile_expert[tile];
        row0 = g.tile_row0[tile];
        rows = g.tile_rows[tile];  // 1..16
    }

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, grp = lane >> 4;
    const int Kp = g.Kp;
    const int chunks = Kp / kChunk;
    const int steps = (chunks + D - 1) / D * D;
    const int a_row = moe_small_pitch(Kp);  // LDS bytes per activation row
    const int a_plane = 16 * a_row;
    const int sc_row = Kp / 32;            // scale bytes per row
    unsigned char *lds_sc = lds + 2 * a_plane;

    const uint8_t *w_tile[NT];
    const uint8_t *s_tile[NT];
    int col[NT];
#pragma unroll
    for (int f = 0; f < NT; ++f) {
        int n0, wrow0;
        if (GATED) {
            n0 = ((blockIdx.x * 4 + wave) * (NT / 2) + (f >> 1)) * 16;
            wrow0 = ((f & 1) ? g.N : 0) + min(n0, g.N - 16);
        } else {
            n0 = ((blockIdx.x * 4 + wave) * NT + f) * 16;
            wrow0 = min(n0, g.N - 16);
        }
        col[f] = n0 + r;
        const size_t panel = (static_cast<size_t>(expert) * g.rows_per_expert + wrow0) >> 4;
        w_tile[f] = g.w_nib + (panel * chunks * 64 + lane) * 16;
        s_tile[f] = g.w_sc + panel * chunks * 64 + (lane & ~3);  // the dword that holds this lane's scale byte
    }
    // A lane's scale is requested as the aligned dword around it and shifted down at its use: a byte load is
    // widened after the loop's phi, i.e. at the top of every trip for all D sets, and that widening waits for the
    // set requested last.
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
    // Weights first: their HBM round trip overlaps the staging of the activations.
#pragma unroll
    for (int j = 0; j < D; ++j) load_b(j, j);

    if (DIRECT) {
        // the routed entry's row of x, quantised here as the plan launch would have (groups of four threads share
        // a 32-block: Kp / 8 is a multiple of four, so a group is whole or absent)
        const __bf16 *x_row = g.x + static_cast<size_t>(tile / g.a_div) * g.K;
        for (int q = tid; q < Kp / 8; q += 256) mx_quantize_act_item(q, x_row, lds, lds + a_plane, lds_sc, 1, g.K, Kp);
    } else {
        const int per_row = Kp / 16;  // 16-byte pieces per row and plane
        const int pieces = rows * per_row * 2;
        for (int q = tid; q < pieces; q += 256) {
            const int plane = q / (rows * per_row), rem = q - plane * (rows * per_row);
            const int row = rem / per_row, c16 = rem - row * per_row;
            const int slot = row0 + row;
            const int arow = g.a_index ? g.a_index[slot] / g.a_div : slot;
            const mu32x4 v = *reinterpret_cast<const mu32x4 *>((plane ? g.a_lo : g.a_hi) +
                                                                static_cast<size_t>(arow) * Kp + c16 * 16);
            *reinterpret_cast<mu32x4 *>(lds + plane * a_plane + row * a_row + c16 * 16) = v;
        }
        const int sc_words = rows * (sc_row / 4);
        for (int q = tid; q < sc_words; q += 256) {
            const int row = q / (sc_row / 4), w4 = q - row * (sc_row / 4);
            const int slot = row0 + row;
            const int arow = g.a_index ? g.a_index[slot] / g.a_div : slot;
            reinterpret_cast<uint32_t *>(lds_sc + row * sc_row)[w4] =
                reinterpret_cast<const uint32_t *>(g.a_sc + static_cast<size_t>(arow) * sc_row)[w4];
        }
    }
    __syncthreads();

    v4f acc[NT];
#pragma unroll
    for (int f = 0; f < NT; ++f) acc[f] = v4f{0.f, 0.f, 0.f, 0.f};

    // Rows past the tile hold stale LDS bytes; their results are never stored.
    const unsigned char *ap = lds + r * a_row + grp * 16;
    const unsigned char *sp = lds_sc + r * sc_row + grp;
    auto compute = [&](int set, int c) {
        const int cc = min(c, chunks - 1);
        const unsigned char *p = ap + cc * kChunk;
        const mu32x4 h0 = *reinterpret_cast<const mu32x4 *>(p);
        const mu32x4 h1 = *reinterpret_cast<const mu32x4 *>(p + 64);
        const mu32x4 l0 = *reinterpret_cast<const mu32x4 *>(p + a_plane);
        const mu32x4 l1 = *reinterpret_cast<const mu32x4 *>(p + a_plane + 64);
        const int sa = sp[cc * 4];
        const v8i ah = {(int)h0.x, (int)h0.y, (int)h0.z, (int)h0.w, (int)h1.x, (int)h1.y, (int)h1.z, (int)h1.w};
        const v8i al = {(int)l0.x, (int)l0.y, (int)l0.z, (int)l0.w, (int)l1.x, (int)l1.y, (int)l1.z, (int)l1.w};
#pragma unroll
        for (int f = 0; f < NT; ++f) {
            asm volatile("" : "+v"(bs[set].q[f]), "+v"(bs[set].s[f]));
            const mu32x4 zero = {0, 0, 0, 0};
            const mu32x4 q = bs[set].valid ? bs[set].q[f] : zero;
            const int sb = bs[set].valid ? static_cast<int>(bs[set].s[f] >> s_shift) : 127;  // the matrix core reads byte 0
            const v8i b = {(int)q.x, (int)q.y, (int)q.z, (int)q.w, 0, 0, 0, 0};
            acc[f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ah, b, acc[f], 0, 4, 0, sa, 0, sb);
            acc[f] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(al, b, acc[f], 0, 4, 0, sa - kLoShift, 0, sb);
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

    if constexpr (GATED && NT == 2) {
        if (g.q_hi) {
            // Quantise the result for the next GEMM here (same arithmetic as mx_quantize_act_item on the
            // bf16-rounded values).  A wave holds 16 of a block's 32 columns; the two waves of a block exchange
            // their row maxima through LDS, which the K loop no longer needs.
            __syncthreads();  // every wave is done reading the staged activations
            float *pmax = reinterpret_cast<float *>(lds);  // [4 waves][16 rows]
            float a[4];
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float gate = acc[0][v], up = acc[1][v];
                const float act = up * (gate * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * gate)));
                a[v] = col[0] < g.N ? static_cast<float>(static_cast<__bf16>(act)) : 0.f;
                const float mx = row16_max(fabsf(a[v]));
                if (r == 0) pmax[wave * 16 + 4 * grp + v] = mx;
            }
            __syncthreads();
            const int b = blockIdx.x * 2 + (wave >> 1);  // quantisation block of this wave's columns
            const int half = (wave & 1) * 16;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const int m = 4 * grp + v;
                if (m >= rows) continue;
                const float amax = fmaxf(pmax[wave * 16 + m], pmax[(wave ^ 1) * 16 + m]);
                int e = 127;
                float inv = 1.0f;
                if (amax > 0.f && amax < __uint_as_float(0x7f800000u)) {
                    const int ex = static_cast<int>((__float_as_uint(amax) >> 23) & 0xff);
                    e = max(ex - 7, kLoShift + 1);
                    inv = __uint_as_float(static_cast<uint32_t>(254 - e) << 23);
                }
                const float s0 = a[v] * inv;
                const int h = __builtin_amdgcn_cvt_pk_fp8_f32(s0, 0.f, 0, false);
                const int l = __builtin_amdgcn_cvt_pk_fp8_f32((s0 - __builtin_amdgcn_cvt_f32_fp8(h, 0)) * kLoGain, 0.f, 0, false);
                const size_t at = static_cast<size_t>(row0 + m) * g.q_kp + b * 32 + half + r;
                g.q_hi[at] = static_cast<uint8_t>(h);
                g.q_lo[at] = static_cast<uint8_t>(l);
                const size_t sc_at = static_cast<size_t>(row0 + m) * (g.q_kp / 32);
                if (r == 0 && half == 0) g.q_sc[sc_at + b] = static_cast<uint8_t>(e);
                // The last column block also fills the padding past N up to the padded row length: zeros, scale 2^0.
                if (blockIdx.x == gridDim.x - 1 && wave == 0) {
                    const int k0 = (g.N + 63) / 64 * 64;  // the column blocks end here
                    for (int k = k0 + r; k < g.q_kp; k += 16) {
                        g.q_hi[static_cast<size_t>(row0 + m) * g.q_kp + k] = 0;
                        g.q_lo[static_cast<size_t>(row0 + m) * g.q_kp + k] = 0;
                    }
                    if (r == 0)
                        for (int kb = k0 / 32; kb < g.q_kp / 32; ++kb) g.q_sc[sc_at + kb] = 127;
                }
            }
            return;
        }
    }
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int m = 4 * grp + v;
        if (m >= rows) continue;
        const size_t orow = static_cast<size_t>(row0 + m) * g.N;
        if (GATED) {
#pragma unroll
            for (int p = 0; p < NT / 2; ++p)
                if (col[2 * p] < g.N) {
                    const float gate = acc[2 * p][v], up = acc[2 * p + 1][v];
                    const float act = up * (gate * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.44269504f * gate)));
                    static_cast<__bf16 *>(g.out)[orow + col[2 * p]] = static_cast<__bf16>(act);
                }
        } else {
#pragma unroll
            for (int f = 0; f < NT; ++f)
                if (col[f] < g.N) static_cast<float *>(g.out)[orow + col[f]] = acc[f][v];
        }
    }
}

// ---------------------------------------------------------------------------
// Down projection of a handful of routed rows (at most 4: one token's top-4) with the weighted sum over a token's
// experts folded in, for the direct form: no plan, no combine launch.  A workgroup owns 16 output columns for
// ALL routed rows: routed row t multiplies the 16 weight rows of expert sel[t]; the four waves split K (chunk c
// belongs to wave c % 4) and meet in LDS, then y[token][col] = bf16(sum_s wts * down) in the combine kernel's
// order.  The rows' quantised activations (all of K) are staged in LDS once; a wave requests its whole share of
// the weights (all routed rows, K up to 4096) before anything else and holds it in registers.
// ---------------------------------------------------------------------------

struct MoeDownDirectArgs {
    const uint8_t *a_hi, *a_lo, *a_sc;  // quantised activations: R rows of Kp / Kp/32 bytes, row = routed entry
    const uint8_t *w_nib, *w_sc;        // planar down weights of all experts, rows_per_expert rows each
    int rows_per_expert, Kp, N;
    const int *sel;
    const float *wts;
    int R, topk, n_experts;
    float *out;                         // [R][N] f32 rows (read back by lhip_mxfp4_moe_read_intermediates)
    __bf16 *y;                          // [R / topk][N]
};

__global__ __launch_bounds__(256) void mx_moe_down_direct_kernel(MoeDownDirectArgs g) {
    constexpr int D = 8;  // chunks of a routed row per wave: K up to 4 * D * kChunk
    extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, grp = lane >> 4;
    const int Kp = g.Kp, chunks = Kp / kChunk, R = g.R;
    const int a_row = moe_small_pitch(Kp), a_plane = 16 * a_row, sc_row = Kp / 32;
    unsigned char *lds_sc = lds + 2 * a_plane;
    const int n0 = blockIdx.x * 16;  // N is a multiple of 16
    const int col = n0 + r;

    // Per routed row: where its expert's weights start (lane t of a register pair holds routed row t's, read with
    // v_readlane) and whether it names a real expert (a bit mask).  The loads below stay free of branches and of
    // selects between 64-bit scalars (which compile to branches): a branch between loads makes the compiler's
    // wait counts for the sets in flight fall back to "wait for everything".
    unsigned off_lo, off_hi, known;
    {
        const int t = lane & (kDirectRows - 1);
        const int e = t < R ? g.sel[t] : -1;
        const bool ok = e >= 0 && e < g.n_experts;
        const size_t off = ((static_cast<size_t>(ok ? e : 0) * g.rows_per_expert + n0) >> 4) * chunks * 64;
        off_lo = static_cast<unsigned>(off);
        off_hi = static_cast<unsigned>(off >> 32);
        known = static_cast<unsigned>(__ballot(ok)) & ((1u << kDirectRows) - 1u);  // lanes 0..3 are rows 0..3
    }
    const uint8_t *w_lane = g.w_nib + lane * 16;
    const uint8_t *s_lane = g.w_sc + (lane & ~3);
    const int s_shift = 8 * (lane & 3);
    // Chunk wave + 4 * j of routed row t is weight set (t, j), j < D: all of a wave's share - at most
    // kDirectRows * D kilobytes - is requested up front and held in registers (a workgroup has the SIMDs to
    // itself: 512 registers per lane), so the whole launch costs one trip to memory instead of one per D chunks.
    static_assert(D * 4 * kChunk >= 4096, "K up to 4096");
    BSet<1, 1> bs[kDirectRows][D];
#pragma unroll
    for (int t = 0; t < kDirectRows; ++t) {
        const int tc = min(t, R - 1);  // rows past R re-read the last row's lines: never used
        const size_t off = static_cast<size_t>(__builtin_amdgcn_readlane(off_hi, tc)) << 32 | __builtin_amdgcn_readlane(off_lo, tc);
        const uint8_t *wb = w_lane + off * 16;
        const uint8_t *sb = s_lane + off;
#pragma unroll
        for (int j = 0; j < D; ++j) {
            const int cc = min(wave + 4 * j, chunks - 1);  // chunks past the end re-read the last one: never used
            bs[t][j].q[0] = __builtin_nontemporal_load(reinterpret_cast<const mu32x4 *>(wb + static_cast<size_t>(cc) * 1024));
            bs[t][j].s[0] = __builtin_nontemporal_load(reinterpret_cast<const uint32_t *>(sb + cc * 64));
        }
    }
    {
        const int per_row = Kp / 16;
        const int pieces = R * per_row * 2;
        for (int q = tid; q < pieces; q += 256) {
            const int plane = q / (R * per_row), rem = q - plane * (R * per_row);
            const int row = rem / per_row, c16 = rem - row * per_row;
            const mu32x4 v = *reinterpret_cast<const mu32x4 *>((plane ? g.a_lo : g.a_hi) + static_cast<size_t>(row) * Kp + c16 * 16);
            *reinterpret_cast<mu32x4 *>(lds + plane * a_plane + row * a_row + c16 * 16) = v;
        }
        const int sc_words = R * (sc_row / 4);
        for (int q = tid; q < sc_words; q += 256) {
            const int row = q / (sc_row / 4), w4 = q - row * (sc_row / 4);
            reinterpret_cast<uint32_t *>(lds_sc + row * sc_row)[w4] =
                reinterpret_cast<const uint32_t *>(g.a_sc + static_cast<size_t>(row) * sc_row)[w4];
        }
    }
    __syncthreads();

    // Rows past R hold stale LDS bytes; their results are never used.
    const unsigned char *ap = lds + r * a_row + grp * 16;
    const unsigned char *sp = lds_sc + r * sc_row + grp;
    float vals[kDirectRows];  // this wave's share of routed row t's 16 outputs (lanes 0..15)
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
                const mu32x4 h0 = *reinterpret_cast<const mu32x4 *>(p);
                const mu32x4 h1 = *reinterpret_cast<const mu32x4 *>(p + 64);
                const mu32x4 l0 = *reinterpret_cast<const mu32x4 *>(p + a_plane);
                const mu32x4 l1 = *reinterpret_cast<const mu32x4 *>(p + a_plane + 64);
                const int sa = sp[c * 4];
                const v8i ah = {(int)h0.x, (int)h0.y, (int)h0.z, (int)h0.w, (int)h1.x, (int)h1.y, (int)h1.z, (int)h1.w};
                const v8i al = {(int)l0.x, (int)l0.y, (int)l0.z, (int)l0.w, (int)l1.x, (int)l1.y, (int)l1.z, (int)l1.w};
                const mu32x4 q = bs[t][j].q[0];
                const int sb = static_cast<int>(bs[t][j].s[0] >> s_shift);
                const v8i b = {(int)q.x, (int)q.y, (int)q.z, (int)q.w, 0, 0, 0, 0};
                acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(ah, b, acc, 0, 4, 0, sa, 0, sb);
                acc = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(al, b, acc, 0, 4, 0, sa - kLoShift, 0, sb);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        vals[t] = acc[t];  // routed row t is row t of the fragment
    }

    __syncthreads();  // every wave is done reading the staged activations
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

// y[t][h] = bf16( sum_s wts[t][s] * out[slot_of[t*topk+s]][h] ), 4 columns per thread
__global__ __launch_bounds__(256) void moe_combine_kernel(const float *__restrict__ out, const int *__restrict__ slot_of,
                                                          const float *__restrict__ wts, __bf16 *__restrict__ y, int T,
                                                          int H, int topk) {
    const int h4 = H / 4;
    const size_t idx = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (idx >= static_cast<size_t>(T) * h4) return;
    const int t = static_cast<int>(idx / h4), c = static_cast<int>(idx - static_cast<size_t>(t) * h4);
    float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s = 0; s < topk; ++s) {
        const int slot = slot_of[t * topk + s];
        if (slot < 0) continue;
        const float w = wts[t * topk + s];
        const float4 v = reinterpret_cast<const float4 *>(out + static_cast<size_t>(slot) * H)[c];
        a.x = fmaf(w, v.x, a.x);
        a.y = fmaf(w, v.y, a.y);
        a.z = fmaf(w, v.z, a.z);
        a.w = fmaf(w, v.w, a.w);
    }
    __bf16 *o = y + static_cast<size_t>(t) * H + c * 4;
    o[0] = static_cast<__bf16>(a.x);
    o[1] = static_cast<__bf16>(a.y);
    o[2] = static_cast<__bf16>(a.z);
    o[3] = static_cast<__bf16>(a.w);
}

// What the two GEMMs of the last layer pass left in the workspace, per routed entry r = t*topk + s (not per slot):
// act[r][k] = the SwiGLU activation as the down GEMM consumed it, (hi + lo) * 2^(scale - 127) of its two fp8
// planes, and down[r][h] = the down projection's f32 row.  Entries whose expert id was invalid give zeros.
__global__ __launch_bounds__(256) void moe_read_intermediates_kernel(const int *__restrict__ slot_of,
                                                                     const uint8_t *__restrict__ a_hi,
                                                                     const uint8_t *__restrict__ a_lo,
                                                                     const uint8_t *__restrict__ a_sc,
                                                                     const float *__restrict__ out, float *__restrict__ act,
                                                                     float *__restrict__ down, int R, int I, int Ip, int H) {
    const int r = blockIdx.x;
    if (r >= R) return;
    const int slot = slot_of[r];
    if (act) {
        for (int k = threadIdx.x; k < I; k += 256) {
            float v = 0.f;
            if (slot >= 0) {
                const size_t at = static_cast<size_t>(slot) * Ip + k;
                const float hi = __builtin_amdgcn_cvt_f32_fp8(a_hi[at], 0), lo = __builtin_amdgcn_cvt_f32_fp8(a_lo[at], 0);
                const uint32_t e = a_sc[static_cast<size_t>(slot) * (Ip / 32) + (k >> 5)];
                v = (hi + lo * (1.0f / kLoGain)) * __uint_as_float(e << 23);  // e > kLoShift: the quantiser's floor
            }
            act[static_cast<size_t>(r) * I + k] = v;
        }
    }
    if (down)
        for (int h = threadIdx.x; h < H; h += 256)
            down[static_cast<size_t>(r) * H + h] = slot >= 0 ? out[static_cast<size_t>(slot) * H + h] : 0.f;
}

template <int MT, int NT, bool GATED, int WR = 1, int D = 4>
static lhip_status launch_moe_gemm(const MoeGemmArgs &a, int col_blocks, int max_tiles, hipStream_t s) {
    constexpr int BM = 16 * MT;
    const size_t lds_bytes = 3 * (2 * static_cast<size_t>(BM) * kARow + BM * 4);
    auto kern = mx_moe_gemm_kernel<MT, NT, GATED, WR, D>;
    static LdsOptIn opt;
    if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(kern), lds_bytes)) return st;
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(col_blocks), static_cast<unsigned>(max_tiles)), dim3(256 * WR),
                       lds_bytes, s, a);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}


template <int NT, bool GATED>
static lhip_status launch_moe_gemm_small(const MoeGemmArgs &a, int col_blocks, int max_tiles, hipStream_t s) {
    const size_t lds_bytes = moe_small_lds_bytes(a.Kp);
    auto kern = mx_moe_gemm_small_kernel<NT, GATED>;
    static LdsOptIn opt;
    if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(kern), lds_bytes)) return st;
    hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>(col_blocks), static_cast<unsigned>(max_tiles)), dim3(256),
                       lds_bytes, s, a);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

// Scratch memory of lhip_mxfp4_moe_bf16_static: the layer's workspace for callers that cannot allocate one.  One copy
// per device, held until the process ends; every call of that entry point on a device shares it.
constexpr size_t kMoeStaticBytes = size_t{8} << 20;
static __device__ __align__(256) unsigned char scratch[kMoeStaticBytes];

// Device address of `scratch` on the current device (in host code the array's name is not a device address): asked
// for once per device, with that device current, and kept.
static lhip_status moe_scratch_address(unsigned char **out) {
    static unsigned char *ptrs[64] = {};
    int dev = 0;
    LHIP_HIP_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64) return LHIP_ERR_UNSUPPORTED;
    unsigned char *p = __atomic_load_n(&ptrs[dev], __ATOMIC_ACQUIRE);
    if (!p) {
        LHIP_HIP_TRY(hipGetSymbolAddress(reinterpret_cast<void **>(&p), HIP_SYMBOL(scratch)));
        if (!p) return LHIP_ERR_HIP;
        __atomic_store_n(&ptrs[dev], p, __ATOMIC_RELEASE);
    }
    *out = p;
    return LHIP_OK;
}

// Called by lhip_init for the device it selects, so that the first lhip_mxfp4_moe_bf16_static call finds the address.
lhip_status moe_static_setup() {
    unsigned char *p = nullptr;
    return moe_scratch_address(&p);
}

lhip_status moe_launch_combine(const float *out, const int *slot_of, const float *wts, __bf16 *y, int T, int H, int topk,
                               hipStream_t s) {
    const size_t threads = static_cast<size_t>(T) * (H / 4);
    hipLaunchKernelGGL(moe_combine_kernel, dim3(static_cast<unsigned>((threads + 255) / 256)), dim3(256), 0, s, out, slot_of,
                       wts, y, T, H, topk);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

static lhip_status check_moe_shape(int64_t T, int64_t H, int64_t I, int64_t E, int64_t topk) {
    if (T <= 0 || H <= 0 || I <= 0 || E <= 0 || topk <= 0) return LHIP_ERR_INVALID_SHAPE;
    if (E > 1024 || topk > E || T * topk > (int64_t{1} << 24)) return LHIP_ERR_INVALID_SHAPE;
    if (H % 32 != 0 || I % 32 != 0 || H > kMaxDim || I > kMaxDim) return LHIP_ERR_INVALID_SHAPE;  // so % 16 == 0 too
    return LHIP_OK;
}

}  // namespace lhip

using namespace lhip;

extern "C" {

lhip_status lhip_moe_route_topk(const float *logits_dev, int32_t *sel_dev, float *wts_dev, int64_t t, int64_t e,
                                int64_t topk, void *stream) {
    if (!logits_dev || !sel_dev || !wts_dev) return LHIP_ERR_NULL_PTR;
    if (t <= 0 || e <= 0 || topk <= 0 || topk > e || t > kMaxDim || e > 1024) return LHIP_ERR_INVALID_SHAPE;
    if (e <= 64 && topk <= 64)
        hipLaunchKernelGGL(moe_route_wave_kernel, dim3(static_cast<unsigned>((t + 3) / 4)), dim3(256), 0,
                           as_stream(stream), logits_dev, static_cast<int>(t), static_cast<int>(e),
                           static_cast<int>(topk), sel_dev, wts_dev);
    else
        hipLaunchKernelGGL(moe_route_kernel, dim3(static_cast<unsigned>((t + 255) / 256)), dim3(256), 0,
                           as_stream(stream), logits_dev, static_cast<int>(t), static_cast<int>(e),
                           static_cast<int>(topk), sel_dev, wts_dev);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

size_t lhip_mxfp4_moe_workspace_nbytes(int64_t t, int64_t h, int64_t i, int64_t e, int64_t topk) {
    if (check_moe_shape(t, h, i, e, topk) != LHIP_OK) return 0;
    return carve(nullptr, t, h, i, e, topk).total;
}

lhip_status lhip_mxfp4_moe_bf16(const void *w_gate_up_planar, const void *w_down_planar, const void *x_dev,
                                const int32_t *sel_dev, const float *wts_dev, void *y_dev, int64_t t, int64_t h,
                                int64_t i, int64_t e, int64_t topk, void *workspace_dev, void *stream) {
    return lhip_mxfp4_moe_bf16_mode(w_gate_up_planar, w_down_planar, x_dev, sel_dev, wts_dev, y_dev, t, h, i, e, topk,
                                    LHIP_MOE_EXACT, workspace_dev, stream);
}

lhip_status lhip_mxfp4_moe_bf16_mode(const void *w_gate_up_planar, const void *w_down_planar, const void *x_dev,
                                     const int32_t *sel_dev, const float *wts_dev, void *y_dev, int64_t t, int64_t h,
                                     int64_t i, int64_t e, int64_t topk, int32_t mode, void *workspace_dev, void *stream) {
    if (!w_gate_up_planar || !w_down_planar || !x_dev || !sel_dev || !wts_dev || !y_dev || !workspace_dev)
        return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_moe_shape(t, h, i, e, topk)) return s;
    if (h % 4 != 0) return LHIP_ERR_INVALID_SHAPE;
    if (mode != LHIP_MOE_EXACT && mode != LHIP_MOE_FAST) return LHIP_ERR_UNSUPPORTED;
    if (!aligned(w_gate_up_planar, 256) || !aligned(w_down_planar, 256) || !aligned(x_dev, 16) ||
        !aligned(workspace_dev, 256) || !aligned(y_dev, 2))
        return LHIP_ERR_MISALIGNED;
    hipStream_t s = as_stream(stream);
    const int T = static_cast<int>(t), H = static_cast<int>(h), I = static_cast<int>(i), E = static_cast<int>(e);
    const int topk_i = static_cast<int>(topk), R = T * topk_i;
    MoeWorkspace w = carve(workspace_dev, t, h, i, e, topk);
    if (mode == LHIP_MOE_EXACT)
        return moe_exact_forward(static_cast<const uint8_t *>(w_gate_up_planar), static_cast<const uint8_t *>(w_down_planar),
                                 static_cast<const __bf16 *>(x_dev), sel_dev, wts_dev, static_cast<__bf16 *>(y_dev), T, H, I,
                                 E, topk_i, w, s);
    const int Hp = static_cast<int>(pad128(h)), Ip = static_cast<int>(pad128(i));

    // Row tile.  Up to 128 rows: the smallest height that holds an expert with two standard deviations more rows
    // than the average (rows per expert are roughly Poisson), so that nearly every expert is one tile and its
    // weights are read once.  Heights of 64 and 80 rows run as four-wave workgroups, two to a CU: each wave then
    // has four or five row fragments of matrix work per weight fragment it loads, enough to cover the two chunks
    // of weights it keeps in flight, and one workgroup's prologue, barrier and epilogue run under the other's
    // matrix work.  Experts with more rows than 128 are cut into 80-row tiles as well: their second and third
    // reads of the weights come out of L2 / the last-level cache, and a short last tile wastes less than it does
    // at 160 rows (measured, us per layer, 80-row / 160-row tiles: T = 1024 269-275 / 272-281, T = 1536 375 / 419,
    // T = 2048 485 / 486, T = 4096 885 / 930; and at T = 512 80-row / 128-row tiles: 161 / 183-201).
    const int avg = (R + E - 1) / E;
    const int need = avg + 2 * static_cast<int>(sqrtf(static_cast<float>(avg)) + 0.5f);
    const int mt = need <= 16 ? 1 : need <= 32 ? 2 : need <= 64 ? 4 : need <= 80 ? 5 : need <= 128 ? 8 : 5;
    const int BM = 16 * mt;
    const int max_tiles = (R / BM + E + 7) / 8 * 8;  // upper bound of the tile count, whole eighths for the per-XCD list
    // One token's worth of routed rows (batch-1 decode): stage each tile's activation rows whole and run the
    // barrier-free weight stream.  From two tokens on the chunked kernel below is faster (measured, us per layer,
    // whole-row kernel / chunked: T = 1 31.6 / 39.5, T = 2 45.9 / 42.8, T = 8 80 / 64, T = 32 126 / 92).
    const bool decode_sized = R <= 4;

    auto *gu = static_cast<const uint8_t *>(w_gate_up_planar);
    auto *dn = static_cast<const uint8_t *>(w_down_planar);
    if (decode_sized && R <= kDirectRows && moe_small_lds_bytes(Hp) <= 150 * 1024 && Ip <= 4096) {
        // Direct form: two launches.  The gate/up GEMM takes routed entry t as its row tile t and quantises the
        // token's row of x itself; the down GEMM sums over the token's experts as it finishes.
        MoeGemmArgs a1{};
        a1.a_div = topk_i;
        a1.w_nib = gu; a1.w_sc = gu + mx_scale_offset(e * 2 * i, h);
        a1.rows_per_expert = 2 * I; a1.K = H; a1.Kp = Hp; a1.N = I;
        a1.out = w.act;
        a1.q_hi = w.a_hi; a1.q_lo = w.a_lo; a1.q_sc = w.a_sc; a1.q_kp = Ip;
        a1.sel = sel_dev; a1.x = static_cast<const __bf16 *>(x_dev); a1.slot_of = w.plan.slot_of;
        a1.n_experts = E; a1.direct_rows = R;
        {
            const size_t lds_bytes = moe_small_lds_bytes(Hp);
            auto kern = mx_moe_gemm_small_kernel<2, true, true>;
            static LdsOptIn opt;
            if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(kern), lds_bytes)) return st;
            hipLaunchKernelGGL(kern, dim3(static_cast<unsigned>((I + 63) / 64), static_cast<unsigned>(R)), dim3(256), lds_bytes, s, a1);
            LHIP_CHECK_LAUNCH();
        }
        MoeDownDirectArgs a2{};
        a2.a_hi = w.a_hi; a2.a_lo = w.a_lo; a2.a_sc = w.a_sc;
        a2.w_nib = dn; a2.w_sc = dn + mx_scale_offset(e * h, i);
        a2.rows_per_expert = H; a2.Kp = Ip; a2.N = H;
        a2.sel = sel_dev; a2.wts = wts_dev; a2.R = R; a2.topk = topk_i; a2.n_experts = E;
        a2.out = w.out; a2.y = static_cast<__bf16 *>(y_dev);
        {
            const size_t lds_bytes = moe_small_lds_bytes(Ip);
            static LdsOptIn opt;
            if (lhip_status st = lds_opt_in(opt, reinterpret_cast<const void *>(mx_moe_down_direct_kernel), lds_bytes)) return st;
            hipLaunchKernelGGL(mx_moe_down_direct_kernel, dim3(static_cast<unsigned>(H / 16)), dim3(256), lds_bytes, s, a2);
            LHIP_CHECK_LAUNCH();
        }
        return LHIP_OK;
    }

    // The decode-sized kernels walk the plain tile list; the chunked kernels take the one laid out per XCD.
    w.plan.max_tiles = max_tiles;
    w.plan.tiles_per_xcd = decode_sized ? 0 : max_tiles / 8;
    {
        const size_t items = static_cast<size_t>(T) * (Hp / 8);
        hipLaunchKernelGGL(moe_prepare_kernel, dim3(static_cast<unsigned>(1 + (items + 1023) / 1024)), dim3(1024), 0, s,
                           sel_dev, R, E, BM, w.plan, static_cast<const __bf16 *>(x_dev), w.x_hi, w.x_lo, w.x_sc, T, H, Hp);
        LHIP_CHECK_LAUNCH();
    }
    MoeGemmArgs a1{};
    a1.a_hi = w.x_hi; a1.a_lo = w.x_lo; a1.a_sc = w.x_sc;
    a1.a_index = w.plan.slot_src; a1.a_div = topk_i;
    a1.w_nib = gu; a1.w_sc = gu + mx_scale_offset(e * 2 * i, h);
    a1.rows_per_expert = 2 * I; a1.K = H; a1.Kp = Hp; a1.N = I;
    a1.tile_expert = w.plan.tile_expert; a1.tile_row0 = w.plan.tile_row0; a1.tile_rows = w.plan.tile_rows;
    a1.tile_run0 = w.plan.tile_run0; a1.tile_runlen = w.plan.tile_runlen;
    a1.n_tiles = w.plan.n_tiles; a1.tiles_per_xcd = w.plan.tiles_per_xcd; a1.out = w.act;
    const bool whole_rows = mt == 1 && decode_sized && moe_small_lds_bytes(Hp) <= 150 * 1024;
    // Every gated kernel launched below quantises its result for the down GEMM in its epilogue.
    a1.q_hi = w.a_hi; a1.q_lo = w.a_lo; a1.q_sc = w.a_sc; a1.q_kp = Ip;
    // Column blocks: 4 waves x (NT/2) gate/up pairs of 16.  Tall row tiles take 4 weight
    // fragments per wave, so each activation fragment read from LDS feeds twice the MFMAs.
    const int cb1 = (I + 63) / 64, cb1w = (I + 127) / 128;
    lhip_status st;
    switch (mt) {
        case 1:
            st = whole_rows ? launch_moe_gemm_small<2, true>(a1, cb1, max_tiles, s)
                                                       : launch_moe_gemm<1, 4, true>(a1, cb1w, max_tiles, s);
            break;
        case 2: st = launch_moe_gemm<2, 4, true>(a1, cb1w, max_tiles, s); break;
        case 4: st = launch_moe_gemm<4, 4, true, 1, 2>(a1, cb1w, max_tiles, s); break;
        case 5: st = launch_moe_gemm<5, 4, true, 1, 2>(a1, cb1w, max_tiles, s); break;
        default: st = launch_moe_gemm<8, 4, true, 2, 2>(a1, cb1w, max_tiles, s); break;
    }
    if (st) return st;
    MoeGemmArgs a2{};
    a2.a_hi = w.a_hi; a2.a_lo = w.a_lo; a2.a_sc = w.a_sc;
    a2.a_index = nullptr; a2.a_div = 1;
    a2.w_nib = dn; a2.w_sc = dn + mx_scale_offset(e * h, i);
    a2.rows_per_expert = H; a2.K = I; a2.Kp = Ip; a2.N = H;
    a2.tile_expert = w.plan.tile_expert; a2.tile_row0 = w.plan.tile_row0; a2.tile_rows = w.plan.tile_rows;
    a2.tile_run0 = w.plan.tile_run0; a2.tile_runlen = w.plan.tile_runlen;
    a2.n_tiles = w.plan.n_tiles; a2.tiles_per_xcd = w.plan.tiles_per_xcd; a2.out = w.out;
    if (mt == 1) {
        st = decode_sized && moe_small_lds_bytes(Ip) <= 150 * 1024
                 ? launch_moe_gemm_small<1, false>(a2, (H + 63) / 64, max_tiles, s)
                                                   : launch_moe_gemm<1, 2, false>(a2, (H + 127) / 128, max_tiles, s);
    } else {
        const int cb2 = (H + 127) / 128, cb2w = (H + 255) / 256;  // 4 waves x NT fragments of 16
        switch (mt) {
            case 2: st = launch_moe_gemm<2, 2, false>(a2, cb2, max_tiles, s); break;
            case 4: st = launch_moe_gemm<4, 4, false, 1, 2>(a2, cb2w, max_tiles, s); break;
            case 5: st = launch_moe_gemm<5, 3, false, 1, 2>(a2, (H + 191) / 192, max_tiles, s); break;
            default: st = launch_moe_gemm<8, 4, false, 2, 2>(a2, cb2w, max_tiles, s); break;
        }
    }
    if (st) return st;
    return moe_launch_combine(w.out, w.plan.slot_of, wts_dev, static_cast<__bf16 *>(y_dev), T, H, topk_i, s);
}

lhip_status lhip_mxfp4_moe_bf16_static(const void *w_gate_up_planar, const void *w_down_planar, const void *x_dev,
                                       const int32_t *sel_dev, const float *wts_dev, void *y_dev, int64_t t, int64_t h,
                                       int64_t i, int64_t e, int64_t topk, void *stream) {
    if (lhip_status s = check_moe_shape(t, h, i, e, topk)) return s;
    if (carve(nullptr, t, h, i, e, topk).total > kMoeStaticBytes) return LHIP_ERR_UNSUPPORTED;  // beyond the scratch array
    unsigned char *ws = nullptr;
    if (lhip_status s = moe_scratch_address(&ws)) return s;
    // Nothing in the workspace has to start at zero: every piece a pass reads is written earlier in the same pass.
    return lhip_mxfp4_moe_bf16(w_gate_up_planar, w_down_planar, x_dev, sel_dev, wts_dev, y_dev, t, h, i, e, topk, ws, stream);
}

lhip_status lhip_mxfp4_moe_read_intermediates(const void *workspace_dev, float *act_dev, float *down_dev, int64_t t,
                                              int64_t h, int64_t i, int64_t e, int64_t topk, void *stream) {
    return lhip_mxfp4_moe_read_intermediates_mode(workspace_dev, act_dev, down_dev, t, h, i, e, topk, LHIP_MOE_EXACT, stream);
}

lhip_status lhip_mxfp4_moe_read_intermediates_mode(const void *workspace_dev, float *act_dev, float *down_dev, int64_t t,
                                                   int64_t h, int64_t i, int64_t e, int64_t topk, int32_t mode,
                                                   void *stream) {
    if (!workspace_dev) return LHIP_ERR_NULL_PTR;
    if (lhip_status s = check_moe_shape(t, h, i, e, topk)) return s;
    if (mode != LHIP_MOE_EXACT && mode != LHIP_MOE_FAST) return LHIP_ERR_UNSUPPORTED;
    if (!aligned(workspace_dev, 256) || !aligned(act_dev, 4) || !aligned(down_dev, 4)) return LHIP_ERR_MISALIGNED;
    if (!act_dev && !down_dev) return LHIP_OK;
    MoeWorkspace w = carve(const_cast<void *>(workspace_dev), t, h, i, e, topk);
    const int R = static_cast<int>(t * topk);
    if (mode == LHIP_MOE_EXACT)
        return moe_exact_read_intermediates(w, act_dev, down_dev, R, static_cast<int>(i), static_cast<int>(h), as_stream(stream));
    hipLaunchKernelGGL(moe_read_intermediates_kernel, dim3(static_cast<unsigned>(R)), dim3(256), 0, as_stream(stream),
                       w.plan.slot_of, w.a_hi, w.a_lo, w.a_sc, w.out, act_dev, down_dev, R, static_cast<int>(i),
                       static_cast<int>(pad128(i)), static_cast<int>(h));
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

}  // extern "C"
