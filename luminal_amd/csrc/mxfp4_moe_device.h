// Shared pieces of the MXFP4 mixture-of-experts kernels (mxfp4_moe.hip: the block-scaled fast form;
// mxfp4_moe_exact.hip: the bf16 form): tile plan, workspace layout, small device helpers.
#pragma once

#include "common.h"

#include <type_traits>
#include <utility>

namespace lhip {


typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef uint32_t mu32x4 __attribute__((ext_vector_type(4)));

constexpr int kChunk = 128;      // K elements per MFMA
constexpr int kLoShift = 5;      // the lo plane of an activation is held times 2^5 and multiplied with block scale - 5
constexpr float kLoGain = 32.f;
constexpr int kARow = 160;       // LDS bytes per activation row of a chunk: 128 fp8 + 32 padding (with 16 the fragment reads,
                                 // lane (r, g) at r * pitch + 16 g, take twice as long: measured 8.0 against 4.3 cycles per read)

static inline int64_t pad128(int64_t k) { return (k + 127) / 128 * 128; }
// Row pitch of a whole quantised activation row in LDS (Kp a multiple of 128): the row plus padding that makes the
// pitch 160 mod 256, the residue measured free of bank conflicts for the fragment reads.
__host__ __device__ static inline int moe_small_pitch(int Kp) { return Kp + ((Kp & 255) ? 32 : 160); }

// ---------------------------------------------------------------------------
// Plan: group the R = T*topk routed entries by expert and cut each expert's rows
// into tiles of BM.  One workgroup; E <= 1024.
// ---------------------------------------------------------------------------
struct MoePlan {
    int *offsets;      // [E+1] first slot of each expert
    int *slot_src;     // [R]   slot -> routed entry r = t*topk + s
    int *slot_of;      // [R]   routed entry -> slot (-1 if its expert id is invalid)
    int *tile_expert;  // [max_tiles]
    int *tile_row0;    // [max_tiles] first slot of the tile
    int *tile_rows;    // [max_tiles] valid rows in the tile (0 = unused entry)
    // [max_tiles] the run of a tile: the consecutive list entries that hold tiles of the same expert (on the same XCD,
    // when the list is cut per XCD) start at entry tile_run0 and number tile_runlen (0 = unused entry).  The exact
    // GEMMs walk a run column block by column block, so that the workgroups that read the same weights run together.
    int *tile_run0, *tile_runlen;
    int *n_tiles;      // [1]
    int max_tiles;     // entries of the three tile arrays
    // 0: tiles are listed in expert order from entry 0.  Otherwise the list is cut into eight ranges of this many
    // entries, one per XCD (range x is read by the workgroups whose dispatch number is x modulo 8), and the
    // tiles, still in expert order, are dealt to the ranges in eight contiguous, equal shares: the tiles of an
    // expert, and all column blocks of a tile, then run on one XCD and find each other's weights and
    // activation rows in its L2.
    int tiles_per_xcd;
};

__device__ __forceinline__ void moe_plan_block(const int *__restrict__ sel, int R, int E, int BM, const MoePlan &p) {
    __shared__ int cnt[1024], off[1025], cur[1024];
    for (int e = threadIdx.x; e < E; e += 1024) {
        cnt[e] = 0;
        cur[e] = 0;
    }
    for (int t = threadIdx.x; t < p.max_tiles; t += 1024) {  // entries no tile is written to stay marked unused
        p.tile_expert[t] = 0;
        p.tile_row0[t] = 0;
        p.tile_rows[t] = 0;
        p.tile_run0[t] = t;
        p.tile_runlen[t] = 0;
    }
    __syncthreads();
    for (int r = threadIdx.x; r < R; r += 1024) {
        const int e = sel[r];
        if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    // Thread e lays out expert e: its first slot and first tile are prefix sums over the experts before it
    // (E <= 1024 broadcast reads from LDS), then it writes its own tiles.
    // ceil(cnt / BM) tiles of equal height (a multiple of 16 rows): 140 rows with BM = 128 become 80 + 60 rather
    // than 128 + 12, and the GEMM skips the row fragments a tile does not have.
    for (int e = threadIdx.x; e < E; e += 1024) {
        int o = 0, nt = 0, total = 0;
        for (int q = 0; q < E; ++q) {
            const int tq = (cnt[q] + BM - 1) / BM;  // equals the number of tiles written for q below
            if (q < e) {
                o += cnt[q];
                nt += tq;
            }
            total += tq;
        }
        off[e] = o;
        p.offsets[e] = o;
        const int tiles_e = (cnt[e] + BM - 1) / BM;
        const int per = tiles_e ? ((cnt[e] + tiles_e - 1) / tiles_e + 15) / 16 * 16 : 0;
        const int nt_first = nt, nt_end = nt + tiles_e;
        for (int m0 = 0; m0 < cnt[e]; m0 += per) {
            int at = nt, run_first = nt_first, run_end = nt_end;
            if (p.tiles_per_xcd) {  // tile nt of `total` goes to range x = floor(8 nt / total), behind that range's earlier tiles
                const int x = nt * 8 / total;
                const int x_first = (x * total + 7) / 8, x_end = ((x + 1) * total + 7) / 8;  // the tiles of range x
                at = x * p.tiles_per_xcd + nt - x_first;
                run_first = max(nt_first, x_first);
                run_end = min(nt_end, x_end);
            }
            p.tile_expert[at] = e;
            p.tile_row0[at] = o + m0;
            p.tile_rows[at] = min(per, cnt[e] - m0);
            p.tile_run0[at] = at - (nt - run_first);
            p.tile_runlen[at] = run_end - run_first;
            ++nt;
        }
        if (e == E - 1) {
            off[E] = o + cnt[e];
            p.offsets[E] = o + cnt[e];
            *p.n_tiles = nt;
        }
    }
    __syncthreads();
    // Order inside an expert's range is arbitrary (atomic): every row is computed
    // independently, and slot_of lets the combine step find it again.
    for (int r = threadIdx.x; r < R; r += 1024) {
        const int e = sel[r];
        if (e >= 0 && e < E) {
            const int pos = off[e] + atomicAdd(&cur[e], 1);
            p.slot_src[pos] = r;
            p.slot_of[r] = pos;
        } else {
            p.slot_of[r] = -1;
        }
    }
}


// Maximum over the 16 lanes of a DPP row, in every lane of the row (quad swaps, then the two mirrors): register
// moves only, where a shuffle would go through the LDS pipeline.
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true)));
    v = fmaxf(v, __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true)));
    return v;
}

// f(integral_constant<int, 1>) ... f(integral_constant<int, N-1>), expanded at compile time.
template <class F, int... Is>
__device__ __forceinline__ void static_for_from1_impl(F &&f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is + 1>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for_from1(F &&f) {
    static_for_from1_impl(static_cast<F &&>(f), std::make_integer_sequence<int, (N > 1 ? N - 1 : 0)>{});
}
// f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>), expanded at compile time.
template <class F, int... Is>
__device__ __forceinline__ void static_for_n_impl(F &&f, std::integer_sequence<int, Is...>) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for_n(F &&f) {
    static_for_n_impl(static_cast<F &&>(f), std::make_integer_sequence<int, N>{});
}

template <int MT, int NT>
struct BSet {
    mu32x4 q[NT];
    uint32_t s[NT];
    bool valid;  // wave-uniform: false for a dead chunk past the padded K
};

// ---------------------------------------------------------------------------
// Workspace carving (256-byte aligned pieces, in this order).
// ---------------------------------------------------------------------------
struct MoeWorkspace {
    MoePlan plan;
    uint8_t *x_hi, *x_lo, *x_sc;  // quantised x, T rows of Kp(H)
    __bf16 *act;                  // [R][I]
    uint8_t *a_hi, *a_lo, *a_sc;  // quantised act, R rows of Kp(I)
    float *out;                   // [R][H]
    size_t total;
};

static inline MoeWorkspace carve(void *base, int64_t T, int64_t H, int64_t I, int64_t E, int64_t topk) {
    MoeWorkspace w{};
    const int64_t R = T * topk;
    const int64_t max_tiles = R / 16 + E + 8;  // tiles of at least 16 rows, one partial tile per expert, rounded up to eight
    size_t off = 0;
    auto take = [&](size_t bytes) {
        uint8_t *p = base ? static_cast<uint8_t *>(base) + off : nullptr;
        off += (bytes + 255) & ~size_t{255};
        return p;
    };
    w.plan.offsets = reinterpret_cast<int *>(take((E + 1) * 4));
    w.plan.slot_src = reinterpret_cast<int *>(take(R * 4));
    w.plan.slot_of = reinterpret_cast<int *>(take(R * 4));
    w.plan.tile_expert = reinterpret_cast<int *>(take(max_tiles * 4));
    w.plan.tile_row0 = reinterpret_cast<int *>(take(max_tiles * 4));
    w.plan.tile_rows = reinterpret_cast<int *>(take(max_tiles * 4));
    w.plan.tile_run0 = reinterpret_cast<int *>(take(max_tiles * 4));
    w.plan.tile_runlen = reinterpret_cast<int *>(take(max_tiles * 4));
    w.plan.n_tiles = reinterpret_cast<int *>(take(4));
    const int64_t Hp = pad128(H), Ip = pad128(I);
    w.x_hi = take(T * Hp);
    w.x_lo = take(T * Hp);
    w.x_sc = take(T * (Hp / 32));
    w.act = reinterpret_cast<__bf16 *>(take(R * I * 2));
    w.a_hi = take(R * Ip);
    w.a_lo = take(R * Ip);
    w.a_sc = take(R * (Ip / 32));
    w.out = reinterpret_cast<float *>(take(R * H * 4));
    w.total = off;
    return w;
}

static inline size_t moe_small_lds_bytes(int Kp) { return 2 * 16 * static_cast<size_t>(moe_small_pitch(Kp)) + 16 * (Kp / 32); }

// Routed rows the direct (two-launch) forms take: one token's top-4.
constexpr int kDirectRows = 4;

// mxfp4_moe.hip: y[t][h] = bf16( sum_s wts[t][s] * out[slot_of[t*topk+s]][h] )
lhip_status moe_launch_combine(const float *out, const int *slot_of, const float *wts, __bf16 *y, int T, int H, int topk,
                               hipStream_t s);
// mxfp4_moe_exact.hip: the layer on the bf16 matrix instruction (weights expanded exactly), and its intermediates.
lhip_status moe_exact_forward(const uint8_t *gu, const uint8_t *dn, const __bf16 *x, const int32_t *sel_dev,
                              const float *wts_dev, __bf16 *y, int T, int H, int I, int E, int topk, MoeWorkspace &w,
                              hipStream_t s);
lhip_status moe_exact_read_intermediates(const MoeWorkspace &w, float *act_dev, float *down_dev, int R, int I, int H,
                                         hipStream_t s);

}  // namespace lhip
