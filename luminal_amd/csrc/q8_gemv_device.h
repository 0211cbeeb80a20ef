// Device code of the Q8_0 matrix-vector kernels: shared by the library's launchers (q8_gemv.hip) and by the
// code-object build that exports the same kernels under C names (module/q8_gemv_module.hip).  One definition of
// the arithmetic, so both routes give the same bits.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lhip {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Sum over the 64 lanes of a wavefront; every lane returns the total.
__device__ __forceinline__ float wave_sum(float v) {
    // xor 1, xor 2 inside quads, then mirror inside 8 and inside 16 lanes.
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x4E, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x141, 0xF, 0xF, true));
    v += __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x140, 0xF, 0xF, true));
    // Each row of 16 lanes now holds its row sum in every lane.
    const int b = __builtin_bit_cast(int, v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)) +
           __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48));
}

__device__ __forceinline__ float sb(uint32_t w, int i) {
    return static_cast<float>(static_cast<int8_t>((w >> (8 * i)) & 0xff));
}

// Dot product of 16 int8 quants with 16 f32 activations.
__device__ __forceinline__ float dot16(const u32x4 &q, const float4 (&x)[4]) {
    float s = sb(q.x, 0) * x[0].x;
    s = fmaf(sb(q.x, 1), x[0].y, s);
    s = fmaf(sb(q.x, 2), x[0].z, s);
    s = fmaf(sb(q.x, 3), x[0].w, s);
    s = fmaf(sb(q.y, 0), x[1].x, s);
    s = fmaf(sb(q.y, 1), x[1].y, s);
    s = fmaf(sb(q.y, 2), x[1].z, s);
    s = fmaf(sb(q.y, 3), x[1].w, s);
    s = fmaf(sb(q.z, 0), x[2].x, s);
    s = fmaf(sb(q.z, 1), x[2].y, s);
    s = fmaf(sb(q.z, 2), x[2].z, s);
    s = fmaf(sb(q.z, 3), x[2].w, s);
    s = fmaf(sb(q.w, 0), x[3].x, s);
    s = fmaf(sb(q.w, 1), x[3].y, s);
    s = fmaf(sb(q.w, 2), x[3].z, s);
    s = fmaf(sb(q.w, 3), x[3].w, s);
    return s;
}

// Activation / output element type T (the reference's QuantizedMatmul<T>): float, or __half with every product and
// sum still in f32 (crates/luminal_cuda/src/quantized.rs:72,94-96 accumulate in float and store (T)sum, :106).
// Four consecutive activations as f32.
__device__ __forceinline__ float4 load_x4(const float *x, int i4) { return reinterpret_cast<const float4 *>(x)[i4]; }
__device__ __forceinline__ float4 load_x4(const __half *x, int i4) {
    const uint2 raw = reinterpret_cast<const uint2 *>(x)[i4];
    const __half2 lo = *reinterpret_cast<const __half2 *>(&raw.x), hi = *reinterpret_cast<const __half2 *>(&raw.y);
    return make_float4(__low2float(lo), __high2float(lo), __low2float(hi), __high2float(hi));
}
__device__ __forceinline__ void store_y(float *y, int i, float v) { y[i] = v; }
__device__ __forceinline__ void store_y(__half *y, int i, float v) { y[i] = __float2half(v); }  // round to nearest even

// R rows per wave, W waves per workgroup, U slices of 1024 quants per step.
// grid.x covers ceil(n / (R*W)) row tiles, grid.y the rows of x (m).
template <int R, int W, int U, typename T>
__device__ __forceinline__ void q8_gemv_oneshot_body(const int8_t *__restrict__ qs, const __half *__restrict__ ds,
                                                     const T *__restrict__ x, T *__restrict__ y, int n, int k) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int row0 = (blockIdx.x * W + wave) * R;
    if (row0 >= n) return;  // wave-uniform

    x += static_cast<size_t>(blockIdx.y) * k;
    y += static_cast<size_t>(blockIdx.y) * n;

    const int nblk = k >> 5;
    const int8_t *qrow[R];
    const __half *drow[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        // Rows past the end re-read the last row; their sums are not stored.
        const int row = min(row0 + r, n - 1);
        qrow[r] = qs + static_cast<size_t>(row) * k;
        drow[r] = ds + static_cast<size_t>(row) * nblk;
    }

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;

    int kofs = lane * 16;
    // Full steps: U slices, no bounds checks.
    for (; kofs + (U - 1) * 1024 < k; kofs += U * 1024) {
        u32x4 q[U][R];
        __half d[U][R];
        float4 xv[U][4];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int ko = kofs + u * 1024;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                q[u][r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(qrow[r] + ko));
                d[u][r] = drow[r][ko >> 5];
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) xv[u][j] = load_x4(x, (ko >> 2) + j);
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int r = 0; r < R; ++r) acc[r] = fmaf(dot16(q[u][r], xv[u]), __half2float(d[u][r]), acc[r]);
    }
    // Tail: remaining slices one at a time (lanes past K idle).
    for (; kofs < k; kofs += 1024) {
        float4 xv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) xv[j] = load_x4(x, (kofs >> 2) + j);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const u32x4 q = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(qrow[r] + kofs));
            acc[r] = fmaf(dot16(q, xv), __half2float(drow[r][kofs >> 5]), acc[r]);
        }
    }

    float out = 0.f;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float s = wave_sum(acc[r]);
        if (lane == r) out = s;
    }
    if (lane < R && row0 + lane < n) store_y(y, row0 + lane, out);
}

template <int R, int W, int U, typename T = float>
__global__ __launch_bounds__(W * 64) void q8_gemv_f32_kernel(const int8_t *__restrict__ qs,
                                                              const __half *__restrict__ ds,
                                                              const T *__restrict__ x, T *__restrict__ y,
                                                              int n, int k) {
    q8_gemv_oneshot_body<R, W, U, T>(qs, ds, x, y, n, k);
}

// ---------------------------------------------------------------------------
// Persistent, software-pipelined variant (the one the library normally runs).
// Requires K to be a multiple of S*1024 and at most 16384.
//
// A grid of G workgroups of W wavefronts stays resident; wave w walks the row
// groups w, w + W*G, ...  The activation vector is staged once per workgroup
// into LDS, so the only HBM traffic in the loop is the weight stream.  Work is
// cut into steps of R rows x S slices of 1024 quants; the loads of step t+1
// are issued before the arithmetic of step t starts (two register buffers,
// scheduling fenced), so each wave always has R*S 16-byte loads per lane in
// flight.
//
// LDS layout of the activations: float4 index  slice*256 + j*64 + lane  holds
// x[slice*1024 + lane*16 + j*4 .. +3], so the four 16-byte reads a lane makes
// per slice are contiguous across lanes (no bank conflicts).
// ---------------------------------------------------------------------------

template <int R, int S>
struct StepBuf {
    u32x4 q[S][R];
    unsigned d[S][R];  // f16 scale code, zero-extended
};

// Row bases are wave-uniform (scalar registers); the per-lane part of every
// address is one 32-bit byte offset plus a compile-time slice offset.
template <int R, int S>
__device__ __forceinline__ void load_step(StepBuf<R, S> &b, const int8_t *__restrict__ qs,
                                          const unsigned short *__restrict__ ds, int row0, int n, int k, int slice0,
                                          unsigned lane, bool live) {
    // `live` is wave-uniform.  A dead step (one past the wave's last) still
    // issues its loads, so the count of outstanding loads is the same on every
    // trip through the pipeline, but aims them all at the first bytes of the
    // planes: one cached line instead of a stream from HBM.
    const int nblk = k >> 5;
    const unsigned kbase = live ? static_cast<unsigned>(slice0) * 1024u : 0u;
    const unsigned qoff = live ? lane * 16u : 0u;
    const unsigned doff = live ? (lane >> 1) * 2u : 0u;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int row = live ? min(row0 + r, n - 1) : 0;  // rows past the end re-read the last row
        const char *qrow = reinterpret_cast<const char *>(qs) + static_cast<size_t>(row) * k + kbase;
        const char *drow = reinterpret_cast<const char *>(ds) + (static_cast<size_t>(row) * nblk + (kbase >> 5)) * 2;
#pragma unroll
        for (int s = 0; s < S; ++s) {
            b.q[s][r] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(qrow + (s * 1024u + qoff)));
            b.d[s][r] = __builtin_nontemporal_load(reinterpret_cast<const unsigned short *>(drow + (s * 64u + doff)));
        }
    }
    // The offsets stay live past the last request: otherwise their registers may become the destination of that
    // request, and the next step, which writes the offsets again, first has to wait for it.
    asm volatile("" ::"v"(qoff), "v"(doff));
}

template <int R, int S>
__device__ __forceinline__ void compute_step(StepBuf<R, S> &b, const float4 *xs4, int slice0, unsigned lane,
                                             float (&acc)[R]) {
#pragma unroll
    for (int s = 0; s < S; ++s) {
        const float4 *xp = xs4 + (slice0 + s) * 256 + lane;
        float4 xv[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) xv[j] = xp[j * 64];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            // Opaque to the optimiser: keeps the int8->f32 conversions of this
            // buffer here instead of next to its loads, where they would stall
            // the wave on data it has only just requested.
            asm volatile("" : "+v"(b.q[s][r]), "+v"(b.d[s][r]));
            acc[r] = fmaf(dot16(b.q[s][r], xv),
                          __half2float(__ushort_as_half(static_cast<unsigned short>(b.d[s][r]))), acc[r]);
        }
    }
}

template <int R, int S, int W, typename XT>
__device__ __forceinline__ void q8_gemv_pipe_body(const int8_t *__restrict__ qs, const unsigned short *__restrict__ ds,
                                                  const XT *__restrict__ x, XT *__restrict__ y, int n, int k) {
    extern __shared__ float4 xs4[];
    const unsigned lane = threadIdx.x & 63u;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: stays in a scalar register
    const int wave_global = blockIdx.x * W + wave;
    const int total_waves = gridDim.x * W;
    x += static_cast<size_t>(blockIdx.y) * k;
    y += static_cast<size_t>(blockIdx.y) * n;

    const int n_groups = (n + R - 1) / R;
    const int chunks = k / (S * 1024);  // steps per row group
    const int my_groups = wave_global < n_groups ? (n_groups - wave_global + total_waves - 1) / total_waves : 0;
    const int T = my_groups * chunks;

    StepBuf<R, S> a, b;
    // First weight loads go out before the activations are staged, so the
    // HBM round trip overlaps the staging.
    load_step(a, qs, ds, wave_global * R, n, k, 0, lane, T > 0);

    {
        const int k4 = k >> 2;
#pragma unroll 4
        for (int i = threadIdx.x; i < k4; i += W * 64) {
            // destination index i = slice*256 + j*64 + l  <-  source slice*256 + l*4 + j
            const int src = (i & ~255) | ((i & 63) << 2) | ((i >> 6) & 3);
            xs4[i] = load_x4(x, src);
        }
    }
    __syncthreads();
    if (T == 0) return;

    float acc[R];
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] = 0.f;

    int t = 0;            // step being computed
    int g = wave_global;  // its row group
    int c = 0;            // its chunk within the row group

    auto next = [&](int &gg, int &cc) {
        if (++cc == chunks) {
            cc = 0;
            gg += total_waves;
        }
    };
    auto finish_group = [&](int gg) {
        float out = 0.f;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float s = wave_sum(acc[r]);
            if (lane == static_cast<unsigned>(r)) out = s;
            acc[r] = 0.f;
        }
        const int row0 = gg * R;
        if (lane < static_cast<unsigned>(R) && row0 + static_cast<int>(lane) < n) store_y(y, row0 + lane, out);
    };

    while (true) {
        int g1 = g, c1 = c;
        next(g1, c1);
        load_step(b, qs, ds, g1 * R, n, k, c1 * S, lane, t + 1 < T);
        __builtin_amdgcn_sched_barrier(0);
        compute_step(a, xs4, c * S, lane, acc);
        if (c == chunks - 1) finish_group(g);
        if (++t >= T) break;
        g = g1;
        c = c1;
        next(g1, c1);
        load_step(a, qs, ds, g1 * R, n, k, c1 * S, lane, t + 1 < T);
        __builtin_amdgcn_sched_barrier(0);
        compute_step(b, xs4, c * S, lane, acc);
        if (c == chunks - 1) finish_group(g);
        if (++t >= T) break;
        g = g1;
        c = c1;
    }
}

template <int R, int S, int W, typename XT = float>
__global__ __launch_bounds__(W * 64) void q8_gemv_f32_pipe_kernel(const int8_t *__restrict__ qs,
                                                                const unsigned short *__restrict__ ds,
                                                                const XT *__restrict__ x, XT *__restrict__ y,
                                                                int n, int k) {
    q8_gemv_pipe_body<R, S, W, XT>(qs, ds, x, y, n, k);
}

}  // namespace lhip
