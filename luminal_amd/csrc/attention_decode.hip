// Batch-1 decode attention with rotary embedding and KV append folded in.
//
// What the reference's graph does for one new token (examples/llama/src/model.rs:52-72
// rotary, :108-110 cache concat, :112-139 grouped-query attention) as ONE launch:
//   q, k of the new token are rotated; k and v are appended to the caches at *pos;
//   out[h] = softmax(q_h . K / sqrt(hd)) V over positions 0..*pos.
//
// Shape of the launch.  At batch 1 the work is a read of the two caches, which one
// workgroup per head cannot pull fast enough (it exposes several dependent memory round
// trips on a handful of CUs).  So the keys of each KV head are cut into `splits` ranges,
// one workgroup each (grid = kv_heads x splits, about one workgroup per CU), and the G
// query heads that share a KV head are served by the same workgroup, which therefore
// reads every cache row once.  Each workgroup writes its partial softmax state (max, sum,
// weighted V) to a workspace and a second, small kernel (one workgroup per query head) merges
// the partials into the output rows.  The bodies of both kernels live in
// attention_decode_device.h, which describes the work inside a workgroup.
#include "attention_decode_device.h"
#include "common.h"

namespace lhip {

template <int G, int HD>
__global__ __launch_bounds__(kDecThreads) void attention_decode_kernel(
    const float *__restrict__ qkv, float *__restrict__ k_cache, float *__restrict__ v_cache,
    const int *__restrict__ pos_dev, int hkv, int max_seq, float theta, int n_splits,
    float *__restrict__ ws_ml, float4 *__restrict__ ws_acc, bool few_ranges) {
    __shared__ AttnShared<G, HD> sh;
    attention_decode_body<G, HD, kDecThreads>(PlainIO{}, sh, blockIdx.x, blockIdx.y, qkv, k_cache, v_cache, *pos_dev, hkv,
                                                     max_seq, theta, n_splits, ws_ml, ws_acc, few_ranges);
}

// One workgroup per query head.
template <int G, int HD>
__global__ __launch_bounds__(kDecThreads) void attention_merge_kernel(float *__restrict__ out,
                                                                      const int *__restrict__ pos_dev, int max_seq,
                                                                      int n_splits, const float *__restrict__ ws_ml,
                                                                      const float4 *__restrict__ ws_acc, bool few_ranges) {
    __shared__ MergeShared sh;
    attention_merge_body<G, HD, kDecThreads>(PlainIO{}, sh, blockIdx.x, out, *pos_dev, max_seq, n_splits, ws_ml, ws_acc,
                                             nullptr, few_ranges);
}

// out == nullptr: the partial states stay in the workspace for a consumer that merges them itself
// (lhip_q8_0_matvec_attn_merge_f32).
template <int G, int HD>
static lhip_status launch_decode(const float *qkv, float *kc, float *vc, float *out, const int *pos, int hkv, int max_seq,
                                 float theta, void *workspace, bool few, hipStream_t s) {
    const int splits = dec_splits(hkv);
    auto *base = static_cast<uint8_t *>(workspace);
    float *ml = reinterpret_cast<float *>(base);
    float4 *acc = reinterpret_cast<float4 *>(base + dec_ml_bytes(hkv, splits, G));
    hipLaunchKernelGGL((attention_decode_kernel<G, HD>), dim3(static_cast<unsigned>(hkv), static_cast<unsigned>(splits)),
                       dim3(kDecThreads), 0, s, qkv, kc, vc, pos, hkv, max_seq, theta, splits, ml, acc, few);
    LHIP_CHECK_LAUNCH();
    if (!out) return LHIP_OK;
    hipLaunchKernelGGL((attention_merge_kernel<G, HD>), dim3(static_cast<unsigned>(hkv * G)), dim3(kDecThreads), 0, s, out,
                       pos, max_seq, splits, ml, acc, few);
    LHIP_CHECK_LAUNCH();
    return LHIP_OK;
}

lhip_status attention_decode_impl(const float *qkv_dev, float *k_cache_dev, float *v_cache_dev, float *out_dev,
                                  bool with_merge, bool few, const int32_t *pos_dev, int64_t q_heads, int64_t kv_heads,
                                  int64_t head_dim, int64_t max_seq, float theta, void *workspace_dev, void *stream);

static bool dec_supported(int64_t q_heads, int64_t kv_heads, int64_t head_dim) {
    if (kv_heads <= 0 || q_heads <= 0 || q_heads % kv_heads != 0) return false;
    const int64_t g = q_heads / kv_heads;
    return (g == 1 || g == 2 || g == 4 || g == 8) && (head_dim == 64 || head_dim == 128);
}

}  // namespace lhip

using namespace lhip;

extern "C" {

size_t lhip_attention_decode_workspace_nbytes(int64_t q_heads, int64_t kv_heads, int64_t head_dim) {
    if (!dec_supported(q_heads, kv_heads, head_dim) || kv_heads > 65535) return 0;
    const size_t g = static_cast<size_t>(q_heads / kv_heads);
    const int splits = dec_splits(kv_heads);
    const size_t slots = static_cast<size_t>(kv_heads) * splits * g;
    return dec_ml_bytes(kv_heads, splits, static_cast<int64_t>(g)) +
           slots * static_cast<size_t>(head_dim) * sizeof(float);
}

lhip_status lhip_attention_decode_partial_f32(const float *qkv_dev, float *k_cache_dev, float *v_cache_dev,
                                              const int32_t *pos_dev, int64_t q_heads, int64_t kv_heads, int64_t head_dim,
                                              int64_t max_seq, float theta, void *workspace_dev, void *stream) {
    return attention_decode_impl(qkv_dev, k_cache_dev, v_cache_dev, nullptr, false, true, pos_dev, q_heads, kv_heads,
                                 head_dim, max_seq, theta, workspace_dev, stream);
}

lhip_status lhip_attention_decode_few_ranges_f32(const float *qkv_dev, float *k_cache_dev, float *v_cache_dev,
                                                 float *out_dev, const int32_t *pos_dev, int64_t q_heads, int64_t kv_heads,
                                                 int64_t head_dim, int64_t max_seq, float theta, void *workspace_dev,
                                                 void *stream) {
    return attention_decode_impl(qkv_dev, k_cache_dev, v_cache_dev, out_dev, true, true, pos_dev, q_heads, kv_heads,
                                 head_dim, max_seq, theta, workspace_dev, stream);
}

lhip_status lhip_attention_decode_f32(const float *qkv_dev, float *k_cache_dev, float *v_cache_dev, float *out_dev,
                                      const int32_t *pos_dev, int64_t q_heads, int64_t kv_heads, int64_t head_dim,
                                      int64_t max_seq, float theta, void *workspace_dev, void *stream) {
    return attention_decode_impl(qkv_dev, k_cache_dev, v_cache_dev, out_dev, true, false, pos_dev, q_heads, kv_heads,
                                 head_dim, max_seq, theta, workspace_dev, stream);
}

}  // extern "C"

namespace lhip {

lhip_status attention_decode_impl(const float *qkv_dev, float *k_cache_dev, float *v_cache_dev, float *out_dev,
                                  bool with_merge, bool few, const int32_t *pos_dev, int64_t q_heads, int64_t kv_heads,
                                  int64_t head_dim, int64_t max_seq, float theta, void *workspace_dev, void *stream) {
    if (!qkv_dev || !k_cache_dev || !v_cache_dev || (with_merge && !out_dev) || !pos_dev || !workspace_dev)
        return LHIP_ERR_NULL_PTR;
    if (q_heads <= 0 || kv_heads <= 0 || head_dim <= 0 || max_seq <= 0 || q_heads % kv_heads != 0 ||
        max_seq > kMaxDim || kv_heads > 65535)
        return LHIP_ERR_INVALID_SHAPE;
    if (!dec_supported(q_heads, kv_heads, head_dim)) return LHIP_ERR_UNSUPPORTED;
    if (!aligned(qkv_dev, 16) || !aligned(k_cache_dev, 16) || !aligned(v_cache_dev, 16) ||
        (with_merge && !aligned(out_dev, 16)) || !aligned(workspace_dev, 256))
        return LHIP_ERR_MISALIGNED;
    const int g = static_cast<int>(q_heads / kv_heads);
    const int hkv = static_cast<int>(kv_heads), ms = static_cast<int>(max_seq);
    hipStream_t s = as_stream(stream);
#define LHIP_CASE(G, HD) \
    if (g == G && head_dim == HD) \
        return launch_decode<G, HD>(qkv_dev, k_cache_dev, v_cache_dev, out_dev, pos_dev, hkv, ms, theta, workspace_dev, few, s);
    LHIP_CASE(1, 64) LHIP_CASE(2, 64) LHIP_CASE(4, 64) LHIP_CASE(8, 64)
    LHIP_CASE(1, 128) LHIP_CASE(2, 128) LHIP_CASE(4, 128) LHIP_CASE(8, 128)
#undef LHIP_CASE
    return LHIP_ERR_UNSUPPORTED;
}

}  // namespace lhip
