// Decode-step glue of a Qwen3-shaped layer between the fused QKV projection and the cache: per-head
// RMSNorm of queries and keys followed by the rotary embedding, one launch.
//
// Reference: model_hub/qwen.py:327-340 (wqkv: split + head_rmsnorm of q and k), :410-431 (head_rmsnorm,
// flashinfer.rmsnorm on [tokens*heads, head_dim]) and :434-498 (rotary embedding, rotate-half form) -
// two norm launches and about sixteen element-wise torch launches per layer and token there.
#include "pkv_common.h"

namespace {

// One wave per head; lane l holds dims l and l + 64 (the rotate-half pair).  head index in [0, Hq + Hkv):
// query heads first.  fp32 arithmetic, one rounding to bf16 at the end.
__global__ __launch_bounds__(256) void pkv_qk_norm_rope_kernel(const uint16_t *__restrict__ qkv, int64_t stride_b, int n_q_heads,
                                                               int n_kv_heads, const uint16_t *__restrict__ q_weight,
                                                               const uint16_t *__restrict__ k_weight, float eps,
                                                               const uint16_t *__restrict__ cos_row,
                                                               const uint16_t *__restrict__ sin_row,
                                                               uint16_t *__restrict__ q_out, uint16_t *__restrict__ k_out,
                                                               int n_tasks) {
  const int task = blockIdx.x * 4 + threadIdx.x / PKV_WAVE;
  if (task >= n_tasks) return;
  const int lane = pkv_lane();
  const int heads = n_q_heads + n_kv_heads;
  const int b = task / heads, head = task % heads;
  const bool is_q = head < n_q_heads;
  const uint16_t *src = qkv + (int64_t)b * stride_b + (int64_t)head * 128;  // q heads, then k heads, contiguous in qkv
  const uint16_t *w = is_q ? q_weight : k_weight;
  float x1 = pkv_bf16_bits_to_f32(src[lane]), x2 = pkv_bf16_bits_to_f32(src[lane + 64]);
  float ss = x1 * x1 + x2 * x2;
#pragma unroll
  for (int m = 1; m < PKV_WAVE; m <<= 1) ss += __shfl_xor(ss, m, PKV_WAVE);
  const float inv = 1.0f / sqrtf(ss * (1.0f / 128.0f) + eps);
  if (w) {
    x1 = x1 * inv * pkv_bf16_bits_to_f32(w[lane]);
    x2 = x2 * inv * pkv_bf16_bits_to_f32(w[lane + 64]);
  }
  const float c = pkv_bf16_bits_to_f32(cos_row[lane]), s = pkv_bf16_bits_to_f32(sin_row[lane]);
  const float y1 = x1 * c - x2 * s, y2 = x2 * c + x1 * s;
  uint16_t *dst = is_q ? q_out + ((int64_t)b * n_q_heads + head) * 128
                       : k_out + ((int64_t)b * n_kv_heads + (head - n_q_heads)) * 128;
  dst[lane] = pkv_f32_to_bf16_bits(y1);
  dst[lane + 64] = pkv_f32_to_bf16_bits(y2);
}

}  // namespace

extern "C" int pkv_qk_norm_rope(const void *qkv, int64_t stride_b, int bs, int n_q_heads, int n_kv_heads,
                                const void *q_weight, const void *k_weight, float eps, const void *cos_row,
                                const void *sin_row, void *q_out, void *k_out, void *stream) {
  PKV_REQUIRE(qkv && cos_row && sin_row && q_out && k_out, "pkv_qk_norm_rope: null pointer");
  PKV_REQUIRE(bs > 0 && n_q_heads > 0 && n_kv_heads > 0 && (int64_t)bs * (n_q_heads + n_kv_heads) < (1 << 24) &&
                  stride_b >= (int64_t)(n_q_heads + n_kv_heads) * 128,
              "pkv_qk_norm_rope: bad shape bs=%d heads=%d+%d stride=%lld", bs, n_q_heads, n_kv_heads, (long long)stride_b);
  PKV_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "q and k norm weights go together");
  const int n_tasks = bs * (n_q_heads + n_kv_heads);
  hipLaunchKernelGGL(pkv_qk_norm_rope_kernel, dim3((unsigned)((n_tasks + 3) / 4)), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t *)qkv, stride_b, n_q_heads, n_kv_heads, (const uint16_t *)q_weight,
                     (const uint16_t *)k_weight, eps, (const uint16_t *)cos_row, (const uint16_t *)sin_row,
                     (uint16_t *)q_out, (uint16_t *)k_out, n_tasks);
  PKV_LAUNCH_CHECK("pkv_qk_norm_rope_kernel");
  return PKV_OK;
}
