// Decode-step glue of a Qwen3-shaped layer between the fused QKV projection and the cache: per-head
// RMSNorm of queries and keys followed by the rotary embedding, one launch.
//
// Reference: model_hub/qwen.py:327-340 (wqkv: split + head_rmsnorm of q and k), :410-431 (head_rmsnorm,
// flashinfer.rmsnorm on [tokens*heads, head_dim]) and :434-498 (rotary embedding, rotate-half form) -
// two norm launches and about sixteen element-wise torch launches per layer and token there.
#include "pkv_common.h"
#include "pkv_lut.h"

namespace {

// RMSNorm + rotary embedding of one head held by one wave: lane l holds dims l and l + 64 (the rotate-half pair) in
// x1 / x2 and gets the same dims of the result.  fp32 arithmetic; the caller rounds to bf16.
__device__ __forceinline__ void qk_norm_rope_head(float x1, float x2, const uint16_t *__restrict__ w, float eps, float c,
                                                  float s, float &y1, float &y2) {
  const int lane = pkv_lane();
  float ss = x1 * x1 + x2 * x2;
#pragma unroll
  for (int m = 1; m < PKV_WAVE; m <<= 1) ss += __shfl_xor(ss, m, PKV_WAVE);
  const float inv = 1.0f / sqrtf(ss * (1.0f / 128.0f) + eps);
  if (w) {
    x1 = x1 * inv * pkv_bf16_bits_to_f32(w[lane]);
    x2 = x2 * inv * pkv_bf16_bits_to_f32(w[lane + 64]);
  }
  y1 = x1 * c - x2 * s, y2 = x2 * c + x1 * s;
}

// One wave per head.  head index in [0, Hq + Hkv): query heads first.
__device__ __forceinline__ void qk_norm_rope_task(int task, const uint16_t *__restrict__ qkv, int64_t stride_b, int n_q_heads,
                                                  int n_kv_heads, const uint16_t *__restrict__ q_weight,
                                                  const uint16_t *__restrict__ k_weight, float eps,
                                                  const uint16_t *__restrict__ cos_row, const uint16_t *__restrict__ sin_row,
                                                  uint16_t *__restrict__ q_out, uint16_t *__restrict__ k_out,
                                                  uint16_t *__restrict__ cache_k = nullptr,
                                                  uint16_t *__restrict__ cache_v = nullptr, int64_t cache_stride_b = 0,
                                                  int64_t cache_stride_h = 0, int64_t cache_slot = 0) {
  const int lane = pkv_lane();
  const int heads = n_q_heads + n_kv_heads;
  const int b = task / heads, head = task % heads;
  const bool is_q = head < n_q_heads;
  const uint16_t *src = qkv + (int64_t)b * stride_b + (int64_t)head * 128;  // q heads, then k heads, contiguous in qkv
  float y1, y2;
  qk_norm_rope_head(pkv_bf16_bits_to_f32(src[lane]), pkv_bf16_bits_to_f32(src[lane + 64]), is_q ? q_weight : k_weight, eps,
                    pkv_bf16_bits_to_f32(cos_row[lane]), pkv_bf16_bits_to_f32(sin_row[lane]), y1, y2);
  uint16_t *dst = is_q ? q_out + ((int64_t)b * n_q_heads + head) * 128
                       : k_out + ((int64_t)b * n_kv_heads + (head - n_q_heads)) * 128;
  dst[lane] = pkv_f32_to_bf16_bits(y1);
  dst[lane + 64] = pkv_f32_to_bf16_bits(y2);
  if (!is_q && cache_k) {  // the token's rows of the cache as well: the finished key, and the value head as it stands in qkv
    const int kvh = head - n_q_heads;
    const int64_t row = (int64_t)b * cache_stride_b + (int64_t)kvh * cache_stride_h + cache_slot * 128;
    cache_k[row + lane] = pkv_f32_to_bf16_bits(y1);
    cache_k[row + lane + 64] = pkv_f32_to_bf16_bits(y2);
    const uint16_t *vsrc = qkv + (int64_t)b * stride_b + (int64_t)(heads + kvh) * 128;
    cache_v[row + lane] = vsrc[lane];
    cache_v[row + lane + 64] = vsrc[lane + 64];
  }
}

__global__ __launch_bounds__(256) void pkv_qk_norm_rope_kernel(const uint16_t *__restrict__ qkv, int64_t stride_b, int n_q_heads,
                                                               int n_kv_heads, const uint16_t *__restrict__ q_weight,
                                                               const uint16_t *__restrict__ k_weight, float eps,
                                                               const uint16_t *__restrict__ cos_row,
                                                               const uint16_t *__restrict__ sin_row,
                                                               uint16_t *__restrict__ q_out, uint16_t *__restrict__ k_out,
                                                               int n_tasks) {
  const int task = blockIdx.x * 4 + threadIdx.x / PKV_WAVE;
  if (task >= n_tasks) return;
  qk_norm_rope_task(task, qkv, stride_b, n_q_heads, n_kv_heads, q_weight, k_weight, eps, cos_row, sin_row, q_out, k_out);
}

// The same launch with the retrieval's query side riding along: workgroups [0, n_rope_blocks) are the norm + rotary
// embedding above; the 16 * rows workgroups after them build one subspace's slice of a (batch, kv-head) row's vote
// table each, from the same raw qkv: the wave that rotates the row's query normalises and rotates the group's query
// heads itself (the arithmetic of qk_norm_rope_head, rounded to bf16 as q_out is), so nothing waits for q_out.
// What pkv_query_prep_lut_kernel would write for those queries lands in the same workspace segments, and the words
// that launch clears for the later stages are cleared here.
__global__ __launch_bounds__(256) void pkv_qk_norm_rope_table_kernel(
    const uint16_t *__restrict__ qkv, int64_t stride_b, int n_q_heads, int n_kv_heads, const uint16_t *__restrict__ q_weight,
    const uint16_t *__restrict__ k_weight, float eps, const uint16_t *__restrict__ cos_row, const uint16_t *__restrict__ sin_row,
    uint16_t *__restrict__ q_out, uint16_t *__restrict__ k_out, int n_tasks, int n_rope_blocks, int bs,
    const float *__restrict__ signs, const int32_t *__restrict__ cc, PkvTiers tiers, float *__restrict__ qhat,
    float *__restrict__ qnorm, uint8_t *__restrict__ lut, uint32_t *__restrict__ row_suf, uint32_t *__restrict__ zero_ptr,
    int64_t zero_words, uint16_t *__restrict__ cache_k, uint16_t *__restrict__ cache_v, int64_t cache_stride_b,
    int64_t cache_stride_h, int64_t cache_slot) {
  const int tid = threadIdx.x;
  if ((int)blockIdx.x < n_rope_blocks) {
    const int task = blockIdx.x * 4 + tid / PKV_WAVE;
    if (task < n_tasks)
      qk_norm_rope_task(task, qkv, stride_b, n_q_heads, n_kv_heads, q_weight, k_weight, eps, cos_row, sin_row, q_out, k_out,
                        cache_k, cache_v, cache_stride_b, cache_stride_h, cache_slot);
    return;
  }
  const int t = blockIdx.x - n_rope_blocks, n_table = 16 * bs * n_kv_heads;
  const int sub = t % 16, row = t / 16;
  const int b = row / n_kv_heads, h = row % n_kv_heads, group = n_q_heads / n_kv_heads;
  for (int64_t i = (int64_t)t * 256 + tid; i < zero_words; i += (int64_t)n_table * 256) zero_ptr[i] = 0u;
  if (sub == 1 && tid < 128) row_suf[(int64_t)row * 128 + tid] = 0u;

  __shared__ PkvLutSmem sm;
  __shared__ float s_head[4][128];  // the group's heads after norm + rotary embedding (bf16 values), four at a time
  const int my_cc = cc[((int64_t)row * 16 + sub) * 256 + tid];
  const int lane = pkv_lane(), wave = tid / PKV_WAVE;
  const float c = pkv_bf16_bits_to_f32(cos_row[lane]), s = pkv_bf16_bits_to_f32(sin_row[lane]);
  // the group mean of pkv_query_group_mean_wave_t over heads that are normalised and rotated on the way: the four
  // waves take a head each, the first wave adds them up in head order
  float a_lo = 0.f, a_hi = 0.f;
  for (int g0 = 0; g0 < group; g0 += 4) {
    if (g0 + wave < group) {
      const uint16_t *src = qkv + (int64_t)b * stride_b + (int64_t)(h * group + g0 + wave) * 128;
      float y1, y2;
      qk_norm_rope_head(pkv_bf16_bits_to_f32(src[lane]), pkv_bf16_bits_to_f32(src[lane + 64]), q_weight, eps, c, s, y1, y2);
      s_head[wave][lane] = pkv_bf16_round(y1), s_head[wave][lane + 64] = pkv_bf16_round(y2);
    }
    __syncthreads();
    if (tid < PKV_WAVE) {
      for (int u = 0; u < 4 && g0 + u < group; ++u) {
        a_lo = g0 + u == 0 ? s_head[u][lane] : a_lo + s_head[u][lane];
        a_hi = g0 + u == 0 ? s_head[u][lane + 64] : a_hi + s_head[u][lane + 64];
      }
    }
    if (g0 + 4 < group) __syncthreads();
  }
  if (tid < PKV_WAVE) {
    float x_lo, x_hi;
    if ((group & (group - 1)) == 0) {
      const float inv = 1.0f / (float)group;
      x_lo = pkv_bf16_round(a_lo * inv), x_hi = pkv_bf16_round(a_hi * inv);
    } else {
      x_lo = pkv_bf16_round(a_lo / (float)group), x_hi = pkv_bf16_round(a_hi / (float)group);
    }
    float y_lo, y_hi;
    const float n = pkv_normalize_rotate_64(x_lo, x_hi, signs[lane], signs[lane + 64], PKV_DTYPE_BF16, y_lo, y_hi);
    sm.y[tid] = y_lo, sm.y[tid + 64] = y_hi;
    if (sub == 0) {
      qhat[(int64_t)row * 128 + tid] = y_lo, qhat[(int64_t)row * 128 + tid + 64] = y_hi;
      if (tid == 0) qnorm[row] = n;
    }
  }
  sm.cc[tid] = my_cc;
  __syncthreads();
  pkv_lut_rank_subspace(PKV_DTYPE_BF16, nullptr, tiers, sub, sm, lut + ((int64_t)row * 16 + sub) * 256, nullptr);
}

// out_sum = x + residual (residual may be NULL), out_norm = RMSNorm(out_sum) * weight.  One workgroup of 256
// threads per token row; width a multiple of 8 up to 16384 (8 bf16 per 128-bit access, at most 8 accesses
// per thread).  fp32 arithmetic; out_sum is rounded to bf16 first and the norm is taken of the rounded sum,
// as a separate add followed by a norm would.
__global__ __launch_bounds__(256) void pkv_add_rmsnorm_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ residual,
                                                              const uint16_t *__restrict__ weight, float eps, int width,
                                                              uint16_t *__restrict__ out_sum, uint16_t *__restrict__ out_norm) {
  __shared__ float s_part[4];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int n_vec = width / 8;
  float v[8][8];
  pkv_u32x4 wts[8];  // the weights do not depend on the sum: requested with the inputs, not after the reduction
  float ss = 0.f;
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int vec = tid + r * 256;
    if (vec < n_vec) {
      const pkv_u32x4 a = *(const pkv_u32x4 *)(x + (int64_t)row * width + vec * 8);
      wts[r] = *(const pkv_u32x4 *)(weight + vec * 8);
      pkv_u32x4 b = {0u, 0u, 0u, 0u};
      if (residual) b = *(const pkv_u32x4 *)(residual + (int64_t)row * width + vec * 8);
      const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
      uint32_t ow[4];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const float lo = pkv_bf16_round(__uint_as_float(aw[p] << 16) + __uint_as_float(bw[p] << 16));
        const float hi = pkv_bf16_round(__uint_as_float(aw[p] & 0xffff0000u) + __uint_as_float(bw[p] & 0xffff0000u));
        v[r][2 * p] = lo, v[r][2 * p + 1] = hi;
        ss += lo * lo + hi * hi;
        ow[p] = (__float_as_uint(lo) >> 16) | (__float_as_uint(hi) & 0xffff0000u);
      }
      if (out_sum) *(pkv_u32x4 *)(out_sum + (int64_t)row * width + vec * 8) = pkv_u32x4{ow[0], ow[1], ow[2], ow[3]};
    }
  }
#pragma unroll
  for (int m = 1; m < PKV_WAVE; m <<= 1) ss += __shfl_xor(ss, m, PKV_WAVE);
  if (pkv_lane() == 0) s_part[tid / PKV_WAVE] = ss;
  __syncthreads();
  const float inv = 1.0f / sqrtf((s_part[0] + s_part[1] + s_part[2] + s_part[3]) / (float)width + eps);
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int vec = tid + r * 256;
    if (vec < n_vec) {
      const uint32_t ww[4] = {wts[r].x, wts[r].y, wts[r].z, wts[r].w};
      uint32_t ow[4];
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const float lo = v[r][2 * p] * inv * __uint_as_float(ww[p] << 16);
        const float hi = v[r][2 * p + 1] * inv * __uint_as_float(ww[p] & 0xffff0000u);
        ow[p] = (uint32_t)pkv_f32_to_bf16_bits(lo) | ((uint32_t)pkv_f32_to_bf16_bits(hi) << 16);
      }
      *(pkv_u32x4 *)(out_norm + (int64_t)row * width + vec * 8) = pkv_u32x4{ow[0], ow[1], ow[2], ow[3]};
    }
  }
}

// out[row][j] = silu(gate_up[row][j]) * gate_up[row][inter + j], bf16, 8 elements per thread.
__global__ __launch_bounds__(256) void pkv_silu_mul_kernel(const uint16_t *__restrict__ gate_up, int64_t row_stride, int inter,
                                                           uint16_t *__restrict__ out, int64_t n_vec_total) {
  const int64_t g = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (g >= n_vec_total) return;
  const int per_row = inter / 8;
  const int64_t row = g / per_row;
  const int vec = (int)(g % per_row);
  const pkv_u32x4 a = *(const pkv_u32x4 *)(gate_up + row * row_stride + vec * 8);
  const pkv_u32x4 b = *(const pkv_u32x4 *)(gate_up + row * row_stride + inter + vec * 8);
  const uint32_t aw[4] = {a.x, a.y, a.z, a.w}, bw[4] = {b.x, b.y, b.z, b.w};
  uint32_t ow[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const float g0 = __uint_as_float(aw[p] << 16), g1 = __uint_as_float(aw[p] & 0xffff0000u);
    const float u0 = __uint_as_float(bw[p] << 16), u1 = __uint_as_float(bw[p] & 0xffff0000u);
    const float s0 = pkv_bf16_round(g0 / (1.0f + __expf(-g0))), s1 = pkv_bf16_round(g1 / (1.0f + __expf(-g1)));
    ow[p] = (uint32_t)pkv_f32_to_bf16_bits(s0 * u0) | ((uint32_t)pkv_f32_to_bf16_bits(s1 * u1) << 16);
  }
  *(pkv_u32x4 *)(out + row * inter + vec * 8) = pkv_u32x4{ow[0], ow[1], ow[2], ow[3]};
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

// Launcher of the norm + rotary embedding with the retrieval's query side in the same launch (pkv_retrieve.hip lays the
// workspace out and checks the retrieval's arguments).
int pkv_launch_qk_norm_rope_table(const void *qkv, int64_t stride_b, int bs, int n_q_heads, int n_kv_heads,
                                  const void *q_weight, const void *k_weight, float eps, const void *cos_row,
                                  const void *sin_row, void *q_out, void *k_out, const float *signs, const int32_t *cc,
                                  const PkvTiers &tiers, float *qhat, float *qnorm, uint8_t *lut, uint32_t *row_suf,
                                  uint32_t *zero_ptr, int64_t zero_words, const pkv_kv_append *append, hipStream_t s) {
  PKV_REQUIRE(qkv && cos_row && sin_row && q_out && k_out, "pkv_qk_norm_rope_table: null pointer");
  if (append) {
    PKV_REQUIRE(append->dst_k && append->dst_v && append->rows > 0 && append->slot >= 0 && append->slot < append->rows &&
                    append->stride_h >= append->rows * 128 && (bs == 1 || append->stride_b >= n_kv_heads * append->stride_h),
                "pkv_qk_norm_rope_table: append needs dst_k / dst_v [bs][kv_heads][rows][128] and 0 <= slot < rows");
    PKV_REQUIRE(stride_b >= (int64_t)(n_q_heads + 2 * n_kv_heads) * 128,
                "pkv_qk_norm_rope_table: append reads the value heads behind the key heads of qkv");
  }
  PKV_REQUIRE(bs > 0 && n_q_heads > 0 && n_kv_heads > 0 && n_q_heads % n_kv_heads == 0 &&
                  (int64_t)bs * (n_q_heads + n_kv_heads) < (1 << 24) && stride_b >= (int64_t)(n_q_heads + n_kv_heads) * 128,
              "pkv_qk_norm_rope_table: bad shape bs=%d heads=%d+%d stride=%lld", bs, n_q_heads, n_kv_heads, (long long)stride_b);
  PKV_REQUIRE((q_weight == nullptr) == (k_weight == nullptr), "q and k norm weights go together");
  const int n_tasks = bs * (n_q_heads + n_kv_heads);
  const int n_rope_blocks = (n_tasks + 3) / 4;
  hipLaunchKernelGGL(pkv_qk_norm_rope_table_kernel, dim3((unsigned)(n_rope_blocks + 16 * bs * n_kv_heads)), dim3(256), 0, s,
                     (const uint16_t *)qkv, stride_b, n_q_heads, n_kv_heads, (const uint16_t *)q_weight,
                     (const uint16_t *)k_weight, eps, (const uint16_t *)cos_row, (const uint16_t *)sin_row, (uint16_t *)q_out,
                     (uint16_t *)k_out, n_tasks, n_rope_blocks, bs, signs, cc, tiers, qhat, qnorm, lut, row_suf, zero_ptr,
                     zero_ptr ? zero_words : 0, append ? (uint16_t *)append->dst_k : nullptr,
                     append ? (uint16_t *)append->dst_v : nullptr, append ? append->stride_b : 0,
                     append ? append->stride_h : 0, append ? append->slot : 0);
  PKV_LAUNCH_CHECK("pkv_qk_norm_rope_table_kernel");
  return PKV_OK;
}

extern "C" int pkv_add_rmsnorm(const void *x, const void *residual, const void *weight, float eps, int rows, int width,
                               void *out_sum, void *out_norm, void *stream) {
  PKV_REQUIRE(x && weight && out_norm, "pkv_add_rmsnorm: null pointer");
  PKV_REQUIRE(rows > 0 && width > 0 && width % 8 == 0 && width <= 16384, "pkv_add_rmsnorm: width must be a multiple of 8 up to 16384 (got %d)", width);
  PKV_REQUIRE(pkv_aligned(x, 16) && pkv_aligned(weight, 16) && pkv_aligned(out_norm, 16) &&
                  (!residual || pkv_aligned(residual, 16)) && (!out_sum || pkv_aligned(out_sum, 16)),
              "pkv_add_rmsnorm: 16-byte aligned buffers required");
  hipLaunchKernelGGL(pkv_add_rmsnorm_kernel, dim3((unsigned)rows), dim3(256), 0, (hipStream_t)stream, (const uint16_t *)x,
                     (const uint16_t *)residual, (const uint16_t *)weight, eps, width, (uint16_t *)out_sum,
                     (uint16_t *)out_norm);
  PKV_LAUNCH_CHECK("pkv_add_rmsnorm_kernel");
  return PKV_OK;
}

extern "C" int pkv_silu_mul(const void *gate_up, int64_t row_stride, int rows, int inter, void *out, void *stream) {
  PKV_REQUIRE(gate_up && out && rows > 0 && inter > 0 && inter % 8 == 0 && row_stride >= 2 * (int64_t)inter && row_stride % 8 == 0,
              "pkv_silu_mul: bad shape rows=%d inter=%d stride=%lld", rows, inter, (long long)row_stride);
  PKV_REQUIRE(pkv_aligned(gate_up, 16) && pkv_aligned(out, 16), "pkv_silu_mul: 16-byte aligned buffers required");
  const int64_t n_vec = (int64_t)rows * (inter / 8);
  hipLaunchKernelGGL(pkv_silu_mul_kernel, dim3((unsigned)((n_vec + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const uint16_t *)gate_up, row_stride, inter, (uint16_t *)out, n_vec);
  PKV_LAUNCH_CHECK("pkv_silu_mul_kernel");
  return PKV_OK;
}
