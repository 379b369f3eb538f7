// Selections: (1) candidate select = top-k of small integer vote counts with a
// fixed tie rule, spread over many workgroups per row; (2) exact top-k of fp32
// scores in descending order.
//
// Reference: cache_hub/topk/radix_topk.cu:39-120 (bucket_topk_kernel) and
// :161-239 (radix_topk_kernel), which use one workgroup per row, three passes
// over the row and atomics for the output slots (so output order and the choice
// among ties vary from run to run); cache_hub/polar_cache.py:1300-1302
// (torch.topk + gather) for the final select.
//
// Here the per-chunk histograms written by the collision scan give every
// workgroup the global threshold and its own output offsets, so the candidate
// list is produced in one pass, in a fixed order: indices above the threshold
// ascending, then indices at the threshold ascending.
#include "pkv_common.h"

namespace {

constexpr int kSelThreads = 256;
constexpr int kSelKeysPerThread = 8;
constexpr int kSelKeysPerIter = kSelThreads * kSelKeysPerThread;  // 2048

// grid (n_chunks, rows).  cnt rows are padded to a multiple of 16 bytes and
// 16-byte aligned, so every thread's 8 counts are one aligned 64-bit load.
__global__ __launch_bounds__(kSelThreads) void pkv_select_kernel(const uint8_t *__restrict__ cnt,
                                                                 int64_t cnt_stride,
                                                                 const uint16_t *__restrict__ chunk_hist,
                                                                 int chunk_keys, int64_t n_keys, int64_t k,
                                                                 int64_t *__restrict__ out) {
  const int row = blockIdx.y;
  const int chunk = blockIdx.x;
  const int n_chunks = gridDim.x;
  const int tid = threadIdx.x;

  __shared__ uint32_t s_tot[129], s_bef[129], s_stot[129], s_sbef[129];
  __shared__ int s_theta;
  __shared__ uint32_t s_ngt, s_gtb, s_eqb;
  __shared__ int s_scan[2][kSelThreads / PKV_WAVE];

  if (tid < 128) {
    const uint16_t *hp = chunk_hist + (int64_t)row * n_chunks * 128 + tid;
    uint32_t tot = 0, bef = 0;
    for (int c = 0; c < n_chunks; ++c) {
      const uint32_t v = hp[(int64_t)c * 128];
      tot += v;
      if (c < chunk) bef += v;
    }
    s_tot[tid] = tot;
    s_bef[tid] = bef;
  } else if (tid == 128) {
    s_tot[128] = 0;
    s_bef[128] = 0;
    s_stot[128] = 0;
    s_sbef[128] = 0;
    s_theta = 0;
    s_ngt = 0;
    s_gtb = 0;
    s_eqb = 0;
  }
  __syncthreads();
  if (tid < 128) {  // suffix sums over bins >= tid
    uint32_t st = 0, sb = 0;
    for (int t = tid; t < 128; ++t) {
      st += s_tot[t];
      sb += s_bef[t];
    }
    s_stot[tid] = st;
    s_sbef[tid] = sb;
  }
  __syncthreads();
  if (tid < 128 && (int64_t)s_stot[tid] >= k && (int64_t)s_stot[tid + 1] < k) {
    s_theta = tid;             // k-th largest count
    s_ngt = s_stot[tid + 1];   // keys strictly above it, whole row
    s_gtb = s_sbef[tid + 1];   // ... of those, in earlier chunks
    s_eqb = s_bef[tid];        // keys equal to it in earlier chunks
  }
  __syncthreads();
  const uint32_t theta = (uint32_t)s_theta;
  int64_t base_gt = s_gtb;
  int64_t base_eq = (int64_t)s_ngt + s_eqb;
  int64_t *orow = out + (int64_t)row * k;
  const uint8_t *crow = cnt + (int64_t)row * cnt_stride;

  const int64_t chunk_begin = (int64_t)chunk * chunk_keys;
  const int64_t chunk_end = (chunk_begin + chunk_keys < n_keys) ? chunk_begin + chunk_keys : n_keys;
  int it = 0;
  for (int64_t blk0 = chunk_begin; blk0 < chunk_end; blk0 += kSelKeysPerIter, ++it) {
    const int64_t i0 = blk0 + (int64_t)tid * kSelKeysPerThread;
    uint32_t gt_mask = 0, eq_mask = 0;
    if (i0 < chunk_end) {
      const pkv_u32x2 w = *(const pkv_u32x2 *)(crow + i0);  // padded rows: always in bounds
      const uint32_t ww[2] = {w.x, w.y};
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const uint32_t v = (ww[j >> 2] >> (8 * (j & 3))) & 0xffu;
        const bool valid = i0 + j < chunk_end;
        gt_mask |= (valid && v > theta) ? (1u << j) : 0u;
        eq_mask |= (valid && v == theta) ? (1u << j) : 0u;
      }
    }
    const int packed = __popc(gt_mask) | (__popc(eq_mask) << 16);
    int total;
    const int excl = pkv_block_excl_scan<kSelThreads>(packed, s_scan[it & 1], total);
    int64_t pg = base_gt + (excl & 0xffff);
    int64_t pe = base_eq + (excl >> 16);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (gt_mask & (1u << j)) {
        if (pg < k) orow[pg] = i0 + j;
        ++pg;
      } else if (eq_mask & (1u << j)) {
        if (pe < k) orow[pe] = i0 + j;
        ++pe;
      }
    }
    base_gt += total & 0xffff;
    base_eq += total >> 16;
  }
}

// out[row][i] = i (i < len) else 0: the reference's `length <= k` branch
// (radix_topk.cu:154-159).
__global__ void pkv_identity_fill_kernel(int64_t *__restrict__ out, int64_t len, int64_t k, int rows) {
  const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= (int64_t)rows * k) return;
  const int64_t i = g % k;
  out[g] = i < len ? i : 0;
}

// int32 counts -> clamped u8 counts (padded rows) + per-chunk histograms.
__global__ __launch_bounds__(256) void pkv_counts_to_u8_kernel(const int32_t *__restrict__ x, int64_t x_stride,
                                                               int64_t len, uint8_t *__restrict__ cnt,
                                                               int64_t cnt_stride, uint16_t *__restrict__ chunk_hist,
                                                               int chunk_keys) {
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
  __shared__ uint32_t s_hist[128];
  if (tid < 128) s_hist[tid] = 0;
  __syncthreads();
  const int64_t k0 = (int64_t)chunk * chunk_keys;
  const int64_t k1 = (k0 + chunk_keys < len) ? k0 + chunk_keys : len;
  for (int64_t i = k0 + tid; i < k1; i += 256) {
    int v = x[(int64_t)row * x_stride + i];
    v = v < 0 ? 0 : (v > 127 ? 127 : v);
    cnt[(int64_t)row * cnt_stride + i] = (uint8_t)v;
    atomicAdd(&s_hist[v], 1u);
  }
  __syncthreads();
  if (tid < 128) chunk_hist[((int64_t)row * gridDim.x + chunk) * 128 + tid] = (uint16_t)s_hist[tid];
}

// ------------------------------------------------------------ exact fp32 top-k

constexpr int kTopkThreads = 1024;
constexpr int kTopkMaxSort = 8192;  // 64 KB of 64-bit keys in LDS

__device__ __forceinline__ uint64_t make_key(const float *__restrict__ x, const int64_t *__restrict__ ids,
                                             int64_t i) {
  const uint32_t id = ids ? (uint32_t)ids[i] : (uint32_t)i;
  return ((uint64_t)pkv_ordered_u32(x[i]) << 32) | (uint64_t)(~id);
}

// Descending bitonic sort of P (power of two) 64-bit keys in LDS.
__device__ __forceinline__ void bitonic_sort_desc(uint64_t *s, int P) {
  for (int size = 2; size <= P; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int t = threadIdx.x; t < P / 2; t += kTopkThreads) {
        const int lo = ((t & ~(stride - 1)) << 1) | (t & (stride - 1));
        const int hi = lo + stride;
        const bool desc = (lo & size) == 0;
        const uint64_t a = s[lo], b = s[hi];
        if (desc ? (a < b) : (a > b)) {
          s[lo] = b;
          s[hi] = a;
        }
      }
      __syncthreads();
    }
  }
}

__device__ __forceinline__ void emit_topk(const uint64_t *s, int64_t k, int64_t *__restrict__ out_ids,
                                          float *__restrict__ out_vals) {
  for (int64_t i = threadIdx.x; i < k; i += kTopkThreads) {
    const uint64_t key = s[i];
    out_ids[i] = (int64_t)(uint32_t)(~(uint32_t)key);
    if (out_vals) out_vals[i] = pkv_from_ordered_u32((uint32_t)(key >> 32));
  }
}

// len <= 8192: sort everything.  One workgroup per row, dynamic LDS P*8 bytes.
__global__ __launch_bounds__(kTopkThreads) void pkv_topk_sort_kernel(const float *__restrict__ x, int64_t x_stride,
                                                                     const int64_t *__restrict__ ids,
                                                                     int64_t ids_stride, int len, int P, int64_t k,
                                                                     int64_t *__restrict__ out_ids,
                                                                     float *__restrict__ out_vals) {
  extern __shared__ uint64_t s_keys[];
  const int row = blockIdx.x;
  const float *xr = x + (int64_t)row * x_stride;
  const int64_t *ir = ids ? ids + (int64_t)row * ids_stride : nullptr;
  for (int i = threadIdx.x; i < P; i += kTopkThreads) s_keys[i] = i < len ? make_key(xr, ir, i) : 0ull;
  __syncthreads();
  bitonic_sort_desc(s_keys, P);
  emit_topk(s_keys, k, out_ids + (int64_t)row * k, out_vals ? out_vals + (int64_t)row * k : nullptr);
}

// len > 8192, k <= 8192: eight 8-bit MSB-first radix passes find the k-th
// largest 64-bit key exactly, the k winners are collected into LDS and sorted.
__global__ __launch_bounds__(kTopkThreads) void pkv_topk_radix_kernel(const float *__restrict__ x, int64_t x_stride,
                                                                      const int64_t *__restrict__ ids,
                                                                      int64_t ids_stride, int64_t len, int P,
                                                                      int64_t k, int64_t *__restrict__ out_ids,
                                                                      float *__restrict__ out_vals) {
  extern __shared__ uint64_t s_keys[];
  __shared__ uint32_t s_hist[257];
  __shared__ uint32_t s_digit, s_need, s_counter;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float *xr = x + (int64_t)row * x_stride;
  const int64_t *ir = ids ? ids + (int64_t)row * ids_stride : nullptr;

  uint64_t prefix = 0;
  uint32_t need = (uint32_t)k;
  for (int pass = 0; pass < 8; ++pass) {
    const int shift = 56 - 8 * pass;
    if (tid < 257) s_hist[tid] = 0;
    __syncthreads();
    for (int64_t i = tid; i < len; i += kTopkThreads) {
      const uint64_t key = make_key(xr, ir, i);
      if (pass == 0 || (key >> (shift + 8)) == (prefix >> (shift + 8)))
        atomicAdd(&s_hist[(uint32_t)(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    uint32_t suf = 0, suf_next = 0;
    if (tid < 256) {
      for (int d = tid + 1; d < 256; ++d) suf_next += s_hist[d];
      suf = suf_next + s_hist[tid];
    }
    __syncthreads();
    if (tid < 256 && suf >= need && suf_next < need) {
      s_digit = (uint32_t)tid;
      s_need = need - suf_next;
    }
    __syncthreads();
    prefix |= (uint64_t)s_digit << shift;
    need = s_need;
  }
  // prefix is now the k-th largest key
  if (tid == 0) s_counter = 0;
  for (int i = tid; i < P; i += kTopkThreads) s_keys[i] = 0ull;
  __syncthreads();
  for (int64_t i = tid; i < len; i += kTopkThreads) {
    const uint64_t key = make_key(xr, ir, i);
    if (key >= prefix) {
      const uint32_t slot = atomicAdd(&s_counter, 1u);
      if (slot < (uint32_t)k) s_keys[slot] = key;
    }
  }
  __syncthreads();
  bitonic_sort_desc(s_keys, P);
  emit_topk(s_keys, k, out_ids + (int64_t)row * k, out_vals ? out_vals + (int64_t)row * k : nullptr);
}

// ------------------------------------------------------------------ adaptive-k
//
// Reference: cache_hub/adaptive_k_fused/adaptive_topk.cu:108-266 (one 512-thread
// block per row, 31 one-bit radix passes, atomic compaction, bitonic sort, serial
// cumsum) with the semantics of adaptive_topk_ref (adaptive_topk.py:255-313).
// Here: eight 8-bit passes over a 64-bit (benefit, position) key, so ties are
// resolved by candidate position and the result is reproducible; sums run in a
// fixed lane/tree order; exp() is a fixed fp32 sequence shared with the CPU checker.

__device__ __forceinline__ float pkv_expf(float x) {
  if (!(x >= -87.0f)) return (x != x) ? x : 0.0f;
  if (x > 88.0f) return __uint_as_float(0x7f800000u);
  const float n = rintf(x * 1.44269504f);
  float r = x - n * 0.693359375f;
  r = r - n * (-2.12194440e-4f);
  float p = 1.9875691500e-4f;
  p = p * r + 1.3981999507e-3f;
  p = p * r + 8.3334519073e-3f;
  p = p * r + 4.1665795894e-2f;
  p = p * r + 1.6666665459e-1f;
  p = p * r + 5.0000001201e-1f;
  const float z = r * r;
  float y = p * z + r;
  y = y + 1.0f;
  return y * __uint_as_float((uint32_t)((int)n + 127) << 23);
}

// Sum over the workgroup's 1024 lanes as a pairwise tree (stride 1, 2, 4, ...): xor butterflies
// inside each wave, then the 16 wave sums.  Every thread returns the same value.
__device__ __forceinline__ float block_tree_sum_1024(float v, float *s_part) {
#pragma unroll
  for (int m = 1; m < PKV_WAVE; m <<= 1) v = v + __shfl_xor(v, m, PKV_WAVE);
  __syncthreads();
  if (pkv_lane() == 0) s_part[threadIdx.x / PKV_WAVE] = v;
  __syncthreads();
  float w[16];
#pragma unroll
  for (int i = 0; i < 16; ++i) w[i] = s_part[i];
#pragma unroll
  for (int h = 1; h < 16; h <<= 1)
#pragma unroll
    for (int i = 0; i < 16; i += 2 * h) w[i] = w[i] + w[i + h];
  return w[0];
}

__device__ __forceinline__ float block_max_1024(float v, float *s_part) {
#pragma unroll
  for (int m = 1; m < PKV_WAVE; m <<= 1) v = fmaxf(v, __shfl_xor(v, m, PKV_WAVE));
  __syncthreads();
  if (pkv_lane() == 0) s_part[threadIdx.x / PKV_WAVE] = v;
  __syncthreads();
  float r = s_part[0];
#pragma unroll
  for (int i = 1; i < 16; ++i) r = fmaxf(r, s_part[i]);
  return r;
}

__device__ __forceinline__ float cand_logit(const void *__restrict__ scores, int dtype, float scale, int64_t i) {
  const float x = (dtype == PKV_DTYPE_BF16) ? pkv_bf16_bits_to_f32(((const uint16_t *)scores)[i])
                                            : ((const float *)scores)[i];
  return x * scale;
}

// One workgroup of 1024 threads per row; dynamic LDS P*8 bytes (P = pow2 >= k_out).
__global__ __launch_bounds__(kTopkThreads) void pkv_adaptive_topk_kernel(
    const float *__restrict__ sl_logits, int64_t sl_stride, const float *__restrict__ sl_vnorm, int64_t slv_stride,
    int64_t sl, const void *__restrict__ cand_scores, int cand_dtype, float cand_scale,
    const float *__restrict__ cand_vnorm, const float *__restrict__ value_norm, int64_t vn_stride, int64_t vn_offset,
    const int64_t *__restrict__ cand_ids, int64_t n_cand, float threshold, int64_t k_out, int P,
    int64_t *__restrict__ adaptive_k, int64_t *__restrict__ topk_ids, float *__restrict__ ws_ben) {
  extern __shared__ uint64_t s_keys[];
  __shared__ float s_part[16];
  __shared__ uint32_t s_hist[257];
  __shared__ uint32_t s_digit, s_need, s_counter;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float *sll = sl_logits + (int64_t)row * sl_stride;
  const float *slv = sl_vnorm + (int64_t)row * slv_stride;
  const char *cs = (const char *)cand_scores + (int64_t)row * n_cand * (cand_dtype == PKV_DTYPE_BF16 ? 2 : 4);
  const int64_t *ci = cand_ids + (int64_t)row * n_cand;
  const float *cv = cand_vnorm ? cand_vnorm + (int64_t)row * n_cand : nullptr;
  const float *vn = value_norm ? value_norm + (int64_t)row * vn_stride : nullptr;
  float *ben = ws_ben + (int64_t)row * n_cand;

  // joint max of the dense (sink/local) logits and the candidate logits
  float m = -__uint_as_float(0x7f800000u);
  for (int64_t i = tid; i < sl; i += kTopkThreads) m = fmaxf(m, sll[i]);
  for (int64_t i = tid; i < n_cand; i += kTopkThreads) m = fmaxf(m, cand_logit(cs, cand_dtype, cand_scale, i));
  const float g = block_max_1024(m, s_part);

  float acc = 0.f;
  for (int64_t i = tid; i < sl; i += kTopkThreads) acc = acc + pkv_expf(sll[i] - g) * slv[i];
  const float sl_benefit = block_tree_sum_1024(acc, s_part);
  acc = 0.f;
  for (int64_t i = tid; i < n_cand; i += kTopkThreads) {
    const float vnorm = cv ? cv[i] : vn[ci[i] + vn_offset];
    const float b = pkv_expf(cand_logit(cs, cand_dtype, cand_scale, i) - g) * vnorm;
    ben[i] = b;
    acc = acc + b;
  }
  const float total = sl_benefit + block_tree_sum_1024(acc, s_part);
  __syncthreads();  // ben[] of this row is complete (written and read by this workgroup only)

  // k_out-th largest (benefit, ~position) key
  uint64_t prefix = 0;
  uint32_t need = (uint32_t)k_out;
  for (int pass = 0; pass < 8; ++pass) {
    const int shift = 56 - 8 * pass;
    if (tid < 257) s_hist[tid] = 0;
    __syncthreads();
    for (int64_t i = tid; i < n_cand; i += kTopkThreads) {
      const uint64_t key = make_key(ben, nullptr, i);
      if (pass == 0 || (key >> (shift + 8)) == (prefix >> (shift + 8)))
        atomicAdd(&s_hist[(uint32_t)(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    uint32_t suf = 0, suf_next = 0;
    if (tid < 256) {
      for (int d = tid + 1; d < 256; ++d) suf_next += s_hist[d];
      suf = suf_next + s_hist[tid];
    }
    __syncthreads();
    if (tid < 256 && suf >= need && suf_next < need) {
      s_digit = (uint32_t)tid;
      s_need = need - suf_next;
    }
    __syncthreads();
    prefix |= (uint64_t)s_digit << shift;
    need = s_need;
  }
  if (tid == 0) s_counter = 0;
  for (int i = tid; i < P; i += kTopkThreads) s_keys[i] = 0ull;
  __syncthreads();
  for (int64_t i = tid; i < n_cand; i += kTopkThreads) {
    const uint64_t key = make_key(ben, nullptr, i);
    if (key >= prefix) {
      const uint32_t slot = atomicAdd(&s_counter, 1u);
      if (slot < (uint32_t)k_out) s_keys[slot] = key;
    }
  }
  __syncthreads();
  bitonic_sort_desc(s_keys, P);

  // smallest k with sl_benefit + cumsum_k >= threshold * total (sequential fp32 cumsum)
  if (tid == 0) {
    int64_t k = k_out;
    if (total <= 0.f) {
      k = 1;
    } else {
      float csum = 0.f;
      const float tgt = threshold * total;
      for (int64_t i = 0; i < k_out; ++i) {
        csum = csum + pkv_from_ordered_u32((uint32_t)(s_keys[i] >> 32));
        if (sl_benefit + csum >= tgt) {
          k = i + 1;
          break;
        }
      }
    }
    adaptive_k[row] = k;
  }
  for (int64_t i = tid; i < k_out; i += kTopkThreads) {
    const uint32_t pos = ~(uint32_t)s_keys[i];
    topk_ids[(int64_t)row * k_out + i] = (pos < (uint64_t)n_cand) ? ci[pos] : 0;
  }
}

static int pow2_ceil(int64_t v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

}  // namespace

int pkv_launch_select(const uint8_t *cnt_u8, int64_t cnt_stride, const uint16_t *chunk_hist, int chunk_keys, int rows,
                      int64_t n_keys, int64_t k, int64_t *out, hipStream_t s) {
  PKV_REQUIRE(k >= 1 && k < n_keys, "select needs 1 <= k < n_keys (k=%lld n=%lld)", (long long)k,
              (long long)n_keys);
  PKV_REQUIRE(cnt_stride % 16 == 0 && cnt_stride >= n_keys && pkv_aligned(cnt_u8, 16),
              "count rows must be 16-byte aligned and padded");
  const int64_t n_chunks = (n_keys + chunk_keys - 1) / chunk_keys;
  dim3 grid((unsigned)n_chunks, (unsigned)rows);
  hipLaunchKernelGGL(pkv_select_kernel, grid, dim3(kSelThreads), 0, s, cnt_u8, cnt_stride, chunk_hist, chunk_keys,
                     n_keys, k, out);
  PKV_LAUNCH_CHECK("pkv_select_kernel");
  return PKV_OK;
}

PKV_INTERNAL int pkv_launch_identity_fill(int64_t *out, int64_t len, int64_t k, int rows, hipStream_t s) {
  const int64_t total = (int64_t)rows * k;
  hipLaunchKernelGGL(pkv_identity_fill_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, out, len, k,
                     rows);
  PKV_LAUNCH_CHECK("pkv_identity_fill_kernel");
  return PKV_OK;
}

static void bucket_ws_layout(int rows, int64_t len, int &chunk_keys, int64_t &cnt_stride, size_t &off_hist,
                             size_t &total) {
  chunk_keys = pkv_pick_chunk_keys(rows, len);
  cnt_stride = (int64_t)pkv_align_up((size_t)len, 16);
  const int64_t n_chunks = (len + chunk_keys - 1) / chunk_keys;
  off_hist = pkv_align_up((size_t)rows * (size_t)cnt_stride, 256);
  total = off_hist + pkv_align_up((size_t)rows * (size_t)n_chunks * 128 * sizeof(uint16_t), 256);
}

extern "C" size_t pkv_bucket_topk_ws_bytes(int rows, int64_t len) {
  if (rows <= 0 || len <= 0) return 256;
  int ck;
  int64_t cs;
  size_t oh, tot;
  bucket_ws_layout(rows, len, ck, cs, oh, tot);
  return tot;
}

extern "C" int pkv_bucket_topk(const int32_t *x, int64_t x_stride, int rows, int64_t len, int64_t k, int64_t *out,
                               void *ws, size_t ws_bytes, void *stream) {
  PKV_REQUIRE(x && out, "pkv_bucket_topk: null pointer");
  PKV_REQUIRE(k > 0, "k must be positive");                       // radix_topk.cu:264
  PKV_REQUIRE(k <= len, "k cannot exceed sequence length");       // radix_topk.cu:269
  PKV_REQUIRE(rows > 0 && rows <= 65535 && len <= PKV_MAX_KEYS_PER_ROW, "bad shape rows=%d len=%lld", rows,
              (long long)len);
  hipStream_t s = (hipStream_t)stream;
  if (len == k) return pkv_launch_identity_fill(out, len, k, rows, s);
  int ck;
  int64_t cs;
  size_t oh, tot;
  bucket_ws_layout(rows, len, ck, cs, oh, tot);
  if (!ws || ws_bytes < tot || !pkv_aligned(ws, 256)) {
    pkv_set_error("pkv_bucket_topk: workspace of %zu bytes (256-aligned) required, got %zu", tot, ws_bytes);
    return PKV_ENOMEM;
  }
  uint8_t *cnt = (uint8_t *)ws;
  uint16_t *hist = (uint16_t *)((char *)ws + oh);
  const int64_t n_chunks = (len + ck - 1) / ck;
  hipLaunchKernelGGL(pkv_counts_to_u8_kernel, dim3((unsigned)n_chunks, (unsigned)rows), dim3(256), 0, s, x, x_stride,
                     len, cnt, cs, hist, ck);
  PKV_LAUNCH_CHECK("pkv_counts_to_u8_kernel");
  return pkv_launch_select(cnt, cs, hist, ck, rows, len, k, out, s);
}

size_t pkv_topk_ws_bytes_impl(int, int64_t, int64_t) { return 256; }

extern "C" size_t pkv_topk_f32_ws_bytes(int rows, int64_t len, int64_t k) {
  return pkv_topk_ws_bytes_impl(rows, len, k);
}

int pkv_launch_topk_f32(const float *x, int64_t x_stride, const int64_t *ids, int64_t ids_stride, int rows,
                        int64_t len, int64_t k, int64_t *out_ids, float *out_vals, void *, size_t, hipStream_t s) {
  PKV_REQUIRE(x && out_ids, "pkv_topk_f32: null pointer");
  PKV_REQUIRE(k > 0, "k must be positive");
  PKV_REQUIRE(k <= len, "k cannot exceed sequence length");
  PKV_REQUIRE(rows > 0 && len < ((int64_t)1 << 31), "bad shape rows=%d len=%lld", rows, (long long)len);
  if (len <= kTopkMaxSort) {
    const int P = pow2_ceil(len);
    hipLaunchKernelGGL(pkv_topk_sort_kernel, dim3((unsigned)rows), dim3(kTopkThreads), (size_t)P * 8, s, x, x_stride,
                       ids, ids_stride, (int)len, P, k, out_ids, out_vals);
    PKV_LAUNCH_CHECK("pkv_topk_sort_kernel");
  } else {
    PKV_REQUIRE(k <= kTopkMaxSort, "k up to %d supported when len > %d (got %lld)", kTopkMaxSort, kTopkMaxSort,
                (long long)k);
    const int P = pow2_ceil(k);
    hipLaunchKernelGGL(pkv_topk_radix_kernel, dim3((unsigned)rows), dim3(kTopkThreads), (size_t)P * 8, s, x,
                       x_stride, ids, ids_stride, len, P, k, out_ids, out_vals);
    PKV_LAUNCH_CHECK("pkv_topk_radix_kernel");
  }
  return PKV_OK;
}

extern "C" int pkv_topk_f32(const float *x, int64_t x_stride, const int64_t *ids, int64_t ids_stride, int rows,
                            int64_t len, int64_t k, int64_t *out_ids, float *out_vals, void *ws, size_t ws_bytes,
                            void *stream) {
  return pkv_launch_topk_f32(x, x_stride, ids, ids_stride, rows, len, k, out_ids, out_vals, ws, ws_bytes,
                             (hipStream_t)stream);
}

extern "C" size_t pkv_adaptive_topk_ws_bytes(int rows, int64_t n_cand, int64_t) {
  if (rows <= 0 || n_cand <= 0) return 256;
  return pkv_align_up((size_t)rows * (size_t)n_cand * sizeof(float), 256);
}

extern "C" int pkv_adaptive_topk(const float *sl_logits, int64_t sl_stride, const float *sl_vnorm, int64_t slv_stride,
                                 int64_t sl, const void *cand_scores, int cand_dtype, float cand_scale,
                                 const float *cand_vnorm, const float *value_norm, int64_t vn_stride, int64_t vn_offset,
                                 const int64_t *cand_ids, int64_t n_cand, float threshold, int64_t k_out, int rows,
                                 int64_t *adaptive_k, int64_t *topk_ids, void *ws, size_t ws_bytes, void *stream) {
  PKV_REQUIRE(cand_scores && cand_ids && adaptive_k && topk_ids && (cand_vnorm || value_norm),
              "pkv_adaptive_topk: null pointer");
  PKV_REQUIRE(sl >= 0 && (sl == 0 || (sl_logits && sl_vnorm)), "pkv_adaptive_topk: dense logits missing");
  PKV_REQUIRE(cand_dtype == PKV_DTYPE_F32 || cand_dtype == PKV_DTYPE_BF16, "unknown candidate score dtype %d", cand_dtype);
  PKV_REQUIRE(rows > 0 && n_cand > 0 && n_cand < ((int64_t)1 << 31) && k_out > 0 && k_out <= n_cand,
              "need 0 < k_out <= n_cand (k_out=%lld n_cand=%lld rows=%d)", (long long)k_out, (long long)n_cand, rows);
  PKV_REQUIRE(k_out <= kTopkMaxSort, "k_out up to %d supported (got %lld)", kTopkMaxSort, (long long)k_out);
  const size_t need = pkv_adaptive_topk_ws_bytes(rows, n_cand, k_out);
  if (!ws || ws_bytes < need || !pkv_aligned(ws, 16)) {
    pkv_set_error("pkv_adaptive_topk: workspace of %zu bytes required, got %zu", need, ws_bytes);
    return PKV_ENOMEM;
  }
  const int P = pow2_ceil(k_out);
  hipLaunchKernelGGL(pkv_adaptive_topk_kernel, dim3((unsigned)rows), dim3(kTopkThreads), (size_t)P * 8,
                     (hipStream_t)stream, sl_logits, sl_stride, sl_vnorm, slv_stride, sl, cand_scores, cand_dtype,
                     cand_scale, cand_vnorm, value_norm, vn_stride, vn_offset, cand_ids, n_cand, threshold, k_out, P,
                     adaptive_k, topk_ids, (float *)ws);
  PKV_LAUNCH_CHECK("pkv_adaptive_topk_kernel");
  return PKV_OK;
}
