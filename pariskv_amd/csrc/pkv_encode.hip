// Encode-on-append: normalise, SRHT rotate, sign code per 8-dim block, 3-bit
// magnitude code per dim, per-block rerank weight, cluster-size histogram.
//
// Reference: cache_hub/polar_cache.py:924-978 (batch_encode: ~15 torch launches,
// three permute copies and [.,S,16,8] intermediates) and :980-996
// (_count_cluster_keys: bincount per batch element).
//
// One key is handled by 16 lanes, lane s owning the 8 dims of block s, so four
// keys share a wave64.  The 128-point Walsh-Hadamard transform is three in-lane
// butterfly stages plus four cross-lane stages (lane xor 1,2,4,8); everything
// after the rotation is lane-local.  256 B read + 112 B written per key.
//
// The order of every floating-point operation is fixed (and contraction into
// FMA is disabled at build time) because the integer outputs must be
// reproducible bit for bit:
//   sum of squares: sequential inside a block, then a pairwise tree over blocks.
#include "pkv_common.h"

namespace {

constexpr int kEncThreads = 256;
constexpr int kEncKeysPerIter = kEncThreads / 16;  // 16
constexpr int kEncKeysPerBlock = 256;

__constant__ float c_thresholds[7] = {0.08447265625f, 0.169921875f, 0.2578125f, 0.349609375f,
                                      0.44921875f,    0.55859375f,  0.69140625f};
__constant__ float c_centers[8] = {0.0419921875f, 0.126953125f, 0.212890625f, 0.302734375f,
                                   0.396484375f,  0.5f,         0.6171875f,   0.76171875f};

// BF16 = the rounding chain of the reference's bf16 tensors (compile-time, so that no rounding point branches).
template <bool BF16>
__global__ __launch_bounds__(kEncThreads) void pkv_encode_kernel(
    const void *__restrict__ keys, int n_kv_heads, int64_t n_keys, int64_t k_stride_b, int64_t k_stride_h,
    int64_t k_stride_key, const float *__restrict__ signs, uint8_t *__restrict__ codes, int64_t cs_b, int64_t cs_h,
    int64_t cs_key, int64_t cs_sub, uint8_t *__restrict__ nib, int64_t ns_b, int64_t ns_h, int64_t ns_key,
    int64_t ns_sub, uint16_t *__restrict__ weight, int64_t ws_b, int64_t ws_h, int64_t ws_key, int64_t ws_sub,
    int32_t *__restrict__ cluster_counts, int64_t cc_b, int64_t cc_h) {
  constexpr int dtype = BF16 ? PKV_DTYPE_BF16 : PKV_DTYPE_F32;
  const int row = blockIdx.y;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  const int tid = threadIdx.x;
  const int s = tid & 15;   // block (subspace) owned by this lane
  const int kq = tid >> 4;  // key slot inside the iteration

  __shared__ uint32_t s_hist[16 * 256];
  __shared__ float s_centers[8];  // magnitude centres, looked up by code (an LDS read instead of a load from constant memory)
  if (tid < 8) s_centers[tid] = c_centers[tid];
  if (!cluster_counts) __syncthreads();
  if (cluster_counts) {
    for (int i = tid; i < 16 * 256; i += kEncThreads) s_hist[i] = 0;
    __syncthreads();
  }

  float sg[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) sg[j] = signs[8 * s + j];

  const int64_t key_begin = (int64_t)blockIdx.x * kEncKeysPerBlock;
  for (int it = 0; it < kEncKeysPerBlock / kEncKeysPerIter; ++it) {
    const int64_t key = key_begin + it * kEncKeysPerIter + kq;
    const bool active = key < n_keys;
    const int64_t kload = active ? key : n_keys - 1;  // keep all lanes in the shuffles
    const int64_t off = (int64_t)b * k_stride_b + (int64_t)h * k_stride_h + kload * k_stride_key + 8 * s;
    float x[8];
    if (BF16) {
      const pkv_u32x4 v = *(const pkv_u32x4 *)((const uint16_t *)keys + off);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        x[2 * p] = __uint_as_float(w[p] << 16);
        x[2 * p + 1] = __uint_as_float(w[p] & 0xffff0000u);
      }
    } else {
      const float4 a = *(const float4 *)((const float *)keys + off);
      const float4 c = *(const float4 *)((const float *)keys + off + 4);
      x[0] = a.x, x[1] = a.y, x[2] = a.z, x[3] = a.w, x[4] = c.x, x[5] = c.y, x[6] = c.z, x[7] = c.w;
    }
    float y[8];
    const float n = pkv_normalize_rotate_16(x, sg, s, dtype, y);

    uint32_t code = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) code |= (y[j] >= 0.0f) ? (1u << j) : 0u;

    if (active) {
      codes[(int64_t)b * cs_b + (int64_t)h * cs_h + key * cs_key + (int64_t)s * cs_sub] = (uint8_t)code;
      if (cluster_counts) atomicAdd(&s_hist[s * 256 + code], 1u);
    }
    if (nib || weight) {
      float r2 = y[0] * y[0];
#pragma unroll
      for (int j = 1; j < 8; ++j) r2 = r2 + y[j] * y[j];
      const float r = pkv_rdt(sqrtf(r2), dtype);
      const float rden = r < 1e-8f ? 1e-8f : r;
      uint32_t packed = 0;
      float alpha = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float u = pkv_rdt(y[j] / rden, dtype);
        const float au = fabsf(u);
        // t = number of thresholds below au (the thresholds ascend): three compares instead of seven
        const bool b2 = c_thresholds[3] < au;
        const bool b1 = (b2 ? c_thresholds[5] : c_thresholds[1]) < au;
        const float tl = b2 ? (b1 ? c_thresholds[6] : c_thresholds[4]) : (b1 ? c_thresholds[2] : c_thresholds[0]);
        const int t = (b2 ? 4 : 0) + (b1 ? 2 : 0) + ((tl < au) ? 1 : 0);
        packed |= (uint32_t)(((y[j] >= 0.0f) ? 8 : 0) | t) << (4 * j);
        const float p = pkv_rdt(s_centers[t] * au, dtype);
        alpha = (j == 0) ? p : alpha + p;
      }
      if (alpha < 1e-6f) alpha = 1e-6f;
      if (active) {
        if (nib)
          *(uint32_t *)(nib + (int64_t)b * ns_b + (int64_t)h * ns_h + key * ns_key + (int64_t)s * ns_sub) = packed;
        if (weight) {
          const float w = (r / alpha) * n;
          weight[(int64_t)b * ws_b + (int64_t)h * ws_h + key * ws_key + (int64_t)s * ws_sub] = pkv_f32_to_bf16_bits(w);
        }
      }
    }
  }
  if (cluster_counts) {
    __syncthreads();
    int32_t *cc = cluster_counts + (int64_t)b * cc_b + (int64_t)h * cc_h;
    for (int i = tid; i < 16 * 256; i += kEncThreads) {
      const uint32_t v = s_hist[i];
      if (v) atomicAdd(&cc[i], (int32_t)v);
    }
  }
}

// Histogram of existing codes into cluster_counts (+=).  grid (ceil(n/4096), R).
__global__ __launch_bounds__(256) void pkv_count_clusters_kernel(const uint8_t *__restrict__ codes, int64_t cs_b,
                                                                 int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                                                                 int n_kv_heads, int64_t n_keys,
                                                                 int32_t *__restrict__ cluster_counts, int64_t cc_b,
                                                                 int64_t cc_h) {
  const int row = blockIdx.y;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  __shared__ uint32_t s_hist[16 * 256];
  for (int i = threadIdx.x; i < 16 * 256; i += 256) s_hist[i] = 0;
  __syncthreads();
  const uint8_t *base = codes + (int64_t)b * cs_b + (int64_t)h * cs_h;
  const int64_t k0 = (int64_t)blockIdx.x * 4096;
  const int64_t k1 = (k0 + 4096 < n_keys) ? k0 + 4096 : n_keys;
  for (int64_t e = k0 * 16 + threadIdx.x; e < k1 * 16; e += 256) {
    const int64_t key = e >> 4;
    const int s = (int)(e & 15);
    atomicAdd(&s_hist[s * 256 + base[key * cs_key + (int64_t)s * cs_sub]], 1u);
  }
  __syncthreads();
  int32_t *cc = cluster_counts + (int64_t)b * cc_b + (int64_t)h * cc_h;
  for (int i = threadIdx.x; i < 16 * 256; i += 256) {
    const uint32_t v = s_hist[i];
    if (v) atomicAdd(&cc[i], (int32_t)v);
  }
}

}  // namespace

extern "C" int pkv_encode_append(const void *keys, int dtype, int bs, int n_kv_heads, int64_t n_keys,
                                 int64_t k_stride_b, int64_t k_stride_h, int64_t k_stride_key, const float *signs,
                                 uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                                 uint8_t *nib, int64_t ns_b, int64_t ns_h, int64_t ns_key, int64_t ns_sub,
                                 uint16_t *weight, int64_t ws_b, int64_t ws_h, int64_t ws_key, int64_t ws_sub,
                                 int32_t *cluster_counts, int64_t cc_b, int64_t cc_h, void *stream) {
  PKV_REQUIRE(keys && signs && codes, "pkv_encode_append: null pointer");
  PKV_REQUIRE(dtype == PKV_DTYPE_F32 || dtype == PKV_DTYPE_BF16, "unknown dtype %d", dtype);
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && (int64_t)bs * n_kv_heads <= 65535, "bad shape bs=%d kv_heads=%d", bs,
              n_kv_heads);
  if (n_keys == 0) return PKV_OK;
  PKV_REQUIRE(n_keys > 0, "n_keys must be >= 0");
  const int64_t vec = dtype == PKV_DTYPE_BF16 ? 8 : 4;  // elements per 16 bytes
  PKV_REQUIRE(pkv_aligned(keys, 16) && k_stride_b % vec == 0 && k_stride_h % vec == 0 && k_stride_key % vec == 0,
              "keys must be 16-byte aligned with 16-byte-multiple strides");
  PKV_REQUIRE(!nib || (pkv_aligned(nib, 4) && ns_b % 4 == 0 && ns_h % 4 == 0 && ns_key % 4 == 0 && ns_sub % 4 == 0),
              "packed 4-bit blocks must be 4-byte aligned");
  dim3 grid((unsigned)((n_keys + kEncKeysPerBlock - 1) / kEncKeysPerBlock), (unsigned)(bs * n_kv_heads));
#define PKV_ENC(BF)                                                                                                  \
  hipLaunchKernelGGL(pkv_encode_kernel<BF>, grid, dim3(kEncThreads), 0, (hipStream_t)stream, keys, n_kv_heads, n_keys, \
                     k_stride_b, k_stride_h, k_stride_key, signs, codes, cs_b, cs_h, cs_key, cs_sub, nib, ns_b, ns_h,  \
                     ns_key, ns_sub, weight, ws_b, ws_h, ws_key, ws_sub, cluster_counts, cc_b, cc_h)
  if (dtype == PKV_DTYPE_BF16) PKV_ENC(true); else PKV_ENC(false);
#undef PKV_ENC
  PKV_LAUNCH_CHECK("pkv_encode_kernel");
  return PKV_OK;
}

extern "C" int pkv_count_cluster_keys(const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                                      int bs, int n_kv_heads, int64_t n_keys, int32_t *cluster_counts, int64_t cc_b,
                                      int64_t cc_h, void *stream) {
  PKV_REQUIRE(codes && cluster_counts, "pkv_count_cluster_keys: null pointer");
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && (int64_t)bs * n_kv_heads <= 65535 && n_keys >= 0, "bad shape");
  if (n_keys == 0) return PKV_OK;
  dim3 grid((unsigned)((n_keys + 4095) / 4096), (unsigned)(bs * n_kv_heads));
  hipLaunchKernelGGL(pkv_count_clusters_kernel, grid, dim3(256), 0, (hipStream_t)stream, codes, cs_b, cs_h, cs_key,
                     cs_sub, n_kv_heads, n_keys, cluster_counts, cc_b, cc_h);
  PKV_LAUNCH_CHECK("pkv_count_clusters_kernel");
  return PKV_OK;
}
