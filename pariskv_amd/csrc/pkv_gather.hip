// Row gathers of the selected K/V: out of pinned host memory through the GPU's
// unified addressing (PCIe reads issued by the kernel), or HBM to HBM.
//
// Reference: cache_hub/gather_trans/trans_h2d.cu:19-121 (h2d_gather_kv_kernel:
// one 32-thread block per selected index, 16 lanes per 256-byte row) and the
// torch.gather branch cache_hub/polar_cache.py:1089-1095.  Here a wave64 moves
// four 256-byte rows per instruction and every lane keeps several independent
// 16-byte reads in flight, which is what a latency-bound PCIe read stream needs.
#include "pkv_common.h"

namespace {

constexpr int kGatherThreads = 256;
constexpr int kGatherUnroll = 4;  // independent row reads per lane

// task t in [0, rows*k*2): kv = t & 1, (row, slot) = divmod(t >> 1, k).  With row_counts, row r only
// moves its first row_counts[r] slots (the others leave dst untouched).
// `vpr` = 16-byte vectors per row; consecutive lanes cover one row.
__global__ __launch_bounds__(kGatherThreads) void pkv_gather_rows_kernel(
    const pkv_u32x4 *__restrict__ src_k, const pkv_u32x4 *__restrict__ src_v, int64_t src_len,
    const int64_t *__restrict__ idx, int64_t k, int64_t idx_offset, pkv_u32x4 *__restrict__ dst_k,
    pkv_u32x4 *__restrict__ dst_v, int64_t dst_len, int64_t dst_row0, int64_t n_tasks, int vpr,
    const int64_t *__restrict__ row_counts) {
  const int64_t lanes_per_block = kGatherThreads;
  const int64_t g0 = (int64_t)blockIdx.x * lanes_per_block * kGatherUnroll + threadIdx.x;
  pkv_u32x4 val[kGatherUnroll];
  pkv_u32x4 *dst[kGatherUnroll];
#pragma unroll
  for (int u = 0; u < kGatherUnroll; ++u) {
    const int64_t g = g0 + (int64_t)u * lanes_per_block;
    const int64_t task = g / vpr;
    const int lane = (int)(g % vpr);
    dst[u] = nullptr;
    val[u] = pkv_u32x4{0u, 0u, 0u, 0u};
    if (task < n_tasks) {
      const int kv = (int)(task & 1);
      const int64_t rs = task >> 1;
      const int64_t row = rs / k, slot = rs % k;
      if (row_counts && slot >= row_counts[row]) continue;  // ragged selection: this row takes fewer than k
      const int64_t i = idx[rs] + idx_offset;
      const pkv_u32x4 *src = kv ? src_v : src_k;
      pkv_u32x4 *d = kv ? dst_v : dst_k;
      dst[u] = d + ((row * dst_len + dst_row0 + slot) * vpr + lane);
      if ((uint64_t)i < (uint64_t)src_len) val[u] = src[(row * src_len + i) * vpr + lane];
    }
  }
#pragma unroll
  for (int u = 0; u < kGatherUnroll; ++u)
    if (dst[u]) *dst[u] = val[u];
}

// Ragged form: virtual head v owns slots [cu_topk[v], cu_topk[v+1]) of
// idx_packed and writes rows cu_k[v] + sink_local_end + s of the packed
// destination.  grid (ceil(max_k * vpr * 2 / 256), V).
__global__ __launch_bounds__(kGatherThreads) void pkv_gather_packed_kernel(
    const pkv_u32x4 *__restrict__ src_k, const pkv_u32x4 *__restrict__ src_v, int64_t src_len,
    const int64_t *__restrict__ idx_packed, const int32_t *__restrict__ cu_topk, const int32_t *__restrict__ cu_k,
    int64_t sink_local_end, pkv_u32x4 *__restrict__ dst_k, pkv_u32x4 *__restrict__ dst_v, int64_t total_k, int vpr) {
  const int v = blockIdx.y;
  const int64_t g = (int64_t)blockIdx.x * kGatherThreads + threadIdx.x;
  const int64_t task = g / vpr;
  const int lane = (int)(g % vpr);
  const int kv = (int)(task & 1);
  const int64_t s = task >> 1;
  const int64_t begin = cu_topk[v];
  const int64_t n = (int64_t)cu_topk[v + 1] - begin;
  if (s >= n) return;
  const int64_t drow = (int64_t)cu_k[v] + sink_local_end + s;
  if (drow < 0 || drow >= total_k) return;
  const int64_t i = idx_packed[begin + s];
  pkv_u32x4 val = pkv_u32x4{0u, 0u, 0u, 0u};
  if ((uint64_t)i < (uint64_t)src_len) val = (kv ? src_v : src_k)[((int64_t)v * src_len + i) * vpr + lane];
  (kv ? dst_v : dst_k)[drow * vpr + lane] = val;
}

// One new token per sequence: row (b, h) of k_new / v_new goes to row `slot` of
// the [bs][h][dst_len] K and V stores.  Lane g: (task, lane) = divmod(g, vpr),
// kv = task & 1, (b, h) = divmod(task >> 1, n_heads).  Strides in 16-byte vectors.
// VNORM (0 off, 1 bf16 rows, 2 fp32 rows): the value row's Euclidean norm also goes to
// vnorm[b*vn_stride_b + h*vn_stride_h + slot] as fp32: a lane adds the squares of its 16 bytes in
// order, the vpr lanes of the row meet in a pairwise tree (lane ^ 1, 2, 4, ...), then the square
// root, rounded to bf16 for bf16 rows (the norm of a bf16 tensor is a bf16 tensor).
template <int VNORM>
__global__ __launch_bounds__(kGatherThreads) void pkv_append_rows_kernel(
    const pkv_u32x4 *__restrict__ k_new, const pkv_u32x4 *__restrict__ v_new, int64_t k_stride_b, int64_t k_stride_h,
    int64_t v_stride_b, int64_t v_stride_h, pkv_u32x4 *__restrict__ dst_k, pkv_u32x4 *__restrict__ dst_v,
    int64_t dst_stride_b, int64_t dst_stride_h, int64_t slot, int n_heads, int n_tasks, int vpr,
    float *__restrict__ vnorm, int64_t vn_stride_b, int64_t vn_stride_h) {
  const int g = blockIdx.x * kGatherThreads + threadIdx.x;
  const int task = g / vpr, lane = g % vpr;
  if (task >= n_tasks) return;
  const int kv = task & 1;
  const int b = (task >> 1) / n_heads, h = (task >> 1) % n_heads;
  const pkv_u32x4 val = kv ? v_new[b * v_stride_b + h * v_stride_h + lane] : k_new[b * k_stride_b + h * k_stride_h + lane];
  (kv ? dst_v : dst_k)[b * dst_stride_b + h * dst_stride_h + slot * vpr + lane] = val;
  if (VNORM != 0) {  // tasks are whole groups of vpr lanes inside a wave: every lane of a row is here
    const uint32_t w[4] = {val.x, val.y, val.z, val.w};
    float acc;
    if (VNORM == 1) {
      float e[8];
#pragma unroll
      for (int p = 0; p < 4; ++p) e[2 * p] = __uint_as_float(w[p] << 16), e[2 * p + 1] = __uint_as_float(w[p] & 0xffff0000u);
      acc = e[0] * e[0];
#pragma unroll
      for (int j = 1; j < 8; ++j) acc = acc + e[j] * e[j];
    } else {
      acc = __uint_as_float(w[0]) * __uint_as_float(w[0]);
#pragma unroll
      for (int j = 1; j < 4; ++j) acc = acc + __uint_as_float(w[j]) * __uint_as_float(w[j]);
    }
    acc = acc + pkv_lane_xor_f<1>(acc);
    acc = acc + pkv_lane_xor_f<2>(acc);
    acc = acc + pkv_lane_xor_f<4>(acc);
    acc = acc + pkv_lane_xor_f<8>(acc);
    if (VNORM == 2) acc = acc + pkv_lane_xor_f<16>(acc);
    if (kv && lane == 0) {
      const float n = sqrtf(acc);
      vnorm[b * vn_stride_b + h * vn_stride_h + slot] = VNORM == 1 ? pkv_bf16_round(n) : n;
    }
  }
}

// Blocks of consecutive rows, one block per (batch, head), from the GPU into the pinned host store:
// dst[(b,h)][dst_row0 + r] = src[(b,h)][r] for K and V.  16-byte vectors, a wave writes 1 KB of
// consecutive host memory per instruction (posted PCIe writes).  grid-stride over all vectors.
__global__ __launch_bounds__(kGatherThreads) void pkv_offload_rows_kernel(
    const pkv_u32x4 *__restrict__ src_k, const pkv_u32x4 *__restrict__ src_v, int64_t src_stride_b,
    int64_t src_stride_h, int64_t src_stride_row, pkv_u32x4 *__restrict__ dst_k, pkv_u32x4 *__restrict__ dst_v,
    int64_t dst_len, int64_t dst_row0, int64_t n_rows, int n_heads, int64_t n_vec, int vpr) {
  const int64_t per_head = n_rows * vpr;  // vectors of one (b, h) block
  for (int64_t g = (int64_t)blockIdx.x * kGatherThreads + threadIdx.x; g < n_vec;
       g += (int64_t)gridDim.x * kGatherThreads) {
    const int64_t kvbh = g / per_head, in_block = g % per_head;
    const int kv = (int)(kvbh & 1);
    const int64_t bh = kvbh >> 1, b = bh / n_heads, h = bh % n_heads;
    const int64_t row = in_block / vpr;
    const int lane = (int)(in_block % vpr);
    const pkv_u32x4 val = (kv ? src_v : src_k)[b * src_stride_b + h * src_stride_h + row * src_stride_row + lane];
    (kv ? dst_v : dst_k)[(bh * dst_len + dst_row0 + row) * vpr + lane] = val;
  }
}

// Plain streaming copy of n 16-byte vectors (calibration of HBM counters, tests).
__global__ __launch_bounds__(256) void pkv_copy_kernel(const pkv_u32x4 *__restrict__ src, pkv_u32x4 *__restrict__ dst,
                                                       int64_t n) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

// Plain streaming read of n 16-byte vectors (what a read-only kernel can pull out of HBM; one word per
// wave is written so that the loads cannot be dropped).  Same access pattern as the collision scan:
// 256-thread workgroups, four 128-bit non-temporal loads per thread in flight.
__global__ __launch_bounds__(256) void pkv_read_kernel(const pkv_u32x4 *__restrict__ src, uint32_t *__restrict__ sink,
                                                       int64_t n) {
  constexpr int kChunk = 4096;  // vectors per workgroup: one contiguous 64 KB slab, like a scan chunk
  const int64_t k0 = (int64_t)blockIdx.x * kChunk, k1 = k0 + kChunk < n ? k0 + kChunk : n;
  uint32_t acc = 0;
  for (int64_t i = k0 + threadIdx.x; i < k1; i += 4 * 256) {
    pkv_u32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t j = i + u * 256;
      v[u] = j < k1 ? __builtin_nontemporal_load(src + j) : pkv_u32x4{0u, 0u, 0u, 0u};
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
#pragma unroll
  for (int m = 1; m < PKV_WAVE; m <<= 1) acc ^= (uint32_t)__shfl_xor((int)acc, m, PKV_WAVE);
  // a plain store: the sink only keeps the loads alive, and atomics on a few shared words would dominate the kernel
  if ((threadIdx.x & (PKV_WAVE - 1)) == 0) sink[(blockIdx.x * 4 + threadIdx.x / PKV_WAVE) & 63] = acc;
}

int check_common(const void *src_k, const void *src_v, const void *dst_k, const void *dst_v, int rows, int row_bytes) {
  PKV_REQUIRE(src_k && src_v && dst_k && dst_v, "gather: null pointer");
  PKV_REQUIRE(rows > 0, "gather: bad row count %d", rows);
  PKV_REQUIRE(row_bytes > 0 && row_bytes % 16 == 0 && row_bytes <= 4096, "row_bytes must be a multiple of 16 (got %d)",
              row_bytes);
  PKV_REQUIRE(pkv_aligned(src_k, 16) && pkv_aligned(src_v, 16) && pkv_aligned(dst_k, 16) && pkv_aligned(dst_v, 16),
              "gather: buffers must be 16-byte aligned");
  return PKV_OK;
}

int device_view_of_host(const void *host, const void **dev) {
  void *d = nullptr;
  hipError_t e = hipHostGetDevicePointer(&d, const_cast<void *>(host), 0);
  if (e != hipSuccess || d == nullptr) {
    (void)hipGetLastError();
    pkv_set_error("source is not pinned, device-mapped host memory (%s)", hipGetErrorString(e));
    return PKV_EINVAL;
  }
  *dev = d;
  return PKV_OK;
}

}  // namespace

int pkv_launch_gather(const void *src_k, const void *src_v, int64_t src_len, const int64_t *idx, int64_t k,
                      int64_t idx_offset, void *dst_k, void *dst_v, int64_t dst_len, int64_t dst_row0, int rows,
                      int row_bytes, hipStream_t s, const int64_t *row_counts) {
  int rc = check_common(src_k, src_v, dst_k, dst_v, rows, row_bytes);
  if (rc) return rc;
  PKV_REQUIRE(idx && k > 0 && src_len > 0 && dst_row0 >= 0 && dst_row0 + k <= dst_len,
              "gather: k=%lld src_len=%lld dst_row0=%lld dst_len=%lld", (long long)k, (long long)src_len,
              (long long)dst_row0, (long long)dst_len);
  const int vpr = row_bytes / 16;
  const int64_t n_tasks = (int64_t)rows * k * 2;
  const int64_t lanes = n_tasks * vpr;
  const int64_t per_block = (int64_t)kGatherThreads * kGatherUnroll;
  const int64_t blocks = (lanes + per_block - 1) / per_block;
  PKV_REQUIRE(blocks < ((int64_t)1 << 31), "gather too large");
  hipLaunchKernelGGL(pkv_gather_rows_kernel, dim3((unsigned)blocks), dim3(kGatherThreads), 0, s,
                     (const pkv_u32x4 *)src_k, (const pkv_u32x4 *)src_v, src_len, idx, k, idx_offset,
                     (pkv_u32x4 *)dst_k, (pkv_u32x4 *)dst_v, dst_len, dst_row0, n_tasks, vpr, row_counts);
  PKV_LAUNCH_CHECK("pkv_gather_rows_kernel");
  return PKV_OK;
}

extern "C" int pkv_gather_hbm(const void *src_k, const void *src_v, int64_t src_len, const int64_t *idx, int64_t k,
                              int64_t idx_offset, void *dst_k, void *dst_v, int64_t dst_len, int64_t dst_row0, int bs,
                              int n_kv_heads, int row_bytes, void *stream) {
  return pkv_launch_gather(src_k, src_v, src_len, idx, k, idx_offset, dst_k, dst_v, dst_len, dst_row0,
                           bs * n_kv_heads, row_bytes, (hipStream_t)stream);
}

extern "C" int pkv_gather_uva(const void *src_k, const void *src_v, int64_t src_len, const int64_t *idx, int64_t k,
                              int64_t idx_offset, void *dst_k, void *dst_v, int64_t dst_len, int64_t dst_row0, int bs,
                              int n_kv_heads, int row_bytes, void *stream) {
  PKV_REQUIRE(src_k && src_v, "gather: null pointer");
  const void *dk, *dv;
  int rc = device_view_of_host(src_k, &dk);
  if (rc) return rc;
  rc = device_view_of_host(src_v, &dv);
  if (rc) return rc;
  return pkv_launch_gather(dk, dv, src_len, idx, k, idx_offset, dst_k, dst_v, dst_len, dst_row0, bs * n_kv_heads,
                           row_bytes, (hipStream_t)stream);
}

extern "C" int pkv_append_kv(const void *k_new, int64_t k_stride_b, int64_t k_stride_h, const void *v_new,
                             int64_t v_stride_b, int64_t v_stride_h, void *dst_k, void *dst_v, int64_t dst_stride_b,
                             int64_t dst_stride_h, int64_t dst_len, int64_t slot, int bs, int n_kv_heads, int row_bytes,
                             float *vnorm, int64_t vn_stride_b, int64_t vn_stride_h, void *stream) {
  int rc = check_common(k_new, v_new, dst_k, dst_v, bs * n_kv_heads, row_bytes);
  if (rc) return rc;
  PKV_REQUIRE(!vnorm || ((row_bytes == 256 || row_bytes == 512) && vn_stride_b >= 0 && vn_stride_h > slot),
              "append: value norms need rows of 128 bf16 or fp32 elements and a norm row longer than the slot");
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && (int64_t)bs * n_kv_heads <= (1 << 20), "append: bad batch/head count");
  PKV_REQUIRE(slot >= 0 && slot < dst_len, "append: slot %lld outside [0, %lld)", (long long)slot, (long long)dst_len);
  PKV_REQUIRE(k_stride_b % 16 == 0 && k_stride_h % 16 == 0 && v_stride_b % 16 == 0 && v_stride_h % 16 == 0 &&
                  dst_stride_b % 16 == 0 && dst_stride_h % 16 == 0 && k_stride_h >= row_bytes && v_stride_h >= row_bytes &&
                  k_stride_b >= 0 && v_stride_b >= 0 && dst_stride_h >= dst_len * row_bytes && dst_stride_b >= 0,
              "append: strides are bytes, multiples of 16, rows must not overlap");
  const int vpr = row_bytes / 16;
  const int n_tasks = bs * n_kv_heads * 2;
  const int lanes = n_tasks * vpr;
  const dim3 grid((unsigned)((lanes + kGatherThreads - 1) / kGatherThreads));
#define PKV_APPEND(VN)                                                                                              \
  hipLaunchKernelGGL(pkv_append_rows_kernel<VN>, grid, dim3(kGatherThreads), 0, (hipStream_t)stream,                 \
                     (const pkv_u32x4 *)k_new, (const pkv_u32x4 *)v_new, k_stride_b / 16, k_stride_h / 16,          \
                     v_stride_b / 16, v_stride_h / 16, (pkv_u32x4 *)dst_k, (pkv_u32x4 *)dst_v, dst_stride_b / 16,   \
                     dst_stride_h / 16, slot, n_kv_heads, n_tasks, vpr, vnorm, vn_stride_b, vn_stride_h)
  if (!vnorm) PKV_APPEND(0); else if (row_bytes == 256) PKV_APPEND(1); else PKV_APPEND(2);
#undef PKV_APPEND
  PKV_LAUNCH_CHECK("pkv_append_rows_kernel");
  return PKV_OK;
}

extern "C" int pkv_offload_rows(const void *src_k, const void *src_v, int64_t src_stride_b, int64_t src_stride_h,
                                int64_t src_stride_row, void *dst_k_host, void *dst_v_host, int64_t dst_len,
                                int64_t dst_row0, int64_t n_rows, int bs, int n_kv_heads, int row_bytes, void *stream) {
  int rc = check_common(src_k, src_v, dst_k_host, dst_v_host, bs * n_kv_heads, row_bytes);
  if (rc) return rc;
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && n_rows > 0 && dst_row0 >= 0 && dst_row0 + n_rows <= dst_len,
              "offload: rows [%lld, %lld) outside the host store of %lld rows", (long long)dst_row0,
              (long long)(dst_row0 + n_rows), (long long)dst_len);
  PKV_REQUIRE(src_stride_b % 16 == 0 && src_stride_h % 16 == 0 && src_stride_row % 16 == 0 && src_stride_row >= row_bytes,
              "offload: strides are bytes, multiples of 16");
  const void *dk, *dv;
  rc = device_view_of_host(dst_k_host, &dk);
  if (rc) return rc;
  rc = device_view_of_host(dst_v_host, &dv);
  if (rc) return rc;
  const int vpr = row_bytes / 16;
  const int64_t n_vec = (int64_t)2 * bs * n_kv_heads * n_rows * vpr;
  int64_t blocks = (n_vec + kGatherThreads - 1) / kGatherThreads;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(pkv_offload_rows_kernel, dim3((unsigned)blocks), dim3(kGatherThreads), 0, (hipStream_t)stream,
                     (const pkv_u32x4 *)src_k, (const pkv_u32x4 *)src_v, src_stride_b / 16, src_stride_h / 16,
                     src_stride_row / 16, (pkv_u32x4 *)const_cast<void *>(dk), (pkv_u32x4 *)const_cast<void *>(dv), dst_len,
                     dst_row0, n_rows, n_kv_heads, n_vec, vpr);
  PKV_LAUNCH_CHECK("pkv_offload_rows_kernel");
  return PKV_OK;
}

// The same move through the copy engines: hipMemcpyAsync / hipMemcpy2DAsync commands on `stream`, no shader
// kernel, so that kernels on other streams keep the compute units and the shader write path to themselves.
// One command per (b, h) block and tensor: a plain copy where the block's rows are contiguous in the source, a
// pitched copy otherwise; with PKV_OFFLOAD_ONE_COMMAND and a source whose (b, h) blocks are themselves evenly
// spaced (a staging buffer), one pitched copy per tensor whose "rows" are whole blocks.
extern "C" int pkv_offload_rows_dma(const void *src_k, const void *src_v, int64_t src_stride_b, int64_t src_stride_h,
                                    int64_t src_stride_row, void *dst_k_host, void *dst_v_host, int64_t dst_len,
                                    int64_t dst_row0, int64_t n_rows, int bs, int n_kv_heads, int row_bytes, int flags,
                                    void *stream) {
  PKV_REQUIRE(src_k && src_v && dst_k_host && dst_v_host, "offload: null pointer");
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && n_rows > 0 && row_bytes > 0 && dst_row0 >= 0 && dst_row0 + n_rows <= dst_len,
              "offload: rows [%lld, %lld) outside the host store of %lld rows", (long long)dst_row0,
              (long long)(dst_row0 + n_rows), (long long)dst_len);
  PKV_REQUIRE(src_stride_row >= row_bytes && src_stride_b >= 0 && src_stride_h >= 0, "offload: bad source strides");
  hipStream_t st = (hipStream_t)stream;
  const bool rows_contiguous = src_stride_row == row_bytes;
  const size_t block_bytes = (size_t)n_rows * (size_t)row_bytes;
  const size_t dst_block = (size_t)dst_len * (size_t)row_bytes;
  const void *srcs[2] = {src_k, src_v};
  void *dsts[2] = {dst_k_host, dst_v_host};
  const bool blocks_even = rows_contiguous && (bs == 1 || src_stride_b == (int64_t)n_kv_heads * src_stride_h) &&
                           src_stride_h >= (int64_t)block_bytes;
  for (int t = 0; t < 2; ++t) {
    char *d0 = (char *)dsts[t] + (size_t)dst_row0 * (size_t)row_bytes;
    if ((flags & PKV_OFFLOAD_ONE_COMMAND) && blocks_even) {
      PKV_HIP(hipMemcpy2DAsync(d0, dst_block, srcs[t], (size_t)src_stride_h, block_bytes, (size_t)bs * n_kv_heads,
                               hipMemcpyDeviceToHost, st));
      continue;
    }
    for (int b = 0; b < bs; ++b) {
      for (int h = 0; h < n_kv_heads; ++h) {
        const char *sp = (const char *)srcs[t] + (size_t)b * (size_t)src_stride_b + (size_t)h * (size_t)src_stride_h;
        char *dp = d0 + ((size_t)b * n_kv_heads + h) * dst_block;
        if (rows_contiguous) {
          PKV_HIP(hipMemcpyAsync(dp, sp, block_bytes, hipMemcpyDeviceToHost, st));
        } else {
          PKV_HIP(hipMemcpy2DAsync(dp, (size_t)row_bytes, sp, (size_t)src_stride_row, (size_t)row_bytes, (size_t)n_rows,
                                   hipMemcpyDeviceToHost, st));
        }
      }
    }
  }
  return PKV_OK;
}

extern "C" int pkv_gather_uva_ragged(const void *src_k, const void *src_v, int64_t src_len, const int64_t *idx, int64_t k,
                                     const int64_t *row_counts, int64_t idx_offset, void *dst_k, void *dst_v,
                                     int64_t dst_len, int64_t dst_row0, int bs, int n_kv_heads, int row_bytes,
                                     void *stream) {
  PKV_REQUIRE(src_k && src_v && row_counts, "ragged gather: null pointer");
  const void *dk, *dv;
  int rc = device_view_of_host(src_k, &dk);
  if (rc) return rc;
  rc = device_view_of_host(src_v, &dv);
  if (rc) return rc;
  return pkv_launch_gather(dk, dv, src_len, idx, k, idx_offset, dst_k, dst_v, dst_len, dst_row0, bs * n_kv_heads,
                           row_bytes, (hipStream_t)stream, row_counts);
}

extern "C" int pkv_gather_uva_packed(const void *src_k, const void *src_v, int64_t src_len, const int64_t *idx_packed,
                                     const int32_t *cu_topk, const int32_t *cu_k, int64_t sink_local_end,
                                     int64_t max_k, void *dst_k, void *dst_v, int64_t total_k, int bs, int n_kv_heads,
                                     int row_bytes, void *stream) {
  int rc = check_common(src_k, src_v, dst_k, dst_v, bs * n_kv_heads, row_bytes);
  if (rc) return rc;
  PKV_REQUIRE(idx_packed && cu_topk && cu_k && max_k > 0 && total_k > 0 && src_len > 0 && sink_local_end >= 0,
              "packed gather: bad arguments");
  const void *dk = src_k, *dv = src_v;
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, src_k) == hipSuccess && attr.type == hipMemoryTypeHost) {
    rc = device_view_of_host(src_k, &dk);
    if (rc) return rc;
    rc = device_view_of_host(src_v, &dv);
    if (rc) return rc;
  } else {
    (void)hipGetLastError();
  }
  const int vpr = row_bytes / 16;
  const int64_t lanes = max_k * 2 * vpr;
  dim3 grid((unsigned)((lanes + kGatherThreads - 1) / kGatherThreads), (unsigned)(bs * n_kv_heads));
  hipLaunchKernelGGL(pkv_gather_packed_kernel, grid, dim3(kGatherThreads), 0, (hipStream_t)stream,
                     (const pkv_u32x4 *)dk, (const pkv_u32x4 *)dv, src_len, idx_packed, cu_topk, cu_k, sink_local_end,
                     (pkv_u32x4 *)dst_k, (pkv_u32x4 *)dst_v, total_k, vpr);
  PKV_LAUNCH_CHECK("pkv_gather_packed_kernel");
  return PKV_OK;
}

extern "C" int pkv_read_bytes(const void *src, size_t bytes, void *sink256, void *stream) {
  PKV_REQUIRE(src && sink256 && bytes % 16 == 0 && pkv_aligned(src, 16) && pkv_aligned(sink256, 4),
              "pkv_read_bytes: 16-byte aligned buffer and size, 256-byte sink required");
  if (bytes == 0) return PKV_OK;
  const int64_t n = (int64_t)(bytes / 16);
  const int64_t blocks = (n + 4095) / 4096;
  PKV_REQUIRE(blocks < ((int64_t)1 << 31), "pkv_read_bytes: too large");
  hipLaunchKernelGGL(pkv_read_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const pkv_u32x4 *)src, (uint32_t *)sink256, n);
  PKV_LAUNCH_CHECK("pkv_read_kernel");
  return PKV_OK;
}

extern "C" int pkv_copy_bytes(const void *src, void *dst, size_t bytes, void *stream) {
  PKV_REQUIRE(src && dst && bytes % 16 == 0 && pkv_aligned(src, 16) && pkv_aligned(dst, 16),
              "pkv_copy_bytes: 16-byte aligned buffers and size required");
  if (bytes == 0) return PKV_OK;
  const int64_t n = (int64_t)(bytes / 16);
  int64_t blocks = (n + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  hipLaunchKernelGGL(pkv_copy_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const pkv_u32x4 *)src, (pkv_u32x4 *)dst, n);
  PKV_LAUNCH_CHECK("pkv_copy_kernel");
  return PKV_OK;
}
