// Collision vote: cnt[key] = sum over the 16 subspaces of lut[subspace][code].
//
// Reference: cache_hub/collision_fused/collision.cu:163-229
// (update_cache_cnt_kernel: 16 byte loads at stride kv_len and 6 LDS bit tests
// per subspace).  Here the six tier bitsets are one 4 KB byte table per row held
// in LDS, a key's 16 codes are one 128-bit load (key-major storage), and the
// same pass also builds the per-chunk histogram that the candidate select needs,
// so the counts are never re-read to find the threshold.
//
// HBM-bound: 16 B read + 1 B written per key.
#include "pkv_common.h"

namespace {

constexpr int kScanThreads = 256;
constexpr int kHistCopies = 16;  // replicated LDS histogram: copy = lane & 15

__device__ __forceinline__ int lut_sum16(const uint8_t *__restrict__ l8, pkv_u32x4 v) {
  int c = 0;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int d = 0; d < 4; ++d) {
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint32_t code = (w[d] >> (8 * k)) & 0xffu;
      c += l8[(4 * d + k) * 256 + code];
    }
  }
  return c;
}

__device__ __forceinline__ void load_lut(uint32_t *s_lut, const uint8_t *__restrict__ lut, int row) {
  // 4 KB = one 128-bit load per thread
  const pkv_u32x4 *g = (const pkv_u32x4 *)(lut + (int64_t)row * 4096);
  ((pkv_u32x4 *)s_lut)[threadIdx.x] = g[threadIdx.x];
}

// KPT * 256 whole keys from key k0 on, in the form the retrieval runs (one-byte counts out, histogram kept): every
// load of the thread is issued before the first table lookup, and nothing in between is conditional, so the waits
// of the in-order memory counter name exact counts and the lookups of one key run while the codes of the others are
// still on their way.  Four keys per thread in flight, as in the general loop: with 8 or 16 the launch is slower at
// a full grid (config 3: 36.8 us per step with 4, 38.0 with 8, 40.1 with 16; 37.2 with the general loop), faster
// only where the grid leaves most of the chip idle.
template <int KPT>
__device__ __forceinline__ void scan_whole_keys(const pkv_u32x4 *__restrict__ base, int64_t k0, const uint8_t *l8,
                                                uint8_t *__restrict__ out8, uint32_t *s_hist, int copy) {
  const int64_t i0 = k0 + threadIdx.x;
  pkv_u32x4 v[KPT];
#pragma unroll
  for (int u = 0; u < KPT; ++u) v[u] = __builtin_nontemporal_load(base + i0 + u * kScanThreads);
#pragma unroll
  for (int u = 0; u < KPT; ++u) {
    const int c = lut_sum16(l8, v[u]);
    out8[i0 + u * kScanThreads] = (uint8_t)c;
    atomicAdd(&s_hist[c * kHistCopies + copy], 1u);
  }
}

// Key-major codes ([key][16] bytes, 16-byte aligned).  grid (n_chunks, R).
// sub_blocks = 1: workgroup c scans keys [c * chunk_keys, +chunk_keys) and leaves one suffix histogram.
// sub_blocks = S > 1: the chunk is S pieces of chunk_keys / S keys spread over the row, workgroup c scans pieces
// c, c + n_chunks, c + 2 n_chunks, ... (numbered in key order) and leaves one suffix histogram per piece, in the
// bin-major table chunk_suf[row][bin][chunk][piece of the chunk] (S = 4): the candidate select that follows works on the same pieces, so that where candidates
// bunch along the row (keys whose mean drifts) every workgroup gets a share of the crowded and of the sparse parts.
__global__ __launch_bounds__(kScanThreads) void pkv_scan_keymajor_kernel(
    const uint8_t *__restrict__ codes, int64_t cs_b, int64_t cs_h, int n_kv_heads, int64_t n_keys,
    const uint8_t *__restrict__ lut, uint8_t *__restrict__ cnt_u8, int64_t cnt_u8_stride,
    int32_t *__restrict__ cnt_i32, uint32_t *__restrict__ row_suf, uint16_t *__restrict__ chunk_suf, int chunk_keys,
    int sub_blocks) {
  const int row = blockIdx.y;
  const int chunk = blockIdx.x;
  const int n_chunks = gridDim.x;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  const int tid = threadIdx.x;

  __shared__ __attribute__((aligned(16))) uint32_t s_lut[1024];
  __shared__ uint32_t s_hist[128 * kHistCopies];  // also reused for the compacted histogram
  load_lut(s_lut, lut, row);
  for (int i = tid; i < 128 * kHistCopies; i += kScanThreads) s_hist[i] = 0;
  __syncthreads();
  const uint8_t *l8 = (const uint8_t *)s_lut;
  const int copy = tid & (kHistCopies - 1);

  const pkv_u32x4 *base = (const pkv_u32x4 *)(codes + (int64_t)b * cs_b + (int64_t)h * cs_h);
  uint8_t *out8 = cnt_u8 ? cnt_u8 + (int64_t)row * cnt_u8_stride : nullptr;
  int32_t *out32 = cnt_i32 ? cnt_i32 + (int64_t)row * n_keys : nullptr;
  const int piece_keys = chunk_keys / sub_blocks;
  uint64_t piece_bins = 0;  // sub_blocks == 4: this thread's bin of the four pieces' suffix histograms, 16 bits each
  uint32_t bin_total = 0;

  for (int j = 0; j < sub_blocks; ++j) {
    const int64_t piece = (int64_t)chunk + (int64_t)j * n_chunks;
    const int64_t k0 = piece * piece_keys < n_keys ? piece * piece_keys : n_keys;
    const int64_t k1 = (k0 + piece_keys < n_keys) ? k0 + piece_keys : n_keys;
    int64_t kc = k0;
    if (out8 && !out32 && chunk_suf) {  // uniform: the retrieval's form; whole runs of 1024 keys first
      for (; kc + 4 * kScanThreads <= k1; kc += 4 * kScanThreads) scan_whole_keys<4>(base, kc, l8, out8, s_hist, copy);
    }
    for (int64_t i0 = kc + tid; i0 < k1; i0 += 4 * kScanThreads) {
      pkv_u32x4 v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t i = i0 + u * kScanThreads;
        v[u] = (i < k1) ? __builtin_nontemporal_load(base + i) : pkv_u32x4{0u, 0u, 0u, 0u};
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t i = i0 + u * kScanThreads;
        if (i < k1) {
          const int c = lut_sum16(l8, v[u]);
          if (out8) out8[i] = (uint8_t)c;
          if (out32) out32[i] = c;
          if (chunk_suf) atomicAdd(&s_hist[c * kHistCopies + copy], 1u);
        }
      }
    }
    if (chunk_suf) {
      __syncthreads();
      uint32_t sum = 0;
      if (tid < 128) {
#pragma unroll
        for (int c = 0; c < kHistCopies; ++c) sum += s_hist[tid * kHistCopies + c];
      }
      __syncthreads();
      if (tid < 128) s_hist[tid] = sum;  // compacted histogram in the first 128 words
      __syncthreads();
      if (sub_blocks == 1) {
        pkv_store_suffix_hist(s_hist, &s_hist[128], row_suf + (int64_t)row * 128,
                              chunk_suf + ((int64_t)row * n_chunks + chunk) * 128);
      } else {
        // suffix sums of this piece; thread t owns bin 127 - t and keeps its pieces' values until the last one
        int incl = 0;
        if (tid < 128) {
          incl = pkv_wave_incl_scan((int)s_hist[127 - tid]);
          if (tid == PKV_WAVE - 1) s_hist[128] = (uint32_t)incl;
        }
        __syncthreads();
        if (tid < 128) {
          if (tid >= PKV_WAVE) incl += (int)s_hist[128];
          piece_bins |= (uint64_t)(uint32_t)incl << (16 * j);
          bin_total += (uint32_t)incl;
        }
      }
      if (j + 1 < sub_blocks) {  // the next piece starts from an empty histogram
        __syncthreads();
        for (int i = tid; i < 128 * kHistCopies; i += kScanThreads) s_hist[i] = 0;
        __syncthreads();
      }
    }
  }
  // several pieces: the bin-major table [row][bin][chunk][piece of the chunk] takes the chunk's four values of a bin
  // as one 8-byte store, and the row totals one addition per bin
  if (chunk_suf && sub_blocks > 1 && tid < 128) {
    uint16_t *dst = chunk_suf + ((int64_t)row * 128 + (127 - tid)) * n_chunks * sub_blocks + (int64_t)chunk * sub_blocks;
    *(uint64_t *)dst = piece_bins;
    if (bin_total) atomicAdd(&row_suf[(int64_t)row * 128 + 127 - tid], bin_total);
  }
}

// Any byte strides (e.g. the reference's subspace-major [16][kv_len] tensor).
__global__ __launch_bounds__(kScanThreads) void pkv_scan_strided_kernel(
    const uint8_t *__restrict__ codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub, int n_kv_heads,
    int64_t n_keys, const uint8_t *__restrict__ lut, uint8_t *__restrict__ cnt_u8, int64_t cnt_u8_stride,
    int32_t *__restrict__ cnt_i32, uint32_t *__restrict__ row_suf, uint16_t *__restrict__ chunk_suf, int chunk_keys) {
  const int row = blockIdx.y;
  const int chunk = blockIdx.x;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  const int tid = threadIdx.x;

  __shared__ __attribute__((aligned(16))) uint32_t s_lut[1024];
  __shared__ uint32_t s_hist[128 * kHistCopies];  // also reused for the compacted histogram
  load_lut(s_lut, lut, row);
  for (int i = tid; i < 128 * kHistCopies; i += kScanThreads) s_hist[i] = 0;
  __syncthreads();
  const uint8_t *l8 = (const uint8_t *)s_lut;
  const int copy = tid & (kHistCopies - 1);

  const uint8_t *base = codes + (int64_t)b * cs_b + (int64_t)h * cs_h;
  const int64_t k0 = (int64_t)chunk * chunk_keys;
  const int64_t k1 = (k0 + chunk_keys < n_keys) ? k0 + chunk_keys : n_keys;
  uint8_t *out8 = cnt_u8 ? cnt_u8 + (int64_t)row * cnt_u8_stride : nullptr;
  int32_t *out32 = cnt_i32 ? cnt_i32 + (int64_t)row * n_keys : nullptr;

  for (int64_t i = k0 + tid; i < k1; i += kScanThreads) {
    int c = 0;
#pragma unroll
    for (int s = 0; s < 16; ++s) c += l8[s * 256 + base[i * cs_key + s * cs_sub]];
    if (out8) out8[i] = (uint8_t)c;
    if (out32) out32[i] = c;
    if (chunk_suf) atomicAdd(&s_hist[c * kHistCopies + copy], 1u);
  }
  if (chunk_suf) {
    __syncthreads();
    uint32_t sum = 0;
    if (tid < 128) {
#pragma unroll
      for (int c = 0; c < kHistCopies; ++c) sum += s_hist[tid * kHistCopies + c];
    }
    __syncthreads();
    if (tid < 128) s_hist[tid] = sum;  // compacted histogram in the first 128 words
    __syncthreads();
    pkv_store_suffix_hist(s_hist, &s_hist[128], row_suf + (int64_t)row * 128,
                          chunk_suf + ((int64_t)row * gridDim.x + chunk) * 128);
  }
}

// Legacy int32 codebook [rows][16][n_keys]; codes outside [0,255] get no vote.
__global__ __launch_bounds__(kScanThreads) void pkv_scan_i32_codes_kernel(const int32_t *__restrict__ codebook,
                                                                          int64_t n_keys,
                                                                          const uint8_t *__restrict__ lut,
                                                                          int32_t *__restrict__ cnt) {
  const int row = blockIdx.y;
  __shared__ __attribute__((aligned(16))) uint32_t s_lut[1024];
  load_lut(s_lut, lut, row);
  __syncthreads();
  const uint8_t *l8 = (const uint8_t *)s_lut;
  const int64_t i = (int64_t)blockIdx.x * kScanThreads + threadIdx.x;
  if (i >= n_keys) return;
  const int32_t *base = codebook + (int64_t)row * 16 * n_keys;
  int c = 0;
#pragma unroll
  for (int s = 0; s < 16; ++s) {
    const int32_t code = base[(int64_t)s * n_keys + i];
    if ((uint32_t)code < 256u) c += l8[s * 256 + code];
  }
  cnt[(int64_t)row * n_keys + i] = c;
}

}  // namespace

static int launch_scan_impl(const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub, int bs,
                            int n_kv_heads, int64_t n_keys, const uint8_t *lut, uint8_t *cnt_u8,
                            int64_t cnt_u8_stride, int32_t *cnt_i32, uint32_t *row_suf, uint16_t *chunk_suf,
                            int chunk_keys, hipStream_t s, hipEvent_t ev_start, hipEvent_t ev_stop, int sub_blocks = 1) {
  PKV_REQUIRE(chunk_keys >= 2048 && chunk_keys % 2048 == 0 && chunk_keys <= 32768,
              "chunk_keys must be a multiple of 2048 in [2048,32768], got %d", chunk_keys);
  const int64_t n_chunks = (n_keys + chunk_keys - 1) / chunk_keys;
  PKV_REQUIRE(n_chunks >= 1 && n_chunks <= 65535 * 16, "too many chunks (%lld)", (long long)n_chunks);
  PKV_REQUIRE(pkv_aligned(lut, 4), "lut must be 4-byte aligned");
  dim3 grid((unsigned)n_chunks, (unsigned)(bs * n_kv_heads));
  const bool keymajor = cs_sub == 1 && cs_key == 16 && pkv_aligned(codes, 16) && cs_b % 16 == 0 && cs_h % 16 == 0;
  PKV_REQUIRE((sub_blocks == 1 || (sub_blocks == 4 && keymajor && chunk_suf)) && chunk_keys % (sub_blocks * 1024) == 0,
              "a chunk of %d keys cannot be scanned as %d strided pieces", chunk_keys, sub_blocks);
  if (keymajor) {
    // the ext launch ties the two events to this dispatch's own begin/end timestamps
    hipExtLaunchKernelGGL(pkv_scan_keymajor_kernel, grid, dim3(kScanThreads), 0, s, ev_start, ev_stop, 0, codes, cs_b,
                          cs_h, n_kv_heads, n_keys, lut, cnt_u8, cnt_u8_stride, cnt_i32, row_suf, chunk_suf, chunk_keys,
                          sub_blocks);
    PKV_LAUNCH_CHECK("pkv_scan_keymajor_kernel");
  } else {
    hipExtLaunchKernelGGL(pkv_scan_strided_kernel, grid, dim3(kScanThreads), 0, s, ev_start, ev_stop, 0, codes, cs_b,
                          cs_h, cs_key, cs_sub, n_kv_heads, n_keys, lut, cnt_u8, cnt_u8_stride, cnt_i32, row_suf,
                          chunk_suf, chunk_keys);
    PKV_LAUNCH_CHECK("pkv_scan_strided_kernel");
  }
  return PKV_OK;
}

int pkv_launch_scan(const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub, int bs,
                    int n_kv_heads, int64_t n_keys, const uint8_t *lut, uint8_t *cnt_u8, int64_t cnt_u8_stride,
                    int32_t *cnt_i32, uint32_t *row_suf, uint16_t *chunk_suf, int chunk_keys, hipStream_t s, int sub_blocks) {
  return launch_scan_impl(codes, cs_b, cs_h, cs_key, cs_sub, bs, n_kv_heads, n_keys, lut, cnt_u8, cnt_u8_stride, cnt_i32,
                          row_suf, chunk_suf, chunk_keys, s, nullptr, nullptr, sub_blocks);
}

int pkv_launch_scan_i32_codes(const int32_t *codebook, int rows, int64_t n_keys, const uint8_t *lut, int32_t *cnt,
                              hipStream_t s) {
  dim3 grid((unsigned)((n_keys + kScanThreads - 1) / kScanThreads), (unsigned)rows);
  hipLaunchKernelGGL(pkv_scan_i32_codes_kernel, grid, dim3(kScanThreads), 0, s, codebook, n_keys, lut, cnt);
  PKV_LAUNCH_CHECK("pkv_scan_i32_codes_kernel");
  return PKV_OK;
}

extern "C" int pkv_collision_scan(const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key, int64_t cs_sub,
                                  int bs, int n_kv_heads, int64_t n_keys, const uint8_t *lut, uint8_t *cnt_u8,
                                  int32_t *cnt_i32, uint32_t *row_suf, uint16_t *chunk_suf, int chunk_keys,
                                  void *stream) {
  PKV_REQUIRE(codes && lut && (cnt_u8 || cnt_i32), "pkv_collision_scan: null pointer");
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && (int64_t)bs * n_kv_heads <= 65535 && n_keys > 0 &&
                  n_keys <= PKV_MAX_KEYS_PER_ROW,
              "bad shape bs=%d kv_heads=%d n_keys=%lld", bs, n_kv_heads, (long long)n_keys);
  PKV_REQUIRE((row_suf == nullptr) == (chunk_suf == nullptr), "row_suf and chunk_suf go together");
  return pkv_launch_scan(codes, cs_b, cs_h, cs_key, cs_sub, bs, n_kv_heads, n_keys, lut, cnt_u8, n_keys, cnt_i32,
                         row_suf, chunk_suf, chunk_keys, (hipStream_t)stream);
}

extern "C" int pkv_collision_scan_timed(const uint8_t *codes, int64_t cs_b, int64_t cs_h, int64_t cs_key,
                                        int64_t cs_sub, int bs, int n_kv_heads, int64_t n_keys, const uint8_t *lut,
                                        uint8_t *cnt_u8, int64_t cnt_u8_stride, uint32_t *row_suf, uint16_t *chunk_suf,
                                        int chunk_keys, float *kernel_us, void *stream) {
  PKV_REQUIRE(codes && lut && cnt_u8 && kernel_us, "pkv_collision_scan_timed: null pointer");
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && (int64_t)bs * n_kv_heads <= 65535 && n_keys > 0 &&
                  n_keys <= PKV_MAX_KEYS_PER_ROW && cnt_u8_stride >= n_keys,
              "bad shape bs=%d kv_heads=%d n_keys=%lld", bs, n_kv_heads, (long long)n_keys);
  hipEvent_t e0, e1;
  PKV_HIP(hipEventCreate(&e0));
  PKV_HIP(hipEventCreate(&e1));
  int rc = launch_scan_impl(codes, cs_b, cs_h, cs_key, cs_sub, bs, n_kv_heads, n_keys, lut, cnt_u8, cnt_u8_stride,
                            nullptr, row_suf, chunk_suf, chunk_keys, (hipStream_t)stream, e0, e1);
  if (rc == PKV_OK) {
    float ms = 0.f;
    hipError_t e = hipEventSynchronize(e1);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
    if (e != hipSuccess) {
      pkv_set_error("event timing failed: %s", hipGetErrorString(e));
      rc = PKV_EHIP;
    }
    *kernel_us = ms * 1000.f;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return rc;
}
