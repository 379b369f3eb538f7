// One launch for the first three stages of a layer's retrieval: query prep + vote table, collision scan with
// chunk histograms, candidate select fused with the 4-bit rerank.  The stages depend on each other through whole
// rows (a row's vote table before its scan, a row's histogram before its select), which the separate kernels
// express as launch boundaries; here they are hand-overs between the workgroups of one launch.
//
// Reference: cache_hub/polar_cache.py:1027-1031, 1207-1231 (query prep, collision vote), :1237-1242 (candidate
// select), :1244-1298 (rerank); kernels cache_hub/collision_fused/collision.cu:71-229, topk/radix_topk.cu:39-120,
// rerank/rerank.cu:51-138.  The reference runs them as separate launches (plus torch glue between them).
//
// grid (n_chunks, rows) x 256 threads; workgroup (chunk, row) owns keys [chunk * chunk_keys, +chunk_keys) of the row.
//   1. every workgroup requests its first codes, and rotates the row's query (one wave);
//   2. workgroup `chunk` < 16 ranks the centroids of subspace `chunk` and writes that 256-byte slice of the row's
//      vote table (subspaces chunk, chunk + n_chunks, ... when the row has fewer than 16 chunks), then raises
//      table_flags[row][subspace]; workgroup 0 clears the row's suffix totals before it does;
//   3. every workgroup waits for the row's 16 table flags, loads the 4 KB table, scans its chunk: vote counts into
//      LDS (and into the caller's array when it wants them), chunk histogram, suffix histogram out, row totals added;
//   4. it raises chunk_flags[row][chunk] and waits for the row's other chunks; then threshold and output offsets
//      follow from the suffix histograms, and the chunk's candidates are picked from the counts in LDS and scored.
// Flags hold the launch's epoch (a number no earlier launch used), so they never need clearing.  A workgroup only
// waits for workgroups of its own row: in step 3 for lower-numbered ones, which were dispatched before it; in step
// 4 for all of them, which are resident or next in the dispatch order as long as one row's chunks fit the chip.
// Every wait is bounded by the wall clock; a workgroup that gives up counts itself in `status[0]` and goes on (its
// results are then wrong: the host rejects shapes where that could happen and callers can read the status word).
#include "pkv_common.h"
#include "pkv_lut.h"
#include "pkv_selcore.h"

#include <atomic>
#include <chrono>

namespace {

constexpr int kFusedThreads = 256;
constexpr int kFusedHistCopies = 16;
constexpr int kFusedMaxChunkKeys = 8192;  // vote counts of one chunk held in LDS

struct FusedArgs {
  // query side
  const void *q;
  int dtype, n_kv_heads, group;
  const float *signs;
  const int32_t *cc;
  int64_t cc_b, cc_h;
  PkvTiers tiers;
  float *qhat, *qnorm;
  uint8_t *lut;
  // scan
  const uint8_t *codes;
  int64_t cs_b, cs_h, n_keys;
  int chunk_keys;
  uint8_t *cnt_u8;  // null: the counts stay in LDS
  int64_t cnt_stride;
  uint32_t *row_suf;
  uint16_t *chunk_suf;
  // hand-overs
  uint64_t *table_flags;  // [rows][16]
  uint64_t *chunk_flags;  // [rows][n_chunks]
  uint32_t *status;
  uint64_t epoch, wait_ticks;
  uint32_t *zero_ptr;  // per row: zero_row_words words at zero_ptr + row * zero_row_stride (control block of a wide top-k)
  int64_t zero_row_words, zero_row_stride;
  // select + rerank
  int64_t k;
  const uint8_t *nib;
  int64_t ns_b, ns_h;
  int ns_key;
  const uint16_t *weight;
  int64_t ws_b, ws_h;
  int ws_key;
  const float *centers;
  int64_t *out;
  float *scores;
  int extra_off;
  float *extra_out;
  uint32_t *range_slots;
  int64_t range_row_stride;
};

struct FusedSmem {
  __attribute__((aligned(16))) uint32_t lut[1024];               // the row's vote table
  __attribute__((aligned(16))) uint8_t cnt[kFusedMaxChunkKeys];  // vote counts of this chunk
  float prod[128 * 16];                                           // rerank product table
  union {
    PkvLutSmem table;                            // step 2
    uint32_t hist[128 * kFusedHistCopies];       // step 3
    uint16_t list_key[kSelKeysPerIter];          // step 4
  } u;
  float y[128];
  float qn;
  int scan[2][kFusedThreads / PKV_WAVE];
  uint32_t ok;
};

__device__ __forceinline__ int fused_lut_sum16(const uint8_t *__restrict__ l8, pkv_u32x4 v) {
  int c = 0;
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int d = 0; d < 4; ++d) {
#pragma unroll
    for (int k = 0; k < 4; ++k) c += l8[(4 * d + k) * 256 + ((w[d] >> (8 * k)) & 0xffu)];
  }
  return c;
}

__global__ __launch_bounds__(kFusedThreads) void pkv_fused_retrieve_kernel(const FusedArgs A) {
  const int row = blockIdx.y, chunk = blockIdx.x, n_chunks = gridDim.x, tid = threadIdx.x;
  const int b = row / A.n_kv_heads, h = row % A.n_kv_heads;
  __shared__ FusedSmem sm;
  if (row == 0 && chunk == 0 && tid == 0) pkv_st_agent_u32(A.status, 0u);  // the word counts this launch's failures

  // ---- 1. the row's rotated query; first codes in flight.  A compute unit returns its loads in the order they
  // were requested, so the workgroups that build the table ask for the query first and for their codes only once
  // their slice is out; the others have nothing to wait for and ask for their codes at once.
  const pkv_u32x4 *base = (const pkv_u32x4 *)(A.codes + (int64_t)b * A.cs_b + (int64_t)h * A.cs_h);
  const int64_t k0 = (int64_t)chunk * A.chunk_keys;
  const int64_t k1 = (k0 + A.chunk_keys < A.n_keys) ? k0 + A.chunk_keys : A.n_keys;
  const pkv_u32x4 zero4 = {0u, 0u, 0u, 0u};
  pkv_u32x4 v[4];
  const bool table_wg = chunk < 16;
  int my_cc = 0;
  if (table_wg) my_cc = A.cc[(int64_t)b * A.cc_b + (int64_t)h * A.cc_h + chunk * 256 + tid];
  else {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t i = k0 + tid + u * kFusedThreads;
      v[u] = (i < k1) ? __builtin_nontemporal_load(base + i) : zero4;
    }
  }
  if (tid < PKV_WAVE) {
    float y_lo, y_hi;
    const float n = pkv_query_mean_rotate_wave(A.q, A.dtype, b, h, A.n_kv_heads, A.group, A.signs, y_lo, y_hi);
    sm.y[tid] = y_lo, sm.y[tid + 64] = y_hi;
    sm.u.table.y[tid] = y_lo, sm.u.table.y[tid + 64] = y_hi;
    if (tid == 0) sm.qn = n;
    if (chunk == 0) {  // for later launches and for callers that look at the intermediates
      A.qhat[(int64_t)row * 128 + tid] = y_lo, A.qhat[(int64_t)row * 128 + tid + 64] = y_hi;
      if (tid == 0) A.qnorm[row] = n;
    }
  }
  // ---- 2. this workgroup's slices of the vote table
  if (table_wg) {
    if (chunk == 0 && tid < 128) pkv_st_agent_u32(A.row_suf + (int64_t)row * 128 + tid, 0u);
    // the row's control words of a multi-workgroup top-k, which the select below and later launches add to
    for (int64_t i = (int64_t)chunk * kFusedThreads + tid; i < A.zero_row_words; i += (int64_t)(n_chunks < 16 ? n_chunks : 16) * kFusedThreads)
      pkv_st_agent_u32(A.zero_ptr + (int64_t)row * A.zero_row_stride + i, 0u);
    sm.u.table.cc[tid] = my_cc;
    __syncthreads();
    for (int sub = chunk; sub < 16; sub += n_chunks) {
      uint8_t *part = (uint8_t *)sm.lut;  // staged in LDS, then written through as 64 words
      pkv_lut_rank_subspace(A.dtype,
                            sub == chunk ? nullptr : A.cc + (int64_t)b * A.cc_b + (int64_t)h * A.cc_h + sub * 256,
                            A.tiers, sub, sm.u.table, part, nullptr);
      __syncthreads();
      if (tid < 64) pkv_st_agent_u32(A.lut + ((int64_t)row * 16 + sub) * 256 + 4 * tid, sm.lut[tid]);
      pkv_wait_vmem();
      __syncthreads();
      if (tid == 0) pkv_st_agent_u64(A.table_flags + (int64_t)row * 16 + sub, A.epoch);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t i = k0 + tid + u * kFusedThreads;
      v[u] = (i < k1) ? __builtin_nontemporal_load(base + i) : zero4;
    }
  } else {
    __syncthreads();  // sm.y
  }
  // rerank product table, while the table flags travel
  pkv_build_prod_table<kFusedThreads>(sm.prod, sm.y, A.centers);

  // ---- 3. wait for the row's table, scan the chunk
  if (tid < PKV_WAVE) {
    const bool ok = pkv_wait_flags(A.table_flags + (int64_t)row * 16, 16, A.epoch, A.wait_ticks);
    if (tid == 0) {
      sm.ok = ok ? 1u : 0u;
      if (!ok) atomicAdd(A.status, 1u);
    }
  }
  __syncthreads();
  {
    ((pkv_u32x4 *)sm.lut)[tid] = pkv_ld_agent_x4(A.lut + (int64_t)row * 4096 + 16 * tid);
  }
  for (int i = tid; i < 128 * kFusedHistCopies; i += kFusedThreads) sm.u.hist[i] = 0;
  __syncthreads();
  {
    const uint8_t *l8 = (const uint8_t *)sm.lut;
    const int copy = tid & (kFusedHistCopies - 1);
    uint8_t *out8 = A.cnt_u8 ? A.cnt_u8 + (int64_t)row * A.cnt_stride : nullptr;
    for (int64_t i0 = k0 + tid; i0 < k1; i0 += 4 * kFusedThreads) {
      if (i0 != k0 + tid) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int64_t i = i0 + u * kFusedThreads;
          v[u] = (i < k1) ? __builtin_nontemporal_load(base + i) : zero4;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int64_t i = i0 + u * kFusedThreads;
        if (i < k1) {
          const int c = fused_lut_sum16(l8, v[u]);
          sm.cnt[i - k0] = (uint8_t)c;
          if (out8) out8[i] = (uint8_t)c;
          atomicAdd(&sm.u.hist[c * kFusedHistCopies + copy], 1u);
        }
      }
    }
  }
  __syncthreads();
  {
    uint32_t sum = 0;
    if (tid < 128) {
#pragma unroll
      for (int c = 0; c < kFusedHistCopies; ++c) sum += sm.u.hist[tid * kFusedHistCopies + c];
    }
    __syncthreads();
    if (tid < 128) sm.u.hist[tid] = sum;
    __syncthreads();
    // suffix sums: thread t owns bin 127 - t
    int incl = 0;
    if (tid < 128) {
      incl = pkv_wave_incl_scan((int)sm.u.hist[127 - tid]);
      if (tid == PKV_WAVE - 1) sm.u.hist[128] = (uint32_t)incl;
    }
    __syncthreads();
    if (tid < 128) {
      if (tid >= PKV_WAVE) incl += (int)sm.u.hist[128];
      pkv_st_agent_u16(A.chunk_suf + ((int64_t)row * n_chunks + chunk) * 128 + (127 - tid), (uint32_t)incl);
      if (incl) atomicAdd(&A.row_suf[(int64_t)row * 128 + 127 - tid], (uint32_t)incl);
    }
  }
  // ---- 4. the row's histogram is complete when every chunk has raised its flag
  pkv_wait_vmem();
  __syncthreads();
  if (tid == 0) pkv_st_agent_u64(A.chunk_flags + (int64_t)row * n_chunks + chunk, A.epoch);
  if (tid < PKV_WAVE) {
    bool ok = true;
    for (int c0 = 0; c0 < n_chunks && ok; c0 += PKV_WAVE)
      ok = pkv_wait_flags(A.chunk_flags + (int64_t)row * n_chunks + c0, n_chunks - c0 < PKV_WAVE ? n_chunks - c0 : PKV_WAVE,
                          A.epoch, A.wait_ticks);
    if (tid == 0 && !ok) atomicAdd(A.status, 1u);
  }
  __syncthreads();

  const uint32_t rs_mine = tid < 128 ? pkv_ld_agent_u32(A.row_suf + (int64_t)row * 128 + tid) : 0u;
  uint32_t theta;
  int64_t base_gt, base_eq;
  select_prologue<true>(rs_mine, A.chunk_suf, row, chunk, n_chunks, A.k, theta, base_gt, base_eq);
  const int64_t k = A.k;
  int64_t *orow = A.out + (int64_t)row * k;
  float *srow = A.scores + (int64_t)row * k;
  const uint8_t *nrow = A.nib + (int64_t)b * A.ns_b + (int64_t)h * A.ns_h;
  const uint16_t *wrow = A.weight + (int64_t)b * A.ws_b + (int64_t)h * A.ws_h;
  const float qn = sm.qn;
  uint32_t smax = 0u, smin = 0xffffffffu;

  int it = 0;
  for (int64_t blk0 = k0; blk0 < k1; blk0 += kSelKeysPerIter, ++it) {
    const int64_t i0 = blk0 + (int64_t)tid * kSelKeysPerThread;
    const pkv_u32x4 w = i0 < k1 ? *(const pkv_u32x4 *)(sm.cnt + (i0 - k0)) : zero4;
    uint32_t gt[4], eq[4];
    count_masks16(w, theta, k1 - i0, gt, eq);
    const int packed = popc4(gt) | (popc4(eq) << 16);
    int total;
    const int excl = pkv_block_excl_scan<kFusedThreads>(packed, sm.scan[it & 1], total);
    const int n_gt_it = total & 0xffff, n_sel_it = n_gt_it + (total >> 16);
    int lg = excl & 0xffff;
    int le = n_gt_it + (excl >> 16);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t g = gt[d], e = eq[d];
      while (g) {
        const int bit = __ffs((int)g) - 1;
        g &= g - 1;
        sm.u.list_key[lg++] = (uint16_t)(tid * kSelKeysPerThread + 4 * d + (bit >> 3));
      }
      while (e) {
        const int bit = __ffs((int)e) - 1;
        e &= e - 1;
        sm.u.list_key[le++] = (uint16_t)(tid * kSelKeysPerThread + 4 * d + (bit >> 3));
      }
    }
    const int64_t pos_gt0 = base_gt, pos_eq0 = base_eq - n_gt_it, eq_room = k - base_eq;
    const int n_use = eq_room >= (total >> 16) ? n_sel_it : n_gt_it + (int)(eq_room > 0 ? eq_room : 0);
    base_gt += n_gt_it;
    base_eq += total >> 16;
    __syncthreads();
#pragma unroll 1
    for (int j = tid; j < n_use; j += kFusedThreads) {
      const int64_t pos = j < n_gt_it ? pos_gt0 + j : pos_eq0 + j;
      const int64_t key = blk0 + sm.u.list_key[j];
      orow[pos] = key;
      const float sc = pkv_rerank_keymajor(sm.prod, (const pkv_u32x4 *)(nrow + key * A.ns_key),
                                           (const pkv_u32x4 *)(wrow + key * A.ws_key), qn);
      srow[pos] = sc;
      const uint32_t o = pkv_ordered_u32(sc);
      smax = o > smax ? o : smax;
      smin = o < smin ? o : smin;
      if (A.extra_out) A.extra_out[(int64_t)row * k + pos] = *(const float *)(nrow + key * A.ns_key + A.extra_off);
    }
    __syncthreads();
  }
  if (A.range_slots) {
#pragma unroll
    for (int x = 1; x < PKV_WAVE; x <<= 1) {
      const uint32_t a = (uint32_t)__shfl_xor((int)smax, x, PKV_WAVE), c = (uint32_t)__shfl_xor((int)smin, x, PKV_WAVE);
      smax = a > smax ? a : smax;
      smin = c < smin ? c : smin;
    }
    if (pkv_lane() == 0) sm.scan[0][tid / PKV_WAVE] = (int)smax, sm.scan[1][tid / PKV_WAVE] = (int)smin;
    __syncthreads();
    if (tid == 0) {
      for (int wv = 1; wv < kFusedThreads / PKV_WAVE; ++wv) {
        const uint32_t a = (uint32_t)sm.scan[0][wv], c = (uint32_t)sm.scan[1][wv];
        smax = a > smax ? a : smax;
        smin = c < smin ? c : smin;
      }
      if (smax >= smin) {
        uint32_t *slot = A.range_slots + (int64_t)row * A.range_row_stride + 2 * (chunk % 16);
        atomicMax(&slot[0], smax);
        atomicMax(&slot[1], ~smin);
      }
    }
  }
}

std::atomic<uint64_t> g_epoch{0};

// A number that no earlier launch of this process has used as its epoch, and that memory which never held a flag is
// unlikely to contain: a counter started from the clock.
uint64_t next_epoch() {
  uint64_t e = g_epoch.load(std::memory_order_relaxed);
  if (e == 0) {
    const uint64_t seed = ((uint64_t)std::chrono::steady_clock::now().time_since_epoch().count() << 20) ^ 0x9E3779B97F4A7C15ull;
    uint64_t expected = 0;
    g_epoch.compare_exchange_strong(expected, seed | 1ull);
  }
  return g_epoch.fetch_add(1, std::memory_order_relaxed) + 1;
}

}  // namespace

// Bytes of the hand-over area (flags + status word) of a fused launch.
size_t pkv_fused_sync_bytes(int rows, int64_t n_chunks) {
  return pkv_align_up((size_t)rows * 16 * 8, 256) + pkv_align_up((size_t)rows * (size_t)n_chunks * 8, 256) + 256;
}

// Whether the fused launch may be used for this shape on this stream: chunks whose counts fit LDS, a row's chunks
// well inside what the chip holds at once, and a stream that is not being captured (the epoch is a launch argument:
// a replayed graph would present the same epoch again).
bool pkv_fused_usable(int rows, int64_t n_keys, int chunk_keys, hipStream_t s) {
  const int64_t n_chunks = (n_keys + chunk_keys - 1) / chunk_keys;
  // at most 1024 workgroups: with four of them per compute unit the whole launch is resident at once on the
  // 256 compute units, so no wait depends on the order in which workgroups are dispatched
  if (chunk_keys > kFusedMaxChunkKeys || n_chunks > 256 || (int64_t)rows * n_chunks > 1024) return false;
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &st) != hipSuccess || st != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return false;
  }
  return true;
}

int pkv_launch_fused_retrieve(const void *q, int dtype, int bs, int n_kv_heads, int group, const float *signs,
                              const int32_t *cc, int64_t cc_b, int64_t cc_h, const PkvTiers &tiers, float *qhat,
                              float *qnorm, uint8_t *lut, const uint8_t *codes, int64_t cs_b, int64_t cs_h,
                              int64_t n_keys, int chunk_keys, uint8_t *cnt_u8, int64_t cnt_stride, uint32_t *row_suf,
                              uint16_t *chunk_suf, void *sync_area, uint32_t *zero_ptr, int64_t zero_row_words,
                              int64_t zero_row_stride, int64_t k, const uint8_t *nib, int64_t ns_b, int64_t ns_h,
                              int64_t ns_key, const uint16_t *weight, int64_t ws_b, int64_t ws_h, int64_t ws_key,
                              const float *centers, int64_t *cand, float *scores, int64_t extra_off, float *extra_out,
                              uint32_t *range_slots, int64_t range_row_stride, hipStream_t s) {
  const int rows = bs * n_kv_heads;
  const int64_t n_chunks = (n_keys + chunk_keys - 1) / chunk_keys;
  PKV_REQUIRE(chunk_keys >= 2048 && chunk_keys % 2048 == 0 && chunk_keys <= kFusedMaxChunkKeys && n_chunks <= 256,
              "fused retrieval: chunk of %d keys, %lld chunks per row not supported", chunk_keys, (long long)n_chunks);
  PKV_REQUIRE(!extra_out || (extra_off >= 0 && extra_off % 4 == 0 && extra_off + 4 <= ns_key),
              "the extra word must lie inside the key's record (offset %lld, record %lld bytes)", (long long)extra_off,
              (long long)ns_key);
  PKV_REQUIRE(k >= 1 && k < n_keys && k < ((int64_t)1 << 31), "select needs 1 <= k < n_keys (k=%lld n=%lld)", (long long)k,
              (long long)n_keys);
  PKV_REQUIRE(pkv_aligned(nib, 16) && pkv_aligned(weight, 16) && ns_b % 16 == 0 && ns_h % 16 == 0 && ws_b % 8 == 0 &&
                  ws_h % 8 == 0 && ns_key >= 64 && ns_key % 16 == 0 && ws_key >= 16 && ws_key % 8 == 0 &&
                  ns_key < (1 << 20) && ws_key < (1 << 20),
              "key-major nibbles / weights must be 16-byte aligned, 64 bytes / 16 weights per key");
  PKV_REQUIRE(pkv_aligned(codes, 16) && cs_b % 16 == 0 && cs_h % 16 == 0 && pkv_aligned(lut, 16) && pkv_aligned(sync_area, 256),
              "fused retrieval: codes / table / hand-over area misaligned");
  PKV_REQUIRE(!cnt_u8 || (cnt_stride % 16 == 0 && cnt_stride >= n_keys), "count rows must be padded to 16 bytes");
  FusedArgs A;
  memset(&A, 0, sizeof A);
  A.q = q, A.dtype = dtype, A.n_kv_heads = n_kv_heads, A.group = group, A.signs = signs;
  A.cc = cc, A.cc_b = cc_b, A.cc_h = cc_h, A.tiers = tiers, A.qhat = qhat, A.qnorm = qnorm, A.lut = lut;
  A.codes = codes, A.cs_b = cs_b, A.cs_h = cs_h, A.n_keys = n_keys, A.chunk_keys = chunk_keys;
  A.cnt_u8 = cnt_u8, A.cnt_stride = cnt_stride, A.row_suf = row_suf, A.chunk_suf = chunk_suf;
  char *sa = (char *)sync_area;
  A.table_flags = (uint64_t *)sa;
  A.chunk_flags = (uint64_t *)(sa + pkv_align_up((size_t)rows * 16 * 8, 256));
  A.status = (uint32_t *)(sa + pkv_align_up((size_t)rows * 16 * 8, 256) + pkv_align_up((size_t)rows * (size_t)n_chunks * 8, 256));
  A.epoch = next_epoch();
  A.wait_ticks = 200000000ull;  // 2 s of the 100 MHz clock
  A.zero_ptr = zero_ptr, A.zero_row_words = zero_ptr ? zero_row_words : 0, A.zero_row_stride = zero_row_stride;
  A.k = k, A.nib = nib, A.ns_b = ns_b, A.ns_h = ns_h, A.ns_key = (int)ns_key;
  A.weight = weight, A.ws_b = ws_b, A.ws_h = ws_h, A.ws_key = (int)ws_key, A.centers = centers;
  A.out = cand, A.scores = scores, A.extra_off = (int)extra_off, A.extra_out = extra_out;
  A.range_slots = range_slots, A.range_row_stride = range_row_stride;
  dim3 grid((unsigned)n_chunks, (unsigned)rows);
  hipLaunchKernelGGL(pkv_fused_retrieve_kernel, grid, dim3(kFusedThreads), 0, s, A);
  PKV_LAUNCH_CHECK("pkv_fused_retrieve_kernel");
  return PKV_OK;
}
