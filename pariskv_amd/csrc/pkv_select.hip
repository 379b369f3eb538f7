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
#include "pkv_selcore.h"

namespace {

constexpr int kWideRangeSlots = 16;  // per row: score ranges left by a producer's workgroups for a multi-workgroup top-k, (max, ~min) each

// grid (n_chunks, rows).  cnt rows are padded to a multiple of 16 bytes and 16-byte aligned, so every
// thread's 16 counts are one aligned 128-bit load (issued before the threshold is known).
__global__ __launch_bounds__(kSelThreads) void pkv_select_kernel(const uint8_t *__restrict__ cnt,
                                                                 int64_t cnt_stride,
                                                                 const uint32_t *__restrict__ row_suf,
                                                                 const uint16_t *__restrict__ chunk_suf,
                                                                 int chunk_keys, int64_t n_keys, int64_t k,
                                                                 int64_t *__restrict__ out) {
  const int row = blockIdx.y;
  const int chunk = blockIdx.x;
  const int tid = threadIdx.x;
  __shared__ int s_scan[2][kSelThreads / PKV_WAVE];
  const uint8_t *crow = cnt + (int64_t)row * cnt_stride;
  const int64_t chunk_begin = (int64_t)chunk * chunk_keys;
  const int64_t chunk_end = (chunk_begin + chunk_keys < n_keys) ? chunk_begin + chunk_keys : n_keys;
  const pkv_u32x4 zero4 = {0u, 0u, 0u, 0u};
  int64_t i0 = chunk_begin + (int64_t)tid * kSelKeysPerThread;
  pkv_u32x4 w = i0 < chunk_end ? *(const pkv_u32x4 *)(crow + i0) : zero4;  // padded rows: always in bounds
  uint32_t rs_mine = 0u;
  if (tid < 128) {
    if (row_suf) {
      rs_mine = row_suf[(int64_t)row * 128 + tid];
    } else {  // no row totals kept: add the chunks' suffix histograms up (a producer without atomics, nothing to clear)
      const uint16_t *cs = chunk_suf + (int64_t)row * gridDim.x * 128 + tid;
      for (int c = 0; c < (int)gridDim.x; ++c) rs_mine += cs[(int64_t)c * 128];
    }
  }

  uint32_t theta;
  int64_t base_gt, base_eq;
  select_prologue(rs_mine, chunk_suf, row, chunk, gridDim.x, k, theta, base_gt, base_eq);
  int64_t *orow = out + (int64_t)row * k;

  int it = 0;
  for (int64_t blk0 = chunk_begin; blk0 < chunk_end; blk0 += kSelKeysPerIter, ++it) {
    uint32_t gt[4], eq[4];
    count_masks16(w, theta, chunk_end - i0, gt, eq);
    const int64_t i_cur = i0;
    i0 += kSelKeysPerIter;
    if (blk0 + kSelKeysPerIter < chunk_end) w = i0 < chunk_end ? *(const pkv_u32x4 *)(crow + i0) : zero4;
    const int packed = popc4(gt) | (popc4(eq) << 16);
    int total;
    const int excl = pkv_block_excl_scan<kSelThreads>(packed, s_scan[it & 1], total);
    int64_t pg = base_gt + (excl & 0xffff);
    int64_t pe = base_eq + (excl >> 16);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t g = gt[d], e = eq[d];
      while (g) {
        const int bit = __ffs((int)g) - 1;
        g &= g - 1;
        if (pg < k) orow[pg] = i_cur + 4 * d + (bit >> 3);
        ++pg;
      }
      while (e) {
        const int bit = __ffs((int)e) - 1;
        e &= e - 1;
        if (pe < k) orow[pe] = i_cur + 4 * d + (bit >> 3);
        ++pe;
      }
    }
    base_gt += total & 0xffff;
    base_eq += total >> 16;
  }
}

// Candidate select fused with the 4-bit rerank (key-major storage): every workgroup finds the
// candidates of its chunk as above, parks them in LDS and scores them right away, so the candidate
// list is never re-read and one launch disappears from the decode step.
// out/scores: [rows][k]; position p of a row holds the candidate's key index and its score.
// extra_out (optional, [rows][k]): the fp32 word at byte extra_off of the candidate's record, e.g. the value
// norm the adaptive-k stage weighs it with.
__global__ __launch_bounds__(kSelThreads) void pkv_select_rerank_kernel(
    const uint8_t *__restrict__ cnt, int64_t cnt_stride, const uint32_t *__restrict__ row_suf,
    const uint16_t *__restrict__ chunk_suf, int chunk_keys, int n_kv_heads, int64_t n_keys, int64_t k,
    const uint8_t *__restrict__ nib, int64_t ns_b, int64_t ns_h, int ns_key, const uint16_t *__restrict__ weight,
    int64_t ws_b, int64_t ws_h, int ws_key, const float *__restrict__ qhat, const float *__restrict__ qnorm,
    const float *__restrict__ centers, int64_t *__restrict__ out, float *__restrict__ scores, int extra_off,
    float *__restrict__ extra_out, uint32_t *__restrict__ range_slots, int64_t range_row_stride) {
  const int row = blockIdx.y;
  const int chunk = blockIdx.x;
  const int tid = threadIdx.x;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  uint32_t smax = 0u, smin = 0xffffffffu;  // ordered bits of the largest / smallest score this thread wrote

  __shared__ int s_scan[2][kSelThreads / PKV_WAVE];
  __shared__ float s_prod[128 * 16];
  __shared__ uint16_t s_list_key[kSelKeysPerIter];  // offset of the key inside the iteration's 4096-key block

  const uint8_t *crow = cnt + (int64_t)row * cnt_stride;
  const int64_t chunk_begin = (int64_t)chunk * chunk_keys;
  const int64_t chunk_end = (chunk_begin + chunk_keys < n_keys) ? chunk_begin + chunk_keys : n_keys;
  const pkv_u32x4 zero4 = {0u, 0u, 0u, 0u};
  int64_t i0 = chunk_begin + (int64_t)tid * kSelKeysPerThread;
  const uint32_t rs_mine = tid < 128 ? row_suf[(int64_t)row * 128 + tid] : 0u;  // both before the threshold is known
  pkv_u32x4 w = i0 < chunk_end ? *(const pkv_u32x4 *)(crow + i0) : zero4;
  const float qn = qnorm[row];

  pkv_build_prod_table<kSelThreads>(s_prod, qhat + (int64_t)row * 128, centers);
  uint32_t theta;
  int64_t base_gt, base_eq;
  select_prologue(rs_mine, chunk_suf, row, chunk, gridDim.x, k, theta, base_gt, base_eq);
  int64_t *orow = out + (int64_t)row * k;
  float *srow = scores + (int64_t)row * k;
  const uint8_t *nrow = nib + (int64_t)b * ns_b + (int64_t)h * ns_h;
  const uint16_t *wrow = weight + (int64_t)b * ws_b + (int64_t)h * ws_h;

  int it = 0;
  for (int64_t blk0 = chunk_begin; blk0 < chunk_end; blk0 += kSelKeysPerIter, ++it) {
    uint32_t gt[4], eq[4];
    count_masks16(w, theta, chunk_end - i0, gt, eq);
    i0 += kSelKeysPerIter;
    if (blk0 + kSelKeysPerIter < chunk_end) w = i0 < chunk_end ? *(const pkv_u32x4 *)(crow + i0) : zero4;
    const int packed = popc4(gt) | (popc4(eq) << 16);
    int total;
    const int excl = pkv_block_excl_scan<kSelThreads>(packed, s_scan[it & 1], total);
    const int n_gt_it = total & 0xffff, n_sel_it = n_gt_it + (total >> 16);
    // slot in this iteration's LDS list: strictly-above keys first, then the keys at the threshold.  The output
    // position of slot j follows from j alone: pos_gt0 + j for the former, pos_eq0 + j for the latter; ties whose
    // position would reach k are dropped, and they are the list's last slots.
    int lg = excl & 0xffff;
    int le = n_gt_it + (excl >> 16);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t g = gt[d], e = eq[d];
      while (g) {
        const int bit = __ffs((int)g) - 1;
        g &= g - 1;
        s_list_key[lg++] = (uint16_t)(tid * kSelKeysPerThread + 4 * d + (bit >> 3));
      }
      while (e) {
        const int bit = __ffs((int)e) - 1;
        e &= e - 1;
        s_list_key[le++] = (uint16_t)(tid * kSelKeysPerThread + 4 * d + (bit >> 3));
      }
    }
    const int64_t pos_gt0 = base_gt, pos_eq0 = base_eq - n_gt_it, eq_room = k - base_eq;
    const int n_use = eq_room >= (total >> 16) ? n_sel_it : n_gt_it + (int)(eq_room > 0 ? eq_room : 0);
    base_gt += n_gt_it;
    base_eq += total >> 16;
    __syncthreads();
#pragma unroll 1
    for (int j = tid; j < n_use; j += kSelThreads) {
      const int64_t pos = j < n_gt_it ? pos_gt0 + j : pos_eq0 + j;
      {
        const int64_t key = blk0 + s_list_key[j];
        orow[pos] = key;
        const float sc = pkv_rerank_keymajor(s_prod, (const pkv_u32x4 *)(nrow + key * ns_key), (const pkv_u32x4 *)(wrow + key * ws_key), qn);
        srow[pos] = sc;
        const uint32_t o = pkv_ordered_u32(sc);
        smax = o > smax ? o : smax;
        smin = o < smin ? o : smin;
        // one more fp32 word of the key's record (same HBM line), passed through for the caller
        if (extra_out) extra_out[(int64_t)row * k + pos] = *(const float *)(nrow + key * ns_key + extra_off);
      }
    }
    __syncthreads();  // the list is rewritten by the next iteration
  }
  // this chunk's score range for a multi-workgroup top-k that follows: (max, ~min) into one of the row's 16 range
  // slots with atomicMax from zero (one address per row would serialise the atomics of hundreds of workgroups:
  // measured +15 us at 8 rows x 256 chunks; a slot per workgroup costs the readers 3 us of loads)
  if (range_slots) {
#pragma unroll
    for (int x = 1; x < PKV_WAVE; x <<= 1) {
      const uint32_t a = (uint32_t)__shfl_xor((int)smax, x, PKV_WAVE), c = (uint32_t)__shfl_xor((int)smin, x, PKV_WAVE);
      smax = a > smax ? a : smax;
      smin = c < smin ? c : smin;
    }
    if (pkv_lane() == 0) s_scan[0][tid / PKV_WAVE] = (int)smax, s_scan[1][tid / PKV_WAVE] = (int)smin;
    __syncthreads();
    if (tid == 0) {
      for (int wv = 1; wv < kSelThreads / PKV_WAVE; ++wv) {
        const uint32_t a = (uint32_t)s_scan[0][wv], c = (uint32_t)s_scan[1][wv];
        smax = a > smax ? a : smax;
        smin = c < smin ? c : smin;
      }
      if (smax >= smin) {
        uint32_t *slot = range_slots + (int64_t)row * range_row_stride + 2 * (chunk % kWideRangeSlots);
        atomicMax(&slot[0], smax);
        atomicMax(&slot[1], ~smin);
      }
    }
  }
}

// The same for chunks that the collision scan cut into S strided pieces (S even): workgroup c owns pieces
// c, c + n_chunks, ... of piece_keys keys each (pieces numbered in key order), piece_suf holds one suffix histogram per
// piece as a bin-major table [row][bin][chunk][piece of the chunk], and the output positions follow from the prefixes
// over the pieces in key order.  Where the candidates bunch along the row (keys whose
// mean drifts: bands of the zone hold a multiple of the average) a workgroup that owned one contiguous chunk would
// score up to twice the average number of candidates and the launch would last as long as that workgroup; pieces a
// quarter of the row apart average the bands out (8 rows x 1M keys, mean turning 2 degrees per 1K keys: most
// candidates of one workgroup 851 -> 496 for an average of 410).  The candidate list and every score are the same as
// with whole chunks: positions depend on the keys alone.
// Two pieces per pass (threads [0,128) and [128,256) when piece_keys = 2048): the block scan ranks both at once.
constexpr int kSelMaxPieces = 512;

__global__ __launch_bounds__(kSelThreads) void pkv_select_rerank_pieces_kernel(
    const uint8_t *__restrict__ cnt, int64_t cnt_stride, const uint32_t *__restrict__ row_suf,
    const uint16_t *__restrict__ piece_suf, int piece_keys, int pieces_per_chunk, int n_kv_heads, int64_t n_keys, int64_t k,
    const uint8_t *__restrict__ nib, int64_t ns_b, int64_t ns_h, int ns_key, const uint16_t *__restrict__ weight,
    int64_t ws_b, int64_t ws_h, int ws_key, const float *__restrict__ qhat, const float *__restrict__ qnorm,
    const float *__restrict__ centers, int64_t *__restrict__ out, float *__restrict__ scores, int extra_off,
    float *__restrict__ extra_out, uint32_t *__restrict__ range_slots, int64_t range_row_stride) {
  const int row = blockIdx.y;
  const int chunk = blockIdx.x;
  const int n_chunks = gridDim.x;
  const int n_pieces = n_chunks * pieces_per_chunk;
  const int tid = threadIdx.x;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  uint32_t smax = 0u, smin = 0xffffffffu;

  __shared__ int s_scan[2][kSelThreads / PKV_WAVE];
  __shared__ float s_prod[128 * 16];
  __shared__ uint16_t s_list_key[kSelKeysPerIter];  // offset of the key inside the pass's two pieces (second piece: + piece_keys)
  __shared__ uint32_t s_pg[kSelMaxPieces + 1], s_pe[kSelMaxPieces + 1];  // keys above / at the threshold in the pieces before
  __shared__ uint32_t s_rs[129];
  __shared__ uint32_t s_theta, s_ngt;

  const uint8_t *crow = cnt + (int64_t)row * cnt_stride;
  const pkv_u32x4 zero4 = {0u, 0u, 0u, 0u};
  const uint32_t rs_mine = tid < 128 ? row_suf[(int64_t)row * 128 + tid] : 0u;
  // thread t of a pass: half hh = t / (threads per piece), 16 keys at offset (t % threads per piece) * 16 of its piece
  const int tpp = piece_keys / kSelKeysPerThread;  // threads per piece; 2 * tpp <= 256
  const int hh = tid / tpp, tl = tid % tpp;
  const int n_pass = pieces_per_chunk / 2;
  // counts of the first pass, requested before the threshold is known
  auto piece_of = [&](int pass, int half) { return chunk + (pass + half * n_pass) * n_chunks; };  // halves half a chunk's pieces apart
  auto load_counts = [&](int pass) {
    if (hh >= 2) return zero4;
    const int64_t j0 = (int64_t)piece_of(pass, hh) * piece_keys + (int64_t)tl * kSelKeysPerThread;
    return j0 < n_keys ? *(const pkv_u32x4 *)(crow + j0) : zero4;
  };
  pkv_u32x4 w = load_counts(0);
  const float qn = qnorm[row];
  pkv_build_prod_table<kSelThreads>(s_prod, qhat + (int64_t)row * 128, centers);

  // threshold, then the two columns it names for every piece of the row and their prefixes
  if (tid < 128) s_rs[tid] = rs_mine;
  if (tid == 128) s_rs[128] = 0, s_theta = 0, s_ngt = 0;
  __syncthreads();
  if (tid < 128 && (int64_t)s_rs[tid] >= k && (int64_t)s_rs[tid + 1] < k) s_theta = (uint32_t)tid, s_ngt = s_rs[tid + 1];
  __syncthreads();
  const uint32_t theta = s_theta;
  const int64_t n_gt_row = s_ngt;
  {
    // bin-major table [bin][chunk][piece of the chunk]: entries 2t and 2t + 1 of a bin are one 32-bit word; they are
    // put into key order (piece = chunk + j * n_chunks) through LDS before the prefix sums
    const uint32_t *cs = (const uint32_t *)(piece_suf + (int64_t)row * n_pieces * 128);
    if (2 * tid < n_pieces) {
      const uint32_t ge2 = cs[((int64_t)theta * n_pieces) / 2 + tid];
      const uint32_t g2 = theta < 127 ? cs[((int64_t)(theta + 1) * n_pieces) / 2 + tid] : 0u;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        const int idx = 2 * tid + u, c = idx / pieces_per_chunk, jj = idx % pieces_per_chunk;
        const uint32_t gv = u ? g2 >> 16 : g2 & 0xffffu, gev = u ? ge2 >> 16 : ge2 & 0xffffu;
        s_pg[c + jj * n_chunks] = gv;
        s_pe[c + jj * n_chunks] = gev - gv;
      }
    }
    __syncthreads();
    uint32_t g[2] = {0u, 0u}, e[2] = {0u, 0u};
    if (2 * tid < n_pieces) g[0] = s_pg[2 * tid], g[1] = s_pg[2 * tid + 1], e[0] = s_pe[2 * tid], e[1] = s_pe[2 * tid + 1];
    int tot_g, tot_e;
    const uint32_t xg = (uint32_t)pkv_block_excl_scan<kSelThreads>((int)(g[0] + g[1]), s_scan[0], tot_g);
    const uint32_t xe = (uint32_t)pkv_block_excl_scan<kSelThreads>((int)(e[0] + e[1]), s_scan[1], tot_e);
    s_pg[2 * tid] = xg, s_pg[2 * tid + 1] = xg + g[0];
    s_pe[2 * tid] = xe, s_pe[2 * tid + 1] = xe + e[0];
    if (tid == 0) s_pg[kSelMaxPieces] = (uint32_t)tot_g, s_pe[kSelMaxPieces] = (uint32_t)tot_e;  // entry n_pieces when that is the maximum
  }
  __syncthreads();
  int64_t *orow = out + (int64_t)row * k;
  float *srow = scores + (int64_t)row * k;
  const uint8_t *nrow = nib + (int64_t)b * ns_b + (int64_t)h * ns_h;
  const uint16_t *wrow = weight + (int64_t)b * ws_b + (int64_t)h * ws_h;

  for (int pass = 0; pass < n_pass; ++pass) {
    const int p0 = piece_of(pass, 0), p1 = piece_of(pass, 1);
    const int64_t j0 = (int64_t)(hh ? p1 : p0) * piece_keys + (int64_t)tl * kSelKeysPerThread;
    const int64_t piece_end = ((int64_t)(hh ? p1 : p0) + 1) * piece_keys < n_keys ? ((int64_t)(hh ? p1 : p0) + 1) * piece_keys : n_keys;
    uint32_t gt[4], eq[4];
    count_masks16(w, theta, hh < 2 ? piece_end - j0 : 0, gt, eq);
    if (pass + 1 < n_pass) w = load_counts(pass + 1);
    const int packed = popc4(gt) | (popc4(eq) << 16);
    int total;
    const int excl = pkv_block_excl_scan<kSelThreads>(packed, s_scan[pass & 1], total);
    // the piece tables already hold what the scan would tell: keys above / at the threshold in each of the two pieces
    const int n_g0 = (int)(s_pg[p0 + 1] - s_pg[p0]), n_g1 = (int)(s_pg[p1 + 1] - s_pg[p1]);
    const int n_e0 = (int)(s_pe[p0 + 1] - s_pe[p0]);
    const int64_t room0 = k - n_gt_row - (int64_t)s_pe[p0], room1 = k - n_gt_row - (int64_t)s_pe[p1];
    const int u_e0 = (int)(room0 <= 0 ? 0 : (room0 < n_e0 ? room0 : n_e0));                  // keys at the threshold that find room
    const int n_e1 = (int)(s_pe[p1 + 1] - s_pe[p1]);
    const int u_e1 = (int)(room1 <= 0 ? 0 : (room1 < n_e1 ? room1 : n_e1));
    const int n_g = n_g0 + n_g1;
    // list of the pass: [above, piece 0][above, piece 1][at, piece 0, first u_e0][at, piece 1, first u_e1]
    int lg = excl & 0xffff;                                              // ranks both halves in thread order = this layout
    int re = (excl >> 16) - (hh ? n_e0 : 0);                             // rank among the keys at the threshold of the own piece
    const int e_used = hh ? u_e1 : u_e0, e_base = n_g + (hh ? u_e0 : 0);
    const uint32_t off0 = (uint32_t)(hh * piece_keys + tl * kSelKeysPerThread);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      uint32_t g = gt[d], e = eq[d];
      while (g) {
        const int bit = __ffs((int)g) - 1;
        g &= g - 1;
        s_list_key[lg++] = (uint16_t)(off0 + 4 * d + (bit >> 3));
      }
      while (e) {
        const int bit = __ffs((int)e) - 1;
        e &= e - 1;
        if (re < e_used) s_list_key[e_base + re] = (uint16_t)(off0 + 4 * d + (bit >> 3));
        ++re;
      }
    }
    const int n_use = n_g + u_e0 + u_e1;
    const int64_t pg0 = s_pg[p0], pg1 = s_pg[p1], pe0 = n_gt_row + s_pe[p0], pe1 = n_gt_row + s_pe[p1];
    __syncthreads();
#pragma unroll 1
    for (int j = tid; j < n_use; j += kSelThreads) {
      const int64_t pos = j < n_g0 ? pg0 + j : (j < n_g ? pg1 + (j - n_g0) : (j < n_g + u_e0 ? pe0 + (j - n_g) : pe1 + (j - n_g - u_e0)));
      const uint32_t off = s_list_key[j];
      const int64_t key = (off < (uint32_t)piece_keys ? (int64_t)p0 * piece_keys : (int64_t)(p1 - 1) * piece_keys) + off;
      orow[pos] = key;
      const float sc = pkv_rerank_keymajor(s_prod, (const pkv_u32x4 *)(nrow + key * ns_key), (const pkv_u32x4 *)(wrow + key * ws_key), qn);
      srow[pos] = sc;
      const uint32_t o = pkv_ordered_u32(sc);
      smax = o > smax ? o : smax;
      smin = o < smin ? o : smin;
      if (extra_out) extra_out[(int64_t)row * k + pos] = *(const float *)(nrow + key * ns_key + extra_off);
    }
    __syncthreads();  // the list is rewritten by the next pass
  }
  if (range_slots) {
#pragma unroll
    for (int x = 1; x < PKV_WAVE; x <<= 1) {
      const uint32_t a = (uint32_t)__shfl_xor((int)smax, x, PKV_WAVE), c = (uint32_t)__shfl_xor((int)smin, x, PKV_WAVE);
      smax = a > smax ? a : smax;
      smin = c < smin ? c : smin;
    }
    if (pkv_lane() == 0) s_scan[0][tid / PKV_WAVE] = (int)smax, s_scan[1][tid / PKV_WAVE] = (int)smin;
    __syncthreads();
    if (tid == 0) {
      for (int wv = 1; wv < kSelThreads / PKV_WAVE; ++wv) {
        const uint32_t a = (uint32_t)s_scan[0][wv], c = (uint32_t)s_scan[1][wv];
        smax = a > smax ? a : smax;
        smin = c < smin ? c : smin;
      }
      if (smax >= smin) {
        uint32_t *slot = range_slots + (int64_t)row * range_row_stride + 2 * (chunk % kWideRangeSlots);
        atomicMax(&slot[0], smax);
        atomicMax(&slot[1], ~smin);
      }
    }
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

// int32 counts -> clamped u8 counts (padded rows) + per-chunk suffix histograms + row suffix totals.
__global__ __launch_bounds__(256) void pkv_counts_to_u8_kernel(const int32_t *__restrict__ x, int64_t x_stride,
                                                               int64_t len, uint8_t *__restrict__ cnt,
                                                               int64_t cnt_stride, uint32_t *__restrict__ row_suf,
                                                               uint16_t *__restrict__ chunk_suf, int chunk_keys) {
  const int row = blockIdx.y, chunk = blockIdx.x, tid = threadIdx.x;
  __shared__ uint32_t s_hist[128];
  __shared__ uint32_t s_w0;
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
  pkv_store_suffix_hist(s_hist, &s_w0, row_suf ? row_suf + (int64_t)row * 128 : nullptr,
                        chunk_suf + ((int64_t)row * gridDim.x + chunk) * 128);
}

__global__ void pkv_zero_u32_kernel(uint32_t *__restrict__ p, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// ------------------------------------------------------------ exact fp32 top-k

constexpr int kTopkThreads = 1024;
constexpr int kTopkMaxSort = 8192;  // 64 KB of 64-bit keys in LDS

__device__ __forceinline__ uint64_t make_key(const float *__restrict__ x, const int64_t *__restrict__ ids,
                                             int64_t i) {
  const uint32_t id = ids ? (uint32_t)ids[i] : (uint32_t)i;
  return ((uint64_t)pkv_ordered_u32(x[i]) << 32) | (uint64_t)(~id);
}

// Key of lane (lane ^ mask); mask is a constant once the callers' loops are unrolled, so the switch folds.
__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int mask) {
  switch (mask) {
    case 1: return pkv_lane_xor64<1>(v);
    case 2: return pkv_lane_xor64<2>(v);
    case 4: return pkv_lane_xor64<4>(v);
    case 8: return pkv_lane_xor64<8>(v);
    case 16: return pkv_lane_xor64<16>(v);
    default: return pkv_lane_xor64<32>(v);
  }
}

// hist[d] += 1 for every active lane.  In each of `rounds` rounds the lanes of a wave that share the
// leading lane's digit are added with one atomic, which is what keeps the first radix passes, where
// nearly all keys fall into one or two buckets, from serialising on a single LDS address.
__device__ __forceinline__ void wave_hist_add(uint32_t *hist, uint32_t d, bool active, int rounds) {
  for (int r = 0; r < rounds; ++r) {
    const uint64_t act = __ballot(active);
    if (act == 0) return;
    const int leader = __ffsll((long long)act) - 1;
    const uint32_t dl = (uint32_t)__builtin_amdgcn_readlane((int)d, leader);
    const uint64_t same = __ballot(active && d == dl);
    if (pkv_lane() == leader) atomicAdd(&hist[dl], (uint32_t)__popcll((long long)same));
    if (d == dl) active = false;
  }
  if (active) atomicAdd(&hist[d], 1u);
}

// Slot for every lane with `take` set, out of a workgroup-wide counter: one atomic per wave.
__device__ __forceinline__ uint32_t wave_take_slots(uint32_t *counter, bool take) {
  const uint64_t m = __ballot(take);
  if (m == 0) return 0u;
  const int leader = __ffsll((long long)m) - 1;
  uint32_t base = 0;
  if (pkv_lane() == leader) base = atomicAdd(counter, (uint32_t)__popcll((long long)m));
  base = (uint32_t)__builtin_amdgcn_readlane((int)base, leader);
  const uint64_t below = m & (((uint64_t)1 << pkv_lane()) - 1);
  return base + (uint32_t)__popcll((long long)below);
}

// Descending bitonic sort of NT*E 64-bit keys held E per thread by the first NT threads of the
// 1024-thread workgroup (thread t owns sorted positions t*E .. t*E+E-1); ALL 1024 threads must call it,
// the others only take part in the barriers.  Strides below E are exchanged inside the thread, strides
// below 64*E between the lanes of a wave (no barrier), only the remaining strides go through LDS
// (`s_buf`, NT*E keys, laid out [e][thread] so that a wave touches consecutive addresses).
template <int NT, int E>
__device__ __forceinline__ void bitonic_sort_desc_regs(uint64_t (&v)[E], uint64_t *s_buf) {
  constexpr int P = NT * E;
  const int tid = threadIdx.x;
  const bool active = tid < NT;
#pragma unroll
  for (int size = 2; size <= P; size <<= 1) {
#pragma unroll
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      if (stride < E) {
        if (active) {
#pragma unroll
          for (int e = 0; e < E; ++e) {
            if ((e & stride) == 0) {
              const bool desc = ((tid * E + e) & size) == 0;
              const uint64_t a = v[e], b = v[e | stride];
              const bool sw = desc ? (a < b) : (a > b);
              v[e] = sw ? b : a;
              v[e | stride] = sw ? a : b;
            }
          }
        }
      } else if (stride < PKV_WAVE * E) {
        if (active) {  // whole waves: NT is a multiple of 64
#pragma unroll
          for (int e = 0; e < E; ++e) {
            const int i = tid * E + e;
            const uint64_t o = shfl_xor_u64(v[e], stride / E);
            const bool want_max = ((i & stride) == 0) == ((i & size) == 0);
            v[e] = ((v[e] > o) == want_max) ? v[e] : o;  // keys are distinct (or both zero padding)
          }
        }
      } else {
        __syncthreads();  // earlier readers of s_buf are done
        if (active) {
#pragma unroll
          for (int e = 0; e < E; ++e) s_buf[e * NT + tid] = v[e];
        }
        __syncthreads();
        if (active) {
#pragma unroll
          for (int e = 0; e < E; ++e) {
            const int i = tid * E + e;
            const uint64_t o = s_buf[e * NT + (tid ^ (stride / E))];
            const bool want_max = ((i & stride) == 0) == ((i & size) == 0);
            v[e] = ((v[e] > o) == want_max) ? v[e] : o;
          }
        }
      }
    }
  }
}

// Sort the keys in s_keys[0 .. NT*E) (zero padded) and emit the first k.  Called by all 1024 threads.
template <int NT, int E>
__device__ __forceinline__ void sort_lds_keys_and_emit(uint64_t *s_keys, int64_t k, int64_t *__restrict__ out_ids,
                                                       float *__restrict__ out_vals, uint64_t *sorted_copy) {
  const bool active = threadIdx.x < NT;
  uint64_t v[E];
#pragma unroll
  for (int e = 0; e < E; ++e) v[e] = active ? s_keys[threadIdx.x * E + e] : 0ull;
  __syncthreads();
  bitonic_sort_desc_regs<NT, E>(v, s_keys);
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int64_t i = (int64_t)threadIdx.x * E + e;
    if (active && i < k) {
      out_ids[i] = (int64_t)(uint32_t)(~(uint32_t)v[e]);
      if (out_vals) out_vals[i] = pkv_from_ordered_u32((uint32_t)(v[e] >> 32));
    }
  }
  if (sorted_copy) {  // the caller wants the sorted keys back in LDS
    __syncthreads();
    if (active) {
#pragma unroll
      for (int e = 0; e < E; ++e) sorted_copy[threadIdx.x * E + e] = v[e];
    }
    __syncthreads();
  }
}

// P keys (a power of two, at least 1024 slots in LDS): threads x keys per thread.  All 1024 threads
// with few keys each measured faster than fewer threads with more (1024 keys: 11.9 us per launch on
// 1024 threads, 12.3 on 512, 13.5 on 256): the compare-exchanges are issue-bound on the one CU.
#define PKV_DISPATCH_E(P, CALL)               \
  do {                                        \
    if ((P) <= 1024) { CALL(1024, 1); }       \
    else if ((P) == 2048) { CALL(1024, 2); }  \
    else if ((P) == 4096) { CALL(1024, 4); }  \
    else { CALL(1024, 8); }                   \
  } while (0)

// len <= 8192: sort everything.  One workgroup per row, dynamic LDS max(P,1024)*8 bytes.
__global__ __launch_bounds__(kTopkThreads) void pkv_topk_sort_kernel(const float *__restrict__ x, int64_t x_stride,
                                                                     const int64_t *__restrict__ ids,
                                                                     int64_t ids_stride, int len, int P, int64_t k,
                                                                     int64_t *__restrict__ out_ids,
                                                                     float *__restrict__ out_vals) {
  extern __shared__ uint64_t s_keys[];
  const int row = blockIdx.x;
  const float *xr = x + (int64_t)row * x_stride;
  const int64_t *ir = ids ? ids + (int64_t)row * ids_stride : nullptr;
  int64_t *oi = out_ids + (int64_t)row * k;
  float *ov = out_vals ? out_vals + (int64_t)row * k : nullptr;
#define PKV_SORT_ALL(NT, E)                                                        \
  {                                                                                \
    uint64_t v[E];                                                                 \
    _Pragma("unroll") for (int e = 0; e < E; ++e) {                                \
      const int i = threadIdx.x * E + e;                                           \
      v[e] = (threadIdx.x < NT && i < len) ? make_key(xr, ir, i) : 0ull;           \
    }                                                                              \
    bitonic_sort_desc_regs<NT, E>(v, s_keys);                                      \
    _Pragma("unroll") for (int e = 0; e < E; ++e) {                                \
      const int64_t i = (int64_t)threadIdx.x * E + e;                              \
      if (threadIdx.x < NT && i < k) {                                             \
        oi[i] = (int64_t)(uint32_t)(~(uint32_t)v[e]);                              \
        if (ov) ov[i] = pkv_from_ordered_u32((uint32_t)(v[e] >> 32));              \
      }                                                                            \
    }                                                                              \
  }
  PKV_DISPATCH_E(P, PKV_SORT_ALL);
#undef PKV_SORT_ALL
}

// Digit of `key` in radix pass `pass` (8 bits, most significant first) and whether the key still
// matches the prefix found by the earlier passes; works on the 32-bit halves of the key.
__device__ __forceinline__ void radix_digit(uint64_t key, uint64_t prefix, int pass, uint32_t &digit, bool &match) {
  const uint32_t hi = (uint32_t)(key >> 32), lo = (uint32_t)key;
  const uint32_t phi = (uint32_t)(prefix >> 32), plo = (uint32_t)prefix;
  const int sh = 24 - 8 * (pass & 3);
  if (pass < 4) {
    digit = (hi >> sh) & 255u;
    match = pass == 0 || (hi >> (sh + 8)) == (phi >> (sh + 8));
  } else {
    digit = (lo >> sh) & 255u;
    match = hi == phi && (pass == 4 || (lo >> (sh + 8)) == (plo >> (sh + 8)));
  }
}

// Second half of a radix-select pass, called by all 1024 threads after their histogram atomics: the
// first wave scans the pass's 256 bins (lane l owns digits 255 - 4l .. 252 - 4l, descending, so an
// inclusive scan over lanes is the suffix sum over digits) and leaves in s_bcast[(pass & 1) * 4 ..]:
// the threshold digit, the keys still needed inside that bucket, and whether the bucket is taken whole.
// Meanwhile the other histogram buffer is cleared for the next pass.  Two barriers.
__device__ __forceinline__ void radix_pass_decide(uint32_t *s_hist, uint32_t *s_bcast, int pass, uint32_t need) {
  const int tid = threadIdx.x;
  const uint32_t *hist = s_hist + (pass & 1) * 256;
  uint32_t *res = s_bcast + (pass & 1) * 4;
  __syncthreads();
  if (tid < PKV_WAVE) {
    uint32_t h[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) h[j] = hist[255 - 4 * tid - j];
    const uint32_t mine = h[0] + h[1] + h[2] + h[3];
    uint32_t above = (uint32_t)pkv_wave_incl_scan((int)mine) - mine;  // keys in digits above this lane's four
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (above < need && above + h[j] >= need) {
        res[0] = (uint32_t)(255 - 4 * tid - j);
        res[1] = need - above;
        res[2] = (h[j] == need - above);
      }
      above += h[j];
    }
  } else if (tid < PKV_WAVE + 256) {
    s_hist[((pass + 1) & 1) * 256 + tid - PKV_WAVE] = 0;
  }
  __syncthreads();
}

// MSB-first 8-bit radix select of the k-th largest of the 64-bit keys held EIN per thread.
// Returns the threshold prefix and the shift at which it became exact: the k winners are the keys
// with (key >> shift) >= (prefix >> shift).  Stops as soon as the threshold bucket is taken whole.
// s_hist: 512 words (two alternating histograms), s_bcast: 8 words.
template <int EIN>
__device__ __forceinline__ void radix_select_regs(const uint64_t (&v)[EIN], uint32_t k, uint32_t *s_hist,
                                                  uint32_t *s_bcast, uint64_t &prefix_out, int &shift_out) {
  const int tid = threadIdx.x;
  uint64_t prefix = 0;
  uint32_t need = k;
  int shift = 56;
  if (tid < 512) s_hist[tid] = 0;
  __syncthreads();
  for (int pass = 0; pass < 8; ++pass, shift -= 8) {
    uint32_t *hist = s_hist + (pass & 1) * 256;
    uint32_t *res = s_bcast + (pass & 1) * 4;
#pragma unroll
    for (int e = 0; e < EIN; ++e) {
      uint32_t digit;
      bool match;
      radix_digit(v[e], prefix, pass, digit, match);
      wave_hist_add(hist, digit, match, pass < 2 ? 2 : 0);
    }
    radix_pass_decide(s_hist, s_bcast, pass, need);
    prefix |= (uint64_t)res[0] << shift;
    need = res[1];
    if (res[2] != 0 || pass == 7) break;
  }
  prefix_out = prefix;
  shift_out = shift;
}

// ---- selection through kLinBins linear bins of the row's own score range ----
//
// The 8-bit radix passes above look at fixed bit fields: scores of one row share their sign and most exponent
// bits, so the first pass separates almost nothing and three passes are the rule.  Here the bins divide
// [row min, row max] evenly: bin(x) = min(kLinBins - 1, floor((x - lo) * kLinBins / (hi - lo))), a non-decreasing function
// of x whatever the rounding of its three operations, so every key in a higher bin is a larger key.  One
// histogram pass finds the bin b* that holds the k-th largest key and how many of its keys are needed; the
// exact threshold key T is then the need-th largest of that one bin, found by counting (a bin holds len / kLinBins
// keys on average).  Winners: bin > b*, or bin == b* and key >= T.  The bins also order the winners: those
// of bin b occupy the output slots [off[b], off[b] + count[b]), and the slot inside the bin is again found by
// counting, which replaces the bitonic sort (and T: the first `need` of b* by that count are its winners).
// Rows this does not suit take the older steps: non-finite scores, a zero or subnormal range or more than
// kLinBucketMax keys in b* the radix select; more than kLinRankMax winners in one bin the bitonic sort.  The
// result is the same set in the same order either way.
constexpr int kLinBins = 512;   // a multiple of 64: wave 0 owns kLinBins / 64 bins per lane
constexpr int kLinBinBits = 9;
constexpr int kLinBucketMax = 256;
constexpr int kLinRankMax = 128;
constexpr int kCountingSortMaxP = 2048;  // largest winner list whose counting sort (a second copy in LDS) is set up

struct LinSel {
  float lo, scale;        // value bins: bin = floor((x - lo) * scale)
  uint32_t lo_bits;       // bit bins: bin = (ordered bits of x - lo_bits) >> shift, piecewise logarithmic in x
  int shift;              // < 0: value bins
  uint32_t bstar, need;   // threshold bin, keys needed from it
  uint32_t in_bstar;      // keys in the threshold bin
  uint32_t max_winners;   // most winners in one bin
  uint64_t T;             // threshold key inside bin b* (0: the whole bin wins); set by linear_threshold
};

__device__ __forceinline__ uint32_t lin_bin(uint64_t key, const LinSel &L) {
  uint32_t b;
  if (L.shift >= 0) {
    b = ((uint32_t)(key >> 32) - L.lo_bits) >> L.shift;
  } else {
    const float t = (pkv_from_ordered_u32((uint32_t)(key >> 32)) - L.lo) * L.scale;
    b = (uint32_t)t;
  }
  return b > (uint32_t)(kLinBins - 1) ? (uint32_t)(kLinBins - 1) : b;
}

// Bins of the thread's keys and the threshold bin.  On return s_hist[0,kLinBins) = keys per bin, s_hist[kLinBins,2*kLinBins) =
// off[b] = keys in the bins above b, s_cnt[b] = off[b] (a running output slot for the counting sort), s_bcast[6] = 0.
// s_hist: 2*kLinBins words, s_cnt: kLinBins words, s_bcast: 8 words.  All 1024 threads call it; false = not applicable.
// BITS: bins of the ordered key bits instead of the values, for rows of one sign whose values span many binades
// (e.g. the winners of a selection, about to be sorted): kLinBins equal steps of the bit pattern between the row's
// smallest and largest key, i.e. equal steps of the logarithm up to the mantissa's linear pieces.
// range: null, or the largest and the smallest ordered score of the nonzero keys (range[0] < range[1]: no key at
// all) where the caller knows them already, which saves the reduction that finds them.
template <int EIN, bool BITS = false>
__device__ __forceinline__ bool linear_bins(const uint64_t (&v)[EIN], uint32_t k, uint32_t *s_hist, uint32_t *s_cnt,
                                            uint32_t *s_bcast, uint32_t (&bin)[EIN], LinSel &L,
                                            const uint32_t *range = nullptr) {
  const int tid = threadIdx.x, lane = pkv_lane();
  for (int i = tid; i < 2 * kLinBins; i += kTopkThreads) s_hist[i] = 0;
  // [2..4]: threshold bin, keys needed from it, keys in it.  They are set below only if some bin reaches k; a row
  // with fewer than k keys leaves "keys in the threshold bin" at its all-ones start and the caller falls back.
  if (tid == 0)
    s_bcast[0] = 0u, s_bcast[1] = 0xffffffffu, s_bcast[2] = 0u, s_bcast[3] = 0u, s_bcast[4] = 0xffffffffu, s_bcast[5] = 0u,
    s_bcast[6] = 0u;
  __syncthreads();
  uint32_t mx = 0u, mn = 0xffffffffu;
  if (range) {
    mx = range[0], mn = range[1];
  } else {
#pragma unroll
  for (int e = 0; e < EIN; ++e) {
    if (v[e] != 0ull) {
      const uint32_t hi = (uint32_t)(v[e] >> 32);
      mx = hi > mx ? hi : mx;
      mn = hi < mn ? hi : mn;
    }
  }
#define PKV_LIN_RED(M)                              \
  {                                                 \
    const uint32_t a = pkv_lane_xor<M>(mx), c = pkv_lane_xor<M>(mn); \
    mx = a > mx ? a : mx;                           \
    mn = c < mn ? c : mn;                           \
  }
  PKV_LIN_RED(1) PKV_LIN_RED(2) PKV_LIN_RED(4) PKV_LIN_RED(8) PKV_LIN_RED(16) PKV_LIN_RED(32)
#undef PKV_LIN_RED
  if (lane == 0) {
    atomicMax(&s_bcast[0], mx);
    atomicMin(&s_bcast[1], mn);
  }
  __syncthreads();
  mx = s_bcast[0], mn = s_bcast[1];
  }
  L.lo = 0.f, L.scale = 0.f, L.lo_bits = mn, L.shift = -1;
  if (BITS) {
    if (mx <= mn) return false;  // one value (or no key at all)
    const int width = 32 - __clz((int)(mx - mn));
    L.shift = width > kLinBinBits ? width - kLinBinBits : 0;
  } else {
    const float hi = pkv_from_ordered_u32(mx), lo = pkv_from_ordered_u32(mn);
    const float range = hi - lo, scale = (float)kLinBins / range;
    const float inf = __uint_as_float(0x7f800000u);
    // finite scores (ordered keys strictly between those of -inf and +inf), a positive finite range and scale
    if (!(mx < 0xff800000u && mn > 0x007fffffu && range > 0.f && range < inf && scale < inf)) return false;
    L.lo = lo, L.scale = scale;
  }
#pragma unroll
  for (int e = 0; e < EIN; ++e) {
    bin[e] = 0;
    if (v[e] != 0ull) {
      bin[e] = lin_bin(v[e], L);
      atomicAdd(&s_hist[bin[e]], 1u);
    }
  }
  __syncthreads();
  if (tid < PKV_WAVE) {  // lane l owns the kPer bins below kLinBins - kPer * l: an inclusive scan over lanes is the suffix sum over bins
    constexpr int kPer = kLinBins / PKV_WAVE;
    uint32_t h[kPer];
    uint32_t mine = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      h[j] = s_hist[kLinBins - 1 - kPer * tid - j];
      mine += h[j];
    }
    uint32_t above = (uint32_t)pkv_wave_incl_scan((int)mine) - mine;
    uint32_t most = 0;
#pragma unroll
    for (int j = 0; j < kPer; ++j) {
      const int b = kLinBins - 1 - kPer * tid - j;
      s_hist[kLinBins + b] = above;
      s_cnt[b] = above;
      if (above < k) {
        const uint32_t take = above + h[j] >= k ? k - above : h[j];
        most = take > most ? take : most;
        if (above + h[j] >= k) s_bcast[2] = (uint32_t)b, s_bcast[3] = take, s_bcast[4] = h[j];
      }
      above += h[j];
    }
    // every lane exchange is evaluated once, by all lanes: inside a conditional expression the compiler may run it
    // under a partial execution mask, and a lane-crossing read of an inactive lane returns nothing
#define PKV_MAX_XOR(M)                               \
  {                                                  \
    const uint32_t o = pkv_lane_xor<M>(most);        \
    most = o > most ? o : most;                      \
  }
    PKV_MAX_XOR(1) PKV_MAX_XOR(2) PKV_MAX_XOR(4) PKV_MAX_XOR(8)
#undef PKV_MAX_XOR
    if ((tid & 15) == 0) atomicMax(&s_bcast[5], most);
  }
  __syncthreads();
  L.bstar = s_bcast[2], L.need = s_bcast[3], L.in_bstar = s_bcast[4], L.max_winners = s_bcast[5];
  L.T = 0ull;
  return L.in_bstar <= kLinBucketMax;
}

// Threshold key of bin b*: the need-th largest of its keys, found by counting with 16 lanes per key.
// s_bcast[6] must be 0 (linear_bins leaves it so).  All 1024 threads call it.
template <int EIN>
__device__ __forceinline__ void linear_threshold(const uint64_t (&v)[EIN], const uint32_t (&bin)[EIN], uint32_t *s_bcast,
                                                 uint64_t *s_bucket, uint64_t *s_T, LinSel &L) {
  if (L.in_bstar == L.need) return;  // the bin is taken whole: T = 0
#pragma unroll
  for (int e = 0; e < EIN; ++e) {  // about one key in kLinBins: most waves skip the atomic altogether
    if (v[e] != 0ull && bin[e] == L.bstar) s_bucket[atomicAdd(&s_bcast[6], 1u)] = v[e];
  }
  __syncthreads();
  const uint32_t n = L.in_bstar, sub = threadIdx.x & 15u;
  for (uint32_t i = threadIdx.x >> 4; i < n; i += kTopkThreads / 16) {
    const uint64_t key = s_bucket[i];
    uint32_t r = 0;
    for (uint32_t j = sub; j < n; j += 16) r += s_bucket[j] > key ? 1u : 0u;
    r += pkv_lane_xor<1>(r);
    r += pkv_lane_xor<2>(r);
    r += pkv_lane_xor<4>(r);
    r += pkv_lane_xor<8>(r);
    if (sub == 0 && r == L.need - 1) *s_T = key;
  }
  __syncthreads();
  L.T = *s_T;
}

// LDS scratch of a selection / sort over one workgroup's keys.
struct SelSmem {
  uint32_t hist[2 * kLinBins];
  uint32_t cnt[kLinBins];
  uint32_t bcast[8];
  uint32_t counter;
  uint64_t bucket[kLinBucketMax];
  uint64_t T;
};

// win[e] = key e of this thread is one of the k largest of the workgroup's keys (zero keys never are).  Bins of
// the row's own range first (BITS: of the ordered key bits), the radix select where they do not apply.
template <int EIN, bool BITS>
__device__ __forceinline__ void select_topk_flags(const uint64_t (&v)[EIN], uint32_t k, SelSmem &sm, bool (&win)[EIN]) {
  uint32_t bin[EIN];
  LinSel L;
  if (linear_bins<EIN, BITS>(v, k, sm.hist, sm.cnt, sm.bcast, bin, L)) {
    linear_threshold<EIN>(v, bin, sm.bcast, sm.bucket, &sm.T, L);
#pragma unroll
    for (int e = 0; e < EIN; ++e) win[e] = v[e] != 0ull && (bin[e] > L.bstar || (bin[e] == L.bstar && v[e] >= L.T));
  } else {
    uint64_t prefix;
    int shift;
    radix_select_regs<EIN>(v, k, sm.hist, sm.bcast, prefix, shift);
#pragma unroll
    for (int e = 0; e < EIN; ++e) win[e] = v[e] != 0ull && (v[e] >> shift) >= (prefix >> shift);
  }
}

// Descending sort of the n nonzero keys held E per thread (all other entries zero) into s_out[0 .. n), through
// s_tmp (n keys, not s_out): kLinBins bins of the ordered key bits between the smallest and the largest key, every key
// placed at (keys in higher bins) + (larger keys in its own bin).  False, with nothing written, when a bin holds
// more than kLinRankMax keys or all keys are equal: the caller then sorts by compare-exchange.
template <int E>
__device__ __forceinline__ bool counting_sort_desc(const uint64_t (&v)[E], uint32_t n, uint64_t *s_tmp, uint64_t *s_out,
                                                   SelSmem &sm) {
  uint32_t bin[E];
  LinSel L;
  if (!linear_bins<E, true>(v, n, sm.hist, sm.cnt, sm.bcast, bin, L) || L.max_winners > kLinRankMax) return false;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    if (v[e] != 0ull) s_tmp[atomicAdd(&sm.cnt[bin[e]], 1u)] = v[e];
  }
  __syncthreads();
  const uint32_t *s_off = sm.hist + kLinBins;
  for (uint32_t p = threadIdx.x; p < n; p += kTopkThreads) {
    const uint64_t key = s_tmp[p];
    const uint32_t b = lin_bin(key, L);
    const uint32_t start = s_off[b], cnt = sm.cnt[b] - start;
    uint32_t r = 0;
#pragma unroll 4
    for (uint32_t j = 0; j < cnt; ++j) r += s_tmp[start + j] > key ? 1u : 0u;
    s_out[start + r] = key;
  }
  __syncthreads();
  return true;
}

// emit(key, rank) for every key of s_bucket[0 .. n), n <= kLinBucketMax <= 256: rank = number of larger keys, counted
// by 4 lanes per key, the workgroup's last threads first (the callers' other loops keep the first ones busier).
// All 1024 threads call it.
template <typename Emit>
__device__ __forceinline__ void rank_bucket_desc(const uint64_t *s_bucket, uint32_t n, Emit emit) {
  const uint32_t i = (kTopkThreads - 1 - threadIdx.x) >> 2, sub = threadIdx.x & 3u;
  const uint64_t key = s_bucket[i < n ? i : 0];
  uint32_t r = 0;
#pragma unroll 4
  for (uint32_t j = sub; j < n; j += 4) r += s_bucket[j] > key ? 1u : 0u;
  r += pkv_lane_xor<1>(r);
  r += pkv_lane_xor<2>(r);
  if (sub == 0 && i < n) emit(key, r);
}

// Selection and sort in one binning: the k largest of the nonzero keys held E per thread (there are at least k),
// sorted descending, into s_out[0 .. k), through s_tmp (k keys, not s_out).  Bins as in counting_sort_desc, over all
// the keys: those of the bins above the threshold bin b* are placed as there, those of b* are ranked among themselves
// and the first `need` follow.  False, with s_out untouched, when b* holds more than kLinBucketMax keys, a bin more
// than kLinRankMax winners, or all keys are equal: the caller then selects and sorts in two steps.  range: as for
// linear_bins.
template <int E>
__device__ __forceinline__ bool select_sort_desc(const uint64_t (&v)[E], uint32_t k, uint64_t *s_tmp, uint64_t *s_out,
                                                 SelSmem &sm, const uint32_t *range = nullptr) {
  uint32_t bin[E];
  LinSel L;
  if (!linear_bins<E, true>(v, k, sm.hist, sm.cnt, sm.bcast, bin, L, range) || L.max_winners > kLinRankMax) return false;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    if (v[e] != 0ull) {
      if (bin[e] > L.bstar) s_tmp[atomicAdd(&sm.cnt[bin[e]], 1u)] = v[e];
      else if (bin[e] == L.bstar) sm.bucket[atomicAdd(&sm.bcast[6], 1u)] = v[e];
    }
  }
  __syncthreads();
  const uint32_t *s_off = sm.hist + kLinBins;
  const uint32_t n_above = k - L.need;
  // The lower a slot, the fewer keys its bin holds: the slots are handed out in pairs (p, n_above - 1 - p), so that
  // a wave takes crowded and sparse bins in turn.
  const uint32_t half = (n_above + 1) / 2;
  for (uint32_t q = threadIdx.x; q < 2 * half; q += kTopkThreads) {
    const uint32_t p = q < half ? q : n_above - 1 - (q - half);
    if (q >= half && p < half) continue;  // the middle slot of an odd count is the first half's
    const uint64_t key = s_tmp[p];
    const uint32_t b = lin_bin(key, L);
    const uint32_t start = s_off[b], cnt = sm.cnt[b] - start;
    uint32_t r = 0;
#pragma unroll 4
    for (uint32_t j = 0; j < cnt; ++j) r += s_tmp[start + j] > key ? 1u : 0u;
    s_out[start + r] = key;
  }
  rank_bucket_desc(sm.bucket, L.in_bstar, [&](uint64_t key, uint32_t r) {
    if (r < L.need) s_out[n_above + r] = key;
  });
  __syncthreads();
  return true;
}

// s_keys[0 .. P) (the n winners, any order, zero padded) sorted descending in place; s_tmp: P more keys or null.
template <int NT, int E>
__device__ __forceinline__ void sort_lds_keys_desc(uint64_t *s_keys, uint32_t n, uint64_t *s_tmp, SelSmem &sm) {
  const bool active = threadIdx.x < NT;
  uint64_t v[E];
#pragma unroll
  for (int e = 0; e < E; ++e) v[e] = active ? s_keys[threadIdx.x * E + e] : 0ull;
  __syncthreads();
  if (s_tmp && counting_sort_desc<E>(v, n, s_tmp, s_keys, sm)) return;
  bitonic_sort_desc_regs<NT, E>(v, s_keys);
  __syncthreads();
  if (active) {
#pragma unroll
    for (int e = 0; e < E; ++e) s_keys[threadIdx.x * E + e] = v[e];
  }
  __syncthreads();
}

// The same selection over keys that do not fit the registers: key_of(i), i < len, is evaluated again
// in every pass.
template <typename KeyFn>
__device__ __forceinline__ void radix_select_streamed(KeyFn key_of, int64_t len, uint32_t k, uint32_t *s_hist,
                                                      uint32_t *s_bcast, uint64_t &prefix_out, int &shift_out) {
  const int tid = threadIdx.x;
  uint64_t prefix = 0;
  uint32_t need = k;
  int shift = 56;
  if (tid < 512) s_hist[tid] = 0;
  __syncthreads();
  for (int pass = 0; pass < 8; ++pass, shift -= 8) {
    uint32_t *hist = s_hist + (pass & 1) * 256;
    const uint32_t *res = s_bcast + (pass & 1) * 4;
    for (int64_t i0 = 0; i0 < len; i0 += kTopkThreads) {  // whole waves stay in the loop: it uses ballots
      const int64_t i = i0 + tid;
      const uint64_t key = i < len ? key_of(i) : 0ull;
      uint32_t digit;
      bool match;
      radix_digit(key, prefix, pass, digit, match);
      wave_hist_add(hist, digit, i < len && match, pass < 2 ? 2 : 0);
    }
    radix_pass_decide(s_hist, s_bcast, pass, need);
    prefix |= (uint64_t)res[0] << shift;
    need = res[1];
    if (res[2] != 0 || pass == 7) break;
  }
  prefix_out = prefix;
  shift_out = shift;
}

// Winners of a streamed selection into s_keys[0 .. k) (any order); s_counter must be 0.
template <typename KeyFn>
__device__ __forceinline__ void collect_winners_streamed(KeyFn key_of, int64_t len, uint32_t k, uint64_t prefix,
                                                         int shift, uint32_t *s_counter, uint64_t *s_keys) {
  for (int64_t i0 = 0; i0 < len; i0 += kTopkThreads) {
    const int64_t i = i0 + threadIdx.x;
    const uint64_t key = i < len ? key_of(i) : 0ull;
    const bool win = i < len && (key >> shift) >= (prefix >> shift);
    const uint32_t slot = wave_take_slots(s_counter, win);
    if (win && slot < k) s_keys[slot] = key;
  }
}

// len <= 8192 and k well below len: select the k winners exactly, then sort only those.
// SORTED = false leaves the sort out: the winners come out in a fixed order of their positions in the row (by the
// wave that loaded them, then by element index, then by lane: a function of the inputs only), for callers that use
// them as a set (gather + attention).
template <int EIN, bool SORTED>
__global__ __launch_bounds__(kTopkThreads) void pkv_topk_select_sort_kernel(
    const float *__restrict__ x, int64_t x_stride, const int64_t *__restrict__ ids, int64_t ids_stride, int len, int P,
    int64_t k, int64_t *__restrict__ out_ids, float *__restrict__ out_vals) {
  extern __shared__ uint64_t s_keys[];
  __shared__ uint32_t s_hist[2 * kLinBins];
  __shared__ uint32_t s_cnt[kLinBins];
  __shared__ uint32_t s_bcast[8];
  __shared__ uint32_t s_counter;
  __shared__ uint64_t s_bucket[kLinBucketMax];
  __shared__ uint64_t s_T;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float *xr = x + (int64_t)row * x_stride;
  const int64_t *ir = ids ? ids + (int64_t)row * ids_stride : nullptr;
  uint64_t v[EIN];
#pragma unroll
  for (int e = 0; e < EIN; ++e) {
    const int i = tid + e * kTopkThreads;
    v[e] = i < len ? make_key(xr, ir, i) : 0ull;
  }
  if (tid == 0) s_counter = 0;
  if (SORTED)
    for (int i = tid; i < (P < 1024 ? 1024 : P); i += kTopkThreads) s_keys[i] = 0ull;
  bool win[EIN];
  uint32_t bin[EIN];
  LinSel L;
  const bool lin = linear_bins<EIN>(v, (uint32_t)k, s_hist, s_cnt, s_bcast, bin, L);  // uniform over the workgroup
  int64_t *oi = out_ids + (int64_t)row * k;
  float *ov = out_vals ? out_vals + (int64_t)row * k : nullptr;
  if (SORTED && lin && L.max_winners <= kLinRankMax) {
    // counting sort: a key of a bin above b* takes a slot of [off[b], off[b] + count[b]) and the keys of b* go to
    // a list of their own; then every key counts the larger keys of its own bin, which is its place inside the
    // bin, and is written there (of b* only the first `need`)
    const uint32_t *s_off = s_hist + kLinBins;
#pragma unroll
    for (int e = 0; e < EIN; ++e) {
      if (v[e] != 0ull) {
        if (bin[e] > L.bstar) s_keys[atomicAdd(&s_cnt[bin[e]], 1u)] = v[e];
        else if (bin[e] == L.bstar) s_bucket[atomicAdd(&s_bcast[6], 1u)] = v[e];
      }
    }
    __syncthreads();
    const uint32_t n_above = (uint32_t)k - L.need;
    for (uint32_t p = tid; p < n_above; p += kTopkThreads) {
      const uint64_t key = s_keys[p];
      const uint32_t b = lin_bin(key, L);
      const uint32_t start = s_off[b], cnt = s_cnt[b] - start;
      uint32_t r = 0;
#pragma unroll 4
      for (uint32_t j = 0; j < cnt; ++j) r += s_keys[start + j] > key ? 1u : 0u;
      oi[start + r] = (int64_t)(uint32_t)(~(uint32_t)key);
      if (ov) ov[start + r] = pkv_from_ordered_u32((uint32_t)(key >> 32));
    }
    rank_bucket_desc(s_bucket, L.in_bstar, [&](uint64_t key, uint32_t r) {
      if (r < L.need) {
        oi[n_above + r] = (int64_t)(uint32_t)(~(uint32_t)key);
        if (ov) ov[n_above + r] = pkv_from_ordered_u32((uint32_t)(key >> 32));
      }
    });
    return;
  }
  if (!SORTED && lin) {
    // any order, without the threshold key: the keys of the bins above b* all win and take the first k - need slots
    // (slot = winners of the lower waves + winners of the own wave at lower e + those at the same e in lower lanes:
    // one ballot per e and one exchange of the 16 wave totals); the keys of b* are ranked among themselves and the
    // first `need` follow.  A fixed function of the inputs.
    uint64_t ballot[EIN];
    uint32_t wave_total = 0;
#pragma unroll
    for (int e = 0; e < EIN; ++e) {
      const bool nz = v[e] != 0ull;
      if (nz && bin[e] == L.bstar) s_bucket[atomicAdd(&s_bcast[6], 1u)] = v[e];
      ballot[e] = __ballot(nz && bin[e] > L.bstar);
      wave_total += (uint32_t)__popcll(ballot[e]);
    }
    const int wave = tid / PKV_WAVE;
    if (pkv_lane() == 0) s_hist[wave] = wave_total;  // the histograms have been read by everyone
    __syncthreads();
    uint32_t slot = 0;
#pragma unroll
    for (int w = 0; w < kTopkThreads / PKV_WAVE; ++w) slot += w < wave ? s_hist[w] : 0u;
    const uint64_t below = ((uint64_t)1 << pkv_lane()) - 1;
    const uint32_t n_above = (uint32_t)k - L.need;
#pragma unroll
    for (int e = 0; e < EIN; ++e) {
      const uint32_t mine = slot + (uint32_t)__popcll(ballot[e] & below);
      if (((ballot[e] >> pkv_lane()) & 1ull) && mine < n_above) {
        oi[mine] = (int64_t)(uint32_t)(~(uint32_t)v[e]);
        if (ov) ov[mine] = pkv_from_ordered_u32((uint32_t)(v[e] >> 32));
      }
      slot += (uint32_t)__popcll(ballot[e]);
    }
    rank_bucket_desc(s_bucket, L.in_bstar, [&](uint64_t key, uint32_t r) {
      if (r < L.need) {
        oi[n_above + r] = (int64_t)(uint32_t)(~(uint32_t)key);
        if (ov) ov[n_above + r] = pkv_from_ordered_u32((uint32_t)(key >> 32));
      }
    });
    return;
  }
  if (lin) {
    linear_threshold<EIN>(v, bin, s_bcast, s_bucket, &s_T, L);
#pragma unroll
    for (int e = 0; e < EIN; ++e) win[e] = v[e] != 0ull && (bin[e] > L.bstar || (bin[e] == L.bstar && v[e] >= L.T));
  } else {
    uint64_t prefix;
    int shift;
    radix_select_regs<EIN>(v, (uint32_t)k, s_hist, s_bcast, prefix, shift);
#pragma unroll
    for (int e = 0; e < EIN; ++e) win[e] = (v[e] >> shift) >= (prefix >> shift) && v[e] != 0ull;
  }
  if (!SORTED) {
    // slot of a winner = winners of the lower waves + winners of its own wave at lower e + those at its e in lower
    // lanes: a fixed function of the inputs, found with one ballot per e and one exchange of the 16 wave totals
    uint64_t ballot[EIN];
    uint32_t wave_total = 0;
#pragma unroll
    for (int e = 0; e < EIN; ++e) {
      ballot[e] = __ballot(win[e]);
      wave_total += (uint32_t)__popcll(ballot[e]);
    }
    __syncthreads();  // the histograms have been read by everyone: s_hist is free again
    const int wave = tid / PKV_WAVE;
    if (pkv_lane() == 0) s_hist[wave] = wave_total;
    __syncthreads();
    uint32_t slot = 0;
#pragma unroll
    for (int w = 0; w < kTopkThreads / PKV_WAVE; ++w) slot += w < wave ? s_hist[w] : 0u;
    const uint64_t below = ((uint64_t)1 << pkv_lane()) - 1;
#pragma unroll
    for (int e = 0; e < EIN; ++e) {
      const uint32_t mine = slot + (uint32_t)__popcll(ballot[e] & below);
      if (win[e] && mine < (uint32_t)k) {
        oi[mine] = (int64_t)(uint32_t)(~(uint32_t)v[e]);
        if (ov) ov[mine] = pkv_from_ordered_u32((uint32_t)(v[e] >> 32));
      }
      slot += (uint32_t)__popcll(ballot[e]);
    }
    return;
  }
#pragma unroll
  for (int e = 0; e < EIN; ++e) {
    const uint32_t slot = wave_take_slots(&s_counter, win[e]);
    if (win[e] && slot < (uint32_t)k) s_keys[slot] = v[e];
  }
  __syncthreads();
#define PKV_SORT_K(NT, E) sort_lds_keys_and_emit<NT, E>(s_keys, k, oi, ov, nullptr)
  PKV_DISPATCH_E(P, PKV_SORT_K);
#undef PKV_SORT_K
}

// ------------------------------------------------- rows wider than one workgroup
//
// More than 8192 keys in a row: the row is cut into slices of 8192 keys, one workgroup (8 keys per
// thread) each, and the k winners are found in three steps.
//   histogram  every slice adds bits [BINSHIFT, BINSHIFT+11) of its 64-bit keys to a 2048-bin
//              histogram of the row: in LDS first, then one global atomic per non-empty bin;
//   compact    every slice derives the threshold bin b* from the row histogram (the bin in which the
//              k-th largest key lies) and appends its keys above b* to list A (fewer than k in the
//              whole row) and its keys inside b* to list B, slots handed out by two row counters;
//   finish     one workgroup per row picks the k - |A| largest keys of list B exactly (radix select in
//              registers; streamed if B has more than 8192 keys) and sorts the k winners.
// Keys are distinct, so the order in which the lists are filled does not reach the result.
constexpr int kWideSlice = 8192;
constexpr int kWideBins = 2048;
constexpr int kWideCtlSlots = kWideBins + 8;
constexpr int kWideRowWords = kWideCtlSlots + 2 * kWideRangeSlots;  // per-row control block: histogram, |A|, |B|, range, range slots

struct ScoreKeys {  // key i of a row of scores with optional ids
  const float *x;
  const int64_t *ids;
  __device__ __forceinline__ uint64_t operator()(int64_t i) const { return make_key(x, ids, i); }
};

constexpr int kWideE = kWideSlice / kTopkThreads;  // keys per thread
constexpr int kWideCtlMax = kWideBins + 2;     // largest ordered score of the row (0 = not provided)
constexpr int kWideCtlMinInv = kWideBins + 3;  // ~(smallest ordered score): both grow under atomicMax from zero

// Bin (0 .. 2047) of a key of a wide row.  With the row's score range in its control block: 2048 even steps of
// [min, max] (non-decreasing in the score whatever the rounding, so a higher bin means a larger key), which keeps
// the threshold bin at about len / 2048 keys for any distribution without far outliers.  Without it, or where it
// does not apply (non-finite scores, a zero or subnormal range): bits [shift, shift + 11) of the key, which put
// scores that share their exponent into a handful of bins.
struct WideBinning {
  int shift;  // >= 0: fixed bit field; < 0: value bins
  float lo, scale;
  __device__ __forceinline__ uint32_t operator()(uint64_t key) const {
    if (shift >= 0) return (uint32_t)(key >> shift) & (kWideBins - 1);
    const float t = (pkv_from_ordered_u32((uint32_t)(key >> 32)) - lo) * scale;
    const uint32_t b = (uint32_t)t;
    return b > (uint32_t)(kWideBins - 1) ? (uint32_t)(kWideBins - 1) : b;
  }
};

// The same decision in every workgroup of every launch that bins the row: it depends only on the range words and
// the n_slots range slots a producer may have filled (every wave reduces them for itself: no barrier).
__device__ __forceinline__ WideBinning wide_binning(const uint32_t *__restrict__ ctl, int n_slots, int fallback_shift) {
  WideBinning bn;
  bn.shift = fallback_shift, bn.lo = 0.f, bn.scale = 0.f;
  uint32_t mx = ctl[kWideCtlMax], mi = ctl[kWideCtlMinInv];
  if (n_slots > 0) {
    for (int c = pkv_lane(); c < n_slots; c += PKV_WAVE) {
      const pkv_u32x2 sl = *(const pkv_u32x2 *)(ctl + kWideCtlSlots + 2 * c);
      mx = sl.x > mx ? sl.x : mx;
      mi = sl.y > mi ? sl.y : mi;
    }
#pragma unroll
    for (int x = 1; x < PKV_WAVE; x <<= 1) {
      const uint32_t a = (uint32_t)__shfl_xor((int)mx, x, PKV_WAVE), c = (uint32_t)__shfl_xor((int)mi, x, PKV_WAVE);
      mx = a > mx ? a : mx;
      mi = c > mi ? c : mi;
    }
  }
  const uint32_t mn = ~mi;
  const float hi = pkv_from_ordered_u32(mx), lo = pkv_from_ordered_u32(mn);
  const float range = hi - lo, scale = (float)kWideBins / range;
  const float inf = __uint_as_float(0x7f800000u);
  if (mx != 0u && mx < 0xff800000u && mn > 0x007fffffu && mn <= mx && range > 0.f && range < inf && scale < inf)
    bn.shift = -1, bn.lo = lo, bn.scale = scale;
  return bn;
}

// The slice's keys, element e of thread t = slice*8192 + e*1024 + t; 0 beyond the row's end.  The loads are
// unconditional (clamped index) so that all of them are in flight together.
template <typename KeyFn>
__device__ __forceinline__ void wide_load_keys(KeyFn key_of, int64_t len, int slice, uint64_t (&keys)[kWideE]) {
#pragma unroll
  for (int e = 0; e < kWideE; ++e) {
    const int64_t i = (int64_t)slice * kWideSlice + e * kTopkThreads + threadIdx.x;
    const uint64_t key = key_of(i < len ? i : len - 1);
    keys[e] = i < len ? key : 0ull;
  }
}

__device__ __forceinline__ void wide_hist_slice(const WideBinning &bn, const uint64_t (&keys)[kWideE], int64_t len,
                                                int slice, uint32_t *s_bins, uint32_t *__restrict__ g_hist) {
  const int tid = threadIdx.x;
  for (int b = tid; b < kWideBins; b += kTopkThreads) s_bins[b] = 0;
  __syncthreads();
#pragma unroll
  for (int e = 0; e < kWideE; ++e) {
    const int64_t i = (int64_t)slice * kWideSlice + e * kTopkThreads + tid;
    wave_hist_add(s_bins, bn(keys[e]), i < len, 1);
  }
  __syncthreads();
  for (int b = tid; b < kWideBins; b += kTopkThreads) {
    const uint32_t c = s_bins[b];
    if (c) atomicAdd(&g_hist[b], c);
  }
}

// s_tmp: 24 words.  ctl: the row's control block (histogram complete at launch).  Every workgroup
// reserves its share of both lists with one atomic each.
__device__ __forceinline__ void wide_compact_slice(const WideBinning &bn, const uint64_t (&keys)[kWideE], int64_t len,
                                                   int slice, uint32_t k, uint32_t *__restrict__ ctl,
                                                   uint64_t *__restrict__ list_a, uint64_t *__restrict__ list_b,
                                                   uint32_t *s_tmp) {
  const int tid = threadIdx.x;
  // thread t owns bins 2047 - 2t and 2046 - 2t: an exclusive scan over threads counts the keys in higher bins
  const uint32_t h0 = ctl[kWideBins - 1 - 2 * tid], h1 = ctl[kWideBins - 2 - 2 * tid];
  if (tid == 0) s_tmp[16] = 0;
  int total;
  uint32_t above = (uint32_t)pkv_block_excl_scan<kTopkThreads>((int)(h0 + h1), (int *)s_tmp, total);
  if (above < k && above + h0 >= k) s_tmp[16] = (uint32_t)(kWideBins - 1 - 2 * tid);
  above += h0;
  if (above < k && above + h1 >= k) s_tmp[16] = (uint32_t)(kWideBins - 2 - 2 * tid);
  __syncthreads();
  const uint32_t bstar = s_tmp[16];
  uint32_t in_a = 0, in_b = 0, n_a = 0, n_b = 0;  // bit e: key e goes to list A / B
#pragma unroll
  for (int e = 0; e < kWideE; ++e) {
    const int64_t i = (int64_t)slice * kWideSlice + e * kTopkThreads + tid;
    const uint32_t bin = bn(keys[e]);
    const bool a = i < len && bin > bstar, b = i < len && bin == bstar;
    in_a |= (uint32_t)a << e, in_b |= (uint32_t)b << e;
    n_a += a, n_b += b;
  }
  // both counts in one scan: a slice holds at most 8192 keys, so 16 bits each are enough
  const uint32_t excl = (uint32_t)pkv_block_excl_scan<kTopkThreads>((int)(n_a | (n_b << 16)), (int *)s_tmp, total);
  if (tid == 0) s_tmp[17] = atomicAdd(&ctl[kWideBins], (uint32_t)total & 0xffffu);
  if (tid == PKV_WAVE) s_tmp[18] = atomicAdd(&ctl[kWideBins + 1], (uint32_t)total >> 16);
  __syncthreads();
  uint32_t slot_a = s_tmp[17] + (excl & 0xffffu), slot_b = s_tmp[18] + (excl >> 16);
#pragma unroll
  for (int e = 0; e < kWideE; ++e) {
    if ((in_a >> e) & 1u) {
      if (slot_a < k) list_a[slot_a] = keys[e];
      ++slot_a;
    }
    if ((in_b >> e) & 1u) {
      if ((int64_t)slot_b < len) list_b[slot_b] = keys[e];
      ++slot_b;
    }
  }
}

// The k winners into s_keys[0 .. k) in any order (zero padded up to max(P, 1024)).  All 1024 threads.
__device__ __forceinline__ void wide_finish_select(uint32_t k, int P, const uint32_t *__restrict__ ctl,
                                                   const uint64_t *__restrict__ list_a,
                                                   const uint64_t *__restrict__ list_b, int64_t len, uint64_t *s_keys,
                                                   SelSmem &sm) {
  uint32_t *s_hist = sm.hist, *s_bcast = sm.bcast, *s_counter = &sm.counter;
  const int tid = threadIdx.x;
  uint32_t n_a = ctl[kWideBins], n_b = ctl[kWideBins + 1];
  if (n_a > k) n_a = k;  // cannot happen with a consistent histogram; keeps every index in range
  if ((int64_t)n_b > len) n_b = (uint32_t)len;
  const uint32_t need = k - n_a;
  for (int i = tid; i < (P < 1024 ? 1024 : P); i += kTopkThreads) s_keys[i] = (uint32_t)i < n_a ? list_a[i] : 0ull;
  if (tid == 0) *s_counter = n_a;
  __syncthreads();
  if (need == 0) return;
  if (n_b <= (uint32_t)kWideSlice) {
    uint64_t v[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t i = (uint32_t)(tid + e * kTopkThreads);
      v[e] = i < n_b ? list_b[i] : 0ull;
    }
    bool win[8];
    if (need < n_b) {
      select_topk_flags<8, true>(v, need, sm, win);  // list B shares its leading bits: bins of the remaining ones
    } else {  // all of B
#pragma unroll
      for (int e = 0; e < 8; ++e) win[e] = v[e] != 0ull;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t slot = wave_take_slots(s_counter, win[e]);
      if (win[e] && slot < k) s_keys[slot] = v[e];
    }
  } else {
    auto key_of = [&](int64_t i) { return list_b[i]; };
    uint64_t prefix;
    int shift;
    radix_select_streamed(key_of, (int64_t)n_b, need, s_hist, s_bcast, prefix, shift);
    collect_winners_streamed(key_of, (int64_t)n_b, k, prefix, shift, s_counter, s_keys);
  }
  __syncthreads();
}

// The same with the sort: the k winners sorted descending into s_keys[0 .. k) (zero padded up to max(P, 1024)) by
// one binning of list A and list B together; EA = max(P, 1024) / 1024 keys of list A per thread, s_tmp: k more keys.
// Both lists are requested before their lengths are known (clamped indices: one memory round trip, the unused
// entries are dropped afterwards).  False, with s_keys undefined, where that does not apply: wide_finish_select
// and a sort then do the same work in two steps.
template <int EA>
__device__ __forceinline__ bool wide_finish_select_sort(uint32_t k, int P, const uint32_t *__restrict__ ctl,
                                                        const uint64_t *__restrict__ list_a,
                                                        const uint64_t *__restrict__ list_b, int64_t len,
                                                        uint64_t *s_keys, uint64_t *s_tmp, SelSmem &sm) {
  const int tid = threadIdx.x;
  uint64_t v[EA + 8];
#pragma unroll
  for (int e = 0; e < EA; ++e) {
    const uint32_t i = (uint32_t)(tid + e * kTopkThreads);
    v[e] = list_a[i < k ? i : k - 1];
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int64_t i = tid + e * kTopkThreads;
    v[EA + e] = list_b[i < len ? i : len - 1];
  }
  const uint32_t n_a = ctl[kWideBins], n_b = ctl[kWideBins + 1];
  if (n_a > k || n_b > (uint32_t)kWideSlice || (int64_t)n_b > len || n_a + n_b < k) return false;
#pragma unroll
  for (int e = 0; e < EA; ++e) v[e] = (uint32_t)(tid + e * kTopkThreads) < n_a ? v[e] : 0ull;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[EA + e] = (uint32_t)(tid + e * kTopkThreads) < n_b ? v[EA + e] : 0ull;
  for (int i = tid; i < (P < 1024 ? 1024 : P); i += kTopkThreads) s_keys[i] = 0ull;
  return select_sort_desc<EA + 8>(v, k, s_tmp, s_keys, sm);
}

// Either way: true = s_keys is sorted already.  s_tmp: null when the second copy of the list is not set up.
__device__ __forceinline__ bool wide_finish_keys(uint32_t k, int P, const uint32_t *__restrict__ ctl,
                                                 const uint64_t *__restrict__ list_a,
                                                 const uint64_t *__restrict__ list_b, int64_t len, uint64_t *s_keys,
                                                 uint64_t *s_tmp, SelSmem &sm) {
  bool sorted = false;
  if (s_tmp) {
    sorted = P <= 1024 ? wide_finish_select_sort<1>(k, P, ctl, list_a, list_b, len, s_keys, s_tmp, sm)
                       : wide_finish_select_sort<2>(k, P, ctl, list_a, list_b, len, s_keys, s_tmp, sm);
    if (sorted) return true;
    __syncthreads();
  }
  wide_finish_select(k, P, ctl, list_a, list_b, len, s_keys, sm);
  return false;
}

// Largest and smallest ordered score of a workgroup's values into the row's control block.  slot < 0: the range
// words (both grow from zero under atomicMax: the minimum is kept complemented; ctl zero at launch); slot >= 0: that
// range slot, written plainly, no matter what it held.  s_red: 32 words.  All threads of the workgroup.
__device__ __forceinline__ void wide_range_out(uint32_t mx, uint32_t mn, uint32_t *__restrict__ rctl, int slot,
                                               uint32_t *s_red) {
#pragma unroll
  for (int x = 1; x < PKV_WAVE; x <<= 1) {
    const uint32_t a = (uint32_t)__shfl_xor((int)mx, x, PKV_WAVE), c = (uint32_t)__shfl_xor((int)mn, x, PKV_WAVE);
    mx = a > mx ? a : mx;
    mn = c < mn ? c : mn;
  }
  const int wave = threadIdx.x / PKV_WAVE, n_waves = (blockDim.x + PKV_WAVE - 1) / PKV_WAVE;
  if (pkv_lane() == 0) s_red[wave] = mx, s_red[16 + wave] = mn;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < n_waves; ++w) {
      mx = s_red[w] > mx ? s_red[w] : mx;
      mn = s_red[16 + w] < mn ? s_red[16 + w] : mn;
    }
    const bool any = mx >= mn;  // at least one value
    if (slot >= 0) {
      rctl[kWideCtlSlots + 2 * slot] = any ? mx : 0u;
      rctl[kWideCtlSlots + 2 * slot + 1] = any ? ~mn : 0u;
    } else if (any) {
      atomicMax(&rctl[kWideCtlMax], mx);
      atomicMax(&rctl[kWideCtlMinInv], ~mn);
    }
  }
}

// grid (slices, rows).  The rows' score ranges for the launches that follow.  own_slots = 0: ctl zero at launch, the
// ranges go to the range words.  own_slots = 1 (at most kWideRangeSlots slices): nothing is assumed about ctl; every
// slice fills its own range slot and the row's first slice clears the rest of the control block.
__global__ __launch_bounds__(kTopkThreads) void pkv_topk_wide_range_kernel(const float *__restrict__ x, int64_t x_stride,
                                                                           int64_t len, uint32_t *__restrict__ ctl,
                                                                           int own_slots) {
  __shared__ uint32_t s_red[32];
  const int row = blockIdx.y;
  const float *xr = x + (int64_t)row * x_stride;
  uint32_t *rctl = ctl + (int64_t)row * kWideRowWords;
  uint32_t mx = 0u, mn = 0xffffffffu;
#pragma unroll
  for (int e = 0; e < kWideE; ++e) {
    const int64_t i = (int64_t)blockIdx.x * kWideSlice + e * kTopkThreads + threadIdx.x;
    const uint32_t o = pkv_ordered_u32(xr[i < len ? i : len - 1]);
    mx = o > mx ? o : mx;
    mn = o < mn ? o : mn;
  }
  if (own_slots && blockIdx.x == 0) {
    for (int i = threadIdx.x; i < kWideRowWords; i += kTopkThreads)
      if (i < kWideCtlSlots || i >= kWideCtlSlots + 2 * (int)gridDim.x) rctl[i] = 0u;
  }
  wide_range_out(mx, mn, rctl, own_slots ? (int)blockIdx.x : -1, s_red);
}

// grid (slices, rows).  ctl: u32 [rows][kWideRowWords], zero at launch.
__global__ __launch_bounds__(kTopkThreads) void pkv_topk_wide_hist_kernel(const float *__restrict__ x, int64_t x_stride,
                                                                          const int64_t *__restrict__ ids,
                                                                          int64_t ids_stride, int64_t len,
                                                                          uint32_t *__restrict__ ctl, int n_range_slots) {
  __shared__ uint32_t s_bins[kWideBins];
  const int row = blockIdx.y;
  uint64_t keys[kWideE];
  wide_load_keys(ScoreKeys{x + (int64_t)row * x_stride, ids ? ids + (int64_t)row * ids_stride : nullptr}, len, blockIdx.x,
                 keys);
  wide_hist_slice(wide_binning(ctl + (int64_t)row * kWideRowWords, n_range_slots, 53), keys, len, blockIdx.x, s_bins,
                  ctl + (int64_t)row * kWideRowWords);
}

__global__ __launch_bounds__(kTopkThreads) void pkv_topk_wide_compact_kernel(
    const float *__restrict__ x, int64_t x_stride, const int64_t *__restrict__ ids, int64_t ids_stride, int64_t len,
    int64_t k, uint32_t *__restrict__ ctl, uint64_t *__restrict__ list_a, uint64_t *__restrict__ list_b,
    int n_range_slots) {
  __shared__ uint32_t s_tmp[24];
  const int row = blockIdx.y;
  uint64_t keys[kWideE];
  wide_load_keys(ScoreKeys{x + (int64_t)row * x_stride, ids ? ids + (int64_t)row * ids_stride : nullptr}, len, blockIdx.x,
                 keys);
  wide_compact_slice(wide_binning(ctl + (int64_t)row * kWideRowWords, n_range_slots, 53), keys, len, blockIdx.x, (uint32_t)k,
                     ctl + (int64_t)row * kWideRowWords, list_a + (int64_t)row * k,
                         list_b + (int64_t)row * len, s_tmp);
}

// grid rows; dynamic LDS lds_bytes_sort(P): the winners, and as many keys again for the counting sort when they fit.
__global__ __launch_bounds__(kTopkThreads) void pkv_topk_wide_finish_kernel(
    int64_t len, int P, int64_t k, const uint32_t *__restrict__ ctl, const uint64_t *__restrict__ list_a,
    const uint64_t *__restrict__ list_b, int64_t *__restrict__ out_ids, float *__restrict__ out_vals) {
  extern __shared__ uint64_t s_keys[];
  __shared__ SelSmem sm;
  uint64_t *s_tmp = P <= kCountingSortMaxP ? s_keys + (P < 1024 ? 1024 : P) : nullptr;
  const int row = blockIdx.x;
  const bool sorted = wide_finish_keys((uint32_t)k, P, ctl + (int64_t)row * kWideRowWords, list_a + (int64_t)row * k,
                                       list_b + (int64_t)row * len, len, s_keys, s_tmp, sm);
  int64_t *oi = out_ids + (int64_t)row * k;
  float *ov = out_vals ? out_vals + (int64_t)row * k : nullptr;
  if (!sorted) {
#define PKV_SORT_K(NT, E) sort_lds_keys_desc<NT, E>(s_keys, (uint32_t)k, s_tmp, sm)
    PKV_DISPATCH_E(P, PKV_SORT_K);
#undef PKV_SORT_K
  }
  for (int64_t i = threadIdx.x; i < k; i += kTopkThreads) {
    const uint64_t key = s_keys[i];
    oi[i] = (int64_t)(uint32_t)(~(uint32_t)key);
    if (ov) ov[i] = pkv_from_ordered_u32((uint32_t)(key >> 32));
  }
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

// Two sums, each in the order of block_tree_sum_1024, and the largest / smallest of two unsigned words, all in one
// pass (two barriers).  s_red: 64 words.  Every thread returns the same values.
struct AdkReduced {
  float sum_a, sum_b;
  uint32_t mx, mn;
};
__device__ __forceinline__ AdkReduced block_reduce_adk_1024(float a, float b, uint32_t mx, uint32_t mn, uint32_t *s_red) {
#pragma unroll
  for (int m = 1; m < PKV_WAVE; m <<= 1) {
    const float oa = __shfl_xor(a, m, PKV_WAVE), ob = __shfl_xor(b, m, PKV_WAVE);
    const uint32_t ox = (uint32_t)__shfl_xor((int)mx, m, PKV_WAVE), on = (uint32_t)__shfl_xor((int)mn, m, PKV_WAVE);
    a = a + oa, b = b + ob;
    mx = ox > mx ? ox : mx, mn = on < mn ? on : mn;
  }
  __syncthreads();
  if (pkv_lane() == 0) {
    const int w = threadIdx.x / PKV_WAVE;
    s_red[w] = __float_as_uint(a), s_red[16 + w] = __float_as_uint(b), s_red[32 + w] = mx, s_red[48 + w] = mn;
  }
  __syncthreads();
  float wa[16], wb[16];
  AdkReduced r;
  r.mx = 0u, r.mn = 0xffffffffu;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    wa[i] = __uint_as_float(s_red[i]), wb[i] = __uint_as_float(s_red[16 + i]);
    r.mx = s_red[32 + i] > r.mx ? s_red[32 + i] : r.mx;
    r.mn = s_red[48 + i] < r.mn ? s_red[48 + i] : r.mn;
  }
#pragma unroll
  for (int h = 1; h < 16; h <<= 1)
#pragma unroll
    for (int i = 0; i < 16; i += 2 * h) wa[i] = wa[i] + wa[i + h], wb[i] = wb[i] + wb[i + h];
  r.sum_a = wa[0], r.sum_b = wb[0];
  return r;
}

__device__ __forceinline__ float cand_logit(const void *__restrict__ scores, int dtype, float scale, int64_t i) {
  const float x = (dtype == PKV_DTYPE_BF16) ? pkv_bf16_bits_to_f32(((const uint16_t *)scores)[i])
                                            : ((const float *)scores)[i];
  return x * scale;
}

// Sum of x over the workgroup's 1024 lanes for one slice of at most 8192 elements whose per-lane partial
// sums are `acc`; slices are then added in slice order (the first slice is taken as is).
__device__ __forceinline__ float add_slice_sum(float total, bool first, float acc, float *s_part) {
  const float sl = block_tree_sum_1024(acc, s_part);
  return first ? sl : total + sl;
}

// sum_i expf(logit_i - g) * vnorm_i over the dense (sink/local) tokens, in slices of 8192.
__device__ __forceinline__ float dense_benefit_sum(const float *__restrict__ sll, const float *__restrict__ slv,
                                                   int64_t sl, float g, float *s_part) {
  float total = 0.f;
  bool first = true;
  for (int64_t s0 = 0; s0 < sl || first; s0 += kWideSlice) {
    float acc = 0.f;
#pragma unroll
    for (int e = 0; e < kWideSlice / kTopkThreads; ++e) {
      const int64_t i = s0 + e * kTopkThreads + threadIdx.x;
      if (i < sl) acc = acc + pkv_expf(sll[i] - g) * slv[i];
    }
    total = add_slice_sum(total, first, acc, s_part);
    first = false;
  }
  return total;
}

// Running sums of 64 values strictly left to right in fp32: lane l returns carry + v_0 + ... + v_l, added
// in that order.  The chain of dependent adds runs through the lanes: every step adds a lane's value to
// its lower neighbour's running sum (DPP wave_shr:1; lane 0 takes the carry), so after step s lanes
// 0..s hold their final sums.  All 64 lanes must be active.
__device__ __forceinline__ float wave_running_sum(float val, float carry) {
  float acc = val;
#pragma unroll
  for (int s = 0; s < PKV_WAVE; ++s) {
    const float below =
        __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(carry), __float_as_int(acc), 0x138, 0xf, 0xf, false));
    acc = below + val;
  }
  return acc;
}

// Smallest k <= k_out with sl_benefit + prefix_{k-1} >= tgt over the sorted keys in s_keys (k_out if the
// target is never reached).  prefix is the cumulative sum of the reference (adaptive_topk.py:300-303) in
// a fixed two-level order: blocks of 64 consecutive benefits are summed left to right, the block totals
// are summed left to right, prefix_i = (total of the earlier blocks) + (running sum inside the block).
// Benefits are not negative, so the prefixes never decrease: the first block whose last prefix reaches the
// target holds the answer.  Every wave runs the short second level for itself (no barrier for its result);
// the wave that owns that block finds the element.  All 1024 threads call it; k_out <= 8192.
// s_f: 128 floats, s_k: one word.
__device__ __forceinline__ int64_t first_k_reaching(const uint64_t *s_keys, int64_t k_out, float sl_benefit, float tgt,
                                                    float *s_f, uint32_t *s_k) {
  const int lane = pkv_lane(), wave = threadIdx.x / PKV_WAVE;
  const int n_blocks = (int)((k_out + PKV_WAVE - 1) / PKV_WAVE);  // <= 128; wave w owns blocks w, w+16, ...
  float *s_tot = s_f;
  float run[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int c = wave + 16 * j;
    run[j] = 0.f;
    if (c < n_blocks) {
      const int64_t i = (int64_t)c * PKV_WAVE + lane;
      run[j] = wave_running_sum(i < k_out ? pkv_from_ordered_u32((uint32_t)(s_keys[i] >> 32)) : 0.f, 0.f);
      if (lane == PKV_WAVE - 1) s_tot[c] = run[j];
    }
  }
  if (threadIdx.x == 0) *s_k = (uint32_t)k_out;
  __syncthreads();
  // second level: lane l of pass p holds block 64p + l; the chain of adds needs as many steps as there are blocks
  int cstar = -1;
  float before_star = 0.f, carry = 0.f;
  for (int base = 0; base < n_blocks && cstar < 0; base += PKV_WAVE) {
    const int c = base + lane, live = n_blocks - base < PKV_WAVE ? n_blocks - base : PKV_WAVE;
    const float val = c < n_blocks ? s_tot[c] : 0.f;
    float acc = val;
    for (int st = 0; st < live; ++st) {
      const float below =
          __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(carry), __float_as_int(acc), 0x138, 0xf, 0xf, false));
      acc = below + val;
    }
    const float before =
        __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(carry), __float_as_int(acc), 0x138, 0xf, 0xf, false));
    const uint64_t hit = __ballot(c < n_blocks && sl_benefit + acc >= tgt);
    if (hit) {
      const int l = __ffsll((long long)hit) - 1;
      cstar = base + l;
      before_star = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(before), l));
    }
    carry = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(acc), live - 1));
  }
  if (cstar >= 0 && (cstar & 15) == wave) {
    float mine = run[0];
#pragma unroll
    for (int j = 1; j < 8; ++j) mine = (cstar >> 4) == j ? run[j] : mine;
    const int64_t i = (int64_t)cstar * PKV_WAVE + lane;
    const uint64_t hit = __ballot(i < k_out && sl_benefit + (before_star + mine) >= tgt);
    if (lane == 0 && hit) *s_k = (uint32_t)(cstar * PKV_WAVE + __ffsll((long long)hit));
  }
  __syncthreads();
  return (int64_t)*s_k;
}

// Sum of the per-slice sums of a row in slice order, starting from the first.  `first` is ssum[lane] (0 beyond
// n_slices) as loaded by the caller's first wave ahead of time.  All 1024 threads call it (one barrier); s_out: 1 float.
__device__ __forceinline__ float combine_slices(const float *__restrict__ ssum, int n_slices, float first, float *s_out) {
  if (threadIdx.x < PKV_WAVE) {
    const int lane = pkv_lane();
    float carry = 0.f;
    for (int base = 0; base < n_slices; base += PKV_WAVE) {
      const int i = base + lane;
      const float acc = wave_running_sum(base == 0 ? first : (i < n_slices ? ssum[i] : 0.f), carry);
      carry = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(acc), PKV_WAVE - 1));
    }
    if (lane == 0) s_out[0] = carry;
  }
  __syncthreads();
  return s_out[0];
}

// Shared tail: s_keys[0 .. P) holds the k_out winners (zero padded; sorted descending already, or in any order).
// Sorts them where they are not, finds k, writes adaptive_k[row] and the candidate ids in benefit order.
// What the caller does with k right after the kernel, folded into it: the clamp to [k_min, k_max] (off when
// k_max <= 0) and the per-row key count row_keys[row] = row_keys_base + k that the attention kernel reads.
struct AdkClamp {
  int64_t k_min, k_max;
  int32_t *row_keys;
  int64_t row_keys_base;
};

__device__ __forceinline__ void adaptive_tail(uint64_t *s_keys, int P, int64_t k_out, float sl_benefit, float total,
                                              float threshold, const int64_t *__restrict__ ci, int64_t n_cand,
                                              int64_t *__restrict__ adaptive_k_row, int64_t *__restrict__ ids_row,
                                              AdkClamp cl, int row, SelSmem &sm, bool sorted) {
  if (!sorted) {
    uint64_t *s_tmp = P <= kCountingSortMaxP ? s_keys + (P < 1024 ? 1024 : P) : nullptr;
#define PKV_SORT_K(NT, E) sort_lds_keys_desc<NT, E>(s_keys, (uint32_t)k_out, s_tmp, sm)
    PKV_DISPATCH_E(P, PKV_SORT_K);
#undef PKV_SORT_K
  }
  float *s_f = (float *)sm.hist;
  uint32_t *s_k = &sm.counter;
  // the winners' ids do not depend on k: they are requested now and stored after the search for k
  int64_t id[kTopkMaxSort / kTopkThreads];
#pragma unroll
  for (int e = 0; e < kTopkMaxSort / kTopkThreads; ++e) {
    const int64_t i = threadIdx.x + e * kTopkThreads;
    id[e] = 0;
    if (i < k_out) {
      const uint32_t pos = ~(uint32_t)s_keys[i];
      if (pos < (uint64_t)n_cand) id[e] = ci[pos];
    }
  }
  int64_t k = 1;  // total <= 0: adaptive_topk.py:304-306
  if (total > 0.f) k = first_k_reaching(s_keys, k_out, sl_benefit, threshold * total, s_f, s_k);
  if (threadIdx.x == 0) {
    if (cl.k_max > 0) k = k < cl.k_min ? cl.k_min : (k > cl.k_max ? cl.k_max : k);
    *adaptive_k_row = k;
    if (cl.row_keys) cl.row_keys[row] = (int32_t)(cl.row_keys_base + k);
  }
#pragma unroll
  for (int e = 0; e < kTopkMaxSort / kTopkThreads; ++e) {
    const int64_t i = threadIdx.x + e * kTopkThreads;
    if (i < k_out) ids_row[i] = id[e];
  }
}

// Position in a row of the per-position value-norm table, kept inside the row whatever the candidate id says.
__device__ __forceinline__ int64_t vn_index(int64_t pos, int64_t row_len) {
  return pos < 0 ? 0 : (pos >= row_len ? row_len - 1 : pos);
}

struct AdkRow {  // one row's operands
  const float *sll, *slv;
  const char *cs;
  const int64_t *ci;
  const float *cv, *vn;
};

__device__ __forceinline__ AdkRow adk_row(int row, const float *sl_logits, int64_t sl_stride, const float *sl_vnorm,
                                          int64_t slv_stride, const void *cand_scores, int cand_dtype,
                                          const float *cand_vnorm, const float *value_norm, int64_t vn_stride,
                                          const int64_t *cand_ids, int64_t n_cand) {
  AdkRow r;
  r.sll = sl_logits + (int64_t)row * sl_stride;
  r.slv = sl_vnorm + (int64_t)row * slv_stride;
  r.cs = (const char *)cand_scores + (int64_t)row * n_cand * (cand_dtype == PKV_DTYPE_BF16 ? 2 : 4);
  r.ci = cand_ids + (int64_t)row * n_cand;
  r.cv = cand_vnorm ? cand_vnorm + (int64_t)row * n_cand : nullptr;
  r.vn = value_norm ? value_norm + (int64_t)row * vn_stride : nullptr;
  return r;
}

// n_cand <= 1024*EIN <= 8192: one workgroup per row, everything in registers.  Dynamic LDS P*8 bytes
// (P = pow2 >= k_out, at least 1024 keys).
template <int EIN>
__global__ __launch_bounds__(kTopkThreads) void pkv_adaptive_topk_kernel(
    const float *__restrict__ sl_logits, int64_t sl_stride, const float *__restrict__ sl_vnorm, int64_t slv_stride,
    int64_t sl, const void *__restrict__ cand_scores, int cand_dtype, float cand_scale,
    const float *__restrict__ cand_vnorm, const float *__restrict__ value_norm, int64_t vn_stride, int64_t vn_offset,
    int64_t vn_pos_stride, const int64_t *__restrict__ cand_ids, int n_cand, float threshold, int64_t k_out, int P,
    int64_t *__restrict__ adaptive_k, int64_t *__restrict__ topk_ids, AdkClamp cl) {
  extern __shared__ uint64_t s_keys[];
  __shared__ float s_part[16];
  __shared__ uint32_t s_red[64];
  __shared__ SelSmem sm;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const AdkRow r = adk_row(row, sl_logits, sl_stride, sl_vnorm, slv_stride, cand_scores, cand_dtype, cand_vnorm,
                           value_norm, vn_stride, cand_ids, n_cand);
  // candidate logits and value norms: element i = tid + e*1024, so a lane adds its elements in increasing i
  float logit[EIN], vnorm[EIN];
#pragma unroll
  for (int e = 0; e < EIN; ++e) {
    const int i = tid + e * kTopkThreads, ii = i < n_cand ? i : n_cand - 1;  // clamped: the loads carry no branch
    const float lg = cand_logit(r.cs, cand_dtype, cand_scale, ii);
    const float vv = r.cv ? r.cv[ii] : r.vn[vn_index(r.ci[ii] + vn_offset, vn_stride / vn_pos_stride) * vn_pos_stride];
    logit[e] = i < n_cand ? lg : -__uint_as_float(0x7f800000u);
    vnorm[e] = i < n_cand ? vv : 0.f;
  }
  // the first 2048 dense tokens stay in registers for the maximum and for their benefits
  constexpr int kDenseRegs = 2;
  float dl[kDenseRegs], dv[kDenseRegs];
#pragma unroll
  for (int e = 0; e < kDenseRegs; ++e) {
    const int64_t i = tid + e * kTopkThreads;
    dl[e] = -__uint_as_float(0x7f800000u), dv[e] = 0.f;
    if (i < sl) dl[e] = r.sll[i], dv[e] = r.slv[i];
  }
  float m = -__uint_as_float(0x7f800000u);
  for (int64_t i = tid + kDenseRegs * kTopkThreads; i < sl; i += kTopkThreads) m = fmaxf(m, r.sll[i]);
#pragma unroll
  for (int e = 0; e < kDenseRegs; ++e) m = fmaxf(m, dl[e]);
#pragma unroll
  for (int e = 0; e < EIN; ++e) m = fmaxf(m, logit[e]);
  const float g = block_max_1024(m, s_part);  // joint max (adaptive_topk.py:282-286)
  // benefits of the first slice of dense tokens (a lane adds its elements in increasing i, as dense_benefit_sum
  // does) and of the candidates; both sums and the range of the candidates' keys in one reduction
  float dacc = 0.f;
#pragma unroll
  for (int e = 0; e < kWideSlice / kTopkThreads; ++e) {
    const int64_t i = tid + e * kTopkThreads;
    if (i < sl) {
      const float x = e < kDenseRegs ? dl[e < kDenseRegs ? e : 0] : r.sll[i];
      const float w = e < kDenseRegs ? dv[e < kDenseRegs ? e : 0] : r.slv[i];
      dacc = dacc + pkv_expf(x - g) * w;
    }
  }
  uint64_t v[EIN];
  float acc = 0.f;
  uint32_t kmax = 0u, kmin = 0xffffffffu;
#pragma unroll
  for (int e = 0; e < EIN; ++e) {
    const int i = tid + e * kTopkThreads;
    const float b = i < n_cand ? pkv_expf(logit[e] - g) * vnorm[e] : 0.f;
    acc = acc + b;
    const uint32_t ob = pkv_ordered_u32(b);
    v[e] = i < n_cand ? (((uint64_t)ob << 32) | (uint64_t)(~(uint32_t)i)) : 0ull;
    if (i < n_cand) kmax = ob > kmax ? ob : kmax, kmin = ob < kmin ? ob : kmin;
  }
  const AdkReduced red = block_reduce_adk_1024(dacc, acc, kmax, kmin, s_red);
  float sl_benefit = red.sum_a;
  for (int64_t s0 = kWideSlice; s0 < sl; s0 += kWideSlice) {  // further slices of dense tokens, added in slice order
    float a2 = 0.f;
#pragma unroll
    for (int e = 0; e < kWideSlice / kTopkThreads; ++e) {
      const int64_t i = s0 + e * kTopkThreads + tid;
      if (i < sl) a2 = a2 + pkv_expf(r.sll[i] - g) * r.slv[i];
    }
    sl_benefit = add_slice_sum(sl_benefit, false, a2, s_part);
  }
  const float total = sl_benefit + red.sum_b;
  const uint32_t key_range[2] = {red.mx, red.mn};

  // the k_out largest (benefit, ~position) keys, sorted: in one binning where that applies (benefits span many
  // binades: bins of the key bits), else selected first and sorted afterwards
  if (tid == 0) sm.counter = 0;
  const int Pz = P < 1024 ? 1024 : P;
  for (int i = tid; i < Pz; i += kTopkThreads) s_keys[i] = 0ull;
  const bool sorted = P <= kCountingSortMaxP &&
                      select_sort_desc<EIN>(v, (uint32_t)k_out, s_keys + Pz, s_keys, sm, key_range);  // k_out <= n_cand
  if (!sorted) {
    bool win[EIN];
    if (k_out < n_cand) {
      select_topk_flags<EIN, true>(v, (uint32_t)k_out, sm, win);
    } else {
#pragma unroll
      for (int e = 0; e < EIN; ++e) win[e] = v[e] != 0ull;
      __syncthreads();
    }
#pragma unroll
    for (int e = 0; e < EIN; ++e) {
      const uint32_t slot = wave_take_slots(&sm.counter, win[e]);
      if (win[e] && slot < (uint32_t)k_out) s_keys[slot] = v[e];
    }
    __syncthreads();
  }
  adaptive_tail(s_keys, P, k_out, sl_benefit, total, threshold, r.ci, n_cand, adaptive_k + row,
                topk_ids + (int64_t)row * k_out, cl, row, sm, sorted);
}

// ---- n_cand > 8192: slices of 8192 candidates, one workgroup each ----
// Workspace per row: ben f32 [n_cand]; gathered norms f32 [n_cand]; partial maxima f32 [n_cand/2048];
// slice sums f32 [n_slices], then the sum over the dense tokens;
// control block u32 [kWideRowWords]; list A u64 [k_out]; list B u64 [n_cand].

struct BenefitKeys {  // key i = (benefit, ~position)
  const float *ben;
  __device__ __forceinline__ uint64_t operator()(int64_t i) const { return make_key(ben, nullptr, i); }
};

// grid (parts, rows) x 256 threads, 2048 candidates per workgroup: partial maxima of the logits (part 0 also
// covers the dense logits and clears the row's control block for the later launches) and, when the value
// norms come from the per-position table, the candidates' norms gathered into ws_vn.  The gather is a
// random 4-byte read per candidate and is bound by how many misses one CU keeps in flight, hence the
// small workgroups: they spread it over the whole chip.
constexpr int kAdkPart = 2048;
constexpr int kAdkPartThreads = 256;

__global__ __launch_bounds__(kAdkPartThreads) void pkv_adk_max_gather_kernel(
    const float *__restrict__ sl_logits, int64_t sl_stride, int64_t sl, const void *__restrict__ cand_scores,
    int cand_dtype, float cand_scale, const float *__restrict__ value_norm, int64_t vn_stride, int64_t vn_offset,
    int64_t vn_pos_stride, const int64_t *__restrict__ cand_ids, int64_t n_cand, float *__restrict__ ws_max,
    float *__restrict__ ws_vn,
    uint32_t *__restrict__ ctl) {
  __shared__ float s_part[kAdkPartThreads / PKV_WAVE];
  const int row = blockIdx.y, part = blockIdx.x, tid = threadIdx.x;
  const char *cs = (const char *)cand_scores + (int64_t)row * n_cand * (cand_dtype == PKV_DTYPE_BF16 ? 2 : 4);
  constexpr int E = kAdkPart / kAdkPartThreads;
  if (value_norm) {
    const int64_t *ci = cand_ids + (int64_t)row * n_cand;
    const float *vn = value_norm + (int64_t)row * vn_stride;
    float vv[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int64_t i = (int64_t)part * kAdkPart + e * kAdkPartThreads + tid;
      vv[e] = vn[vn_index(ci[i < n_cand ? i : n_cand - 1] + vn_offset, vn_stride / vn_pos_stride) * vn_pos_stride];
    }
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int64_t i = (int64_t)part * kAdkPart + e * kAdkPartThreads + tid;
      if (i < n_cand) ws_vn[(int64_t)row * n_cand + i] = vv[e];
    }
  }
  float m = -__uint_as_float(0x7f800000u);
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int64_t i = (int64_t)part * kAdkPart + e * kAdkPartThreads + tid;
    const float lg = cand_logit(cs, cand_dtype, cand_scale, i < n_cand ? i : n_cand - 1);
    m = fmaxf(m, lg);  // a clamped index repeats the row's last candidate: harmless for a maximum
  }
  if (part == 0) {
    const float *sll = sl_logits + (int64_t)row * sl_stride;
    for (int64_t i = tid; i < sl; i += kAdkPartThreads) m = fmaxf(m, sll[i]);
    for (int i = tid; i < kWideRowWords; i += kAdkPartThreads) ctl[(int64_t)row * kWideRowWords + i] = 0;
  }
#pragma unroll
  for (int x = 1; x < PKV_WAVE; x <<= 1) m = fmaxf(m, __shfl_xor(m, x, PKV_WAVE));
  if (pkv_lane() == 0) s_part[tid / PKV_WAVE] = m;
  __syncthreads();
  if (tid == 0) {
#pragma unroll
    for (int w = 1; w < kAdkPartThreads / PKV_WAVE; ++w) m = fmaxf(m, s_part[w]);
    ws_max[(int64_t)row * gridDim.x + part] = m;
  }
}

// grid (slices + 1, rows) x 1024: benefits of the slice into ws_ben, their sum (lane order, then the 1024-lane tree)
// into ws_sum, and their top key bits into the row histogram; one more workgroup per row sums the benefits of the
// dense tokens meanwhile.
__global__ __launch_bounds__(kTopkThreads) void pkv_adk_benefit_kernel(
    const float *__restrict__ sl_logits, int64_t sl_stride, const float *__restrict__ sl_vnorm, int64_t slv_stride,
    int64_t sl, const void *__restrict__ cand_scores, int cand_dtype, float cand_scale,
    const float *__restrict__ cand_vnorm, int64_t n_cand, const float *__restrict__ ws_max, int n_parts,
    float *__restrict__ ws_ben, float *__restrict__ ws_sum, uint32_t *__restrict__ ctl) {
  __shared__ float s_part[16];
  __shared__ uint32_t s_bins[kWideBins];
  const int row = blockIdx.y, slice = blockIdx.x, tid = threadIdx.x, n_slices = gridDim.x - 1;
  const char *cs = (const char *)cand_scores + (int64_t)row * n_cand * (cand_dtype == PKV_DTYPE_BF16 ? 2 : 4);
  const float *cv = cand_vnorm + (int64_t)row * n_cand;  // the caller's, or the ones gathered by the first launch
  float *ben = ws_ben + (int64_t)row * n_cand;
  float g = -__uint_as_float(0x7f800000u);
  for (int w = tid & (PKV_WAVE - 1); w < n_parts; w += PKV_WAVE) g = fmaxf(g, ws_max[(int64_t)row * n_parts + w]);
#pragma unroll
  for (int x = 1; x < PKV_WAVE; x <<= 1) g = fmaxf(g, __shfl_xor(g, x, PKV_WAVE));
  if (slice == n_slices) {  // the row's last workgroup: the dense tokens' benefit, kept after the slice sums
    const float d = dense_benefit_sum(sl_logits + (int64_t)row * sl_stride, sl_vnorm + (int64_t)row * slv_stride, sl, g,
                                      s_part);
    if (tid == 0) ws_sum[(int64_t)row * (n_slices + 1) + n_slices] = d;
    return;
  }
  float lg[kWideE], vv[kWideE];
#pragma unroll
  for (int e = 0; e < kWideE; ++e) {
    const int64_t i = (int64_t)slice * kWideSlice + e * kTopkThreads + tid, ii = i < n_cand ? i : n_cand - 1;
    lg[e] = cand_logit(cs, cand_dtype, cand_scale, ii);
    vv[e] = cv[ii];
  }
  float acc = 0.f;
  uint64_t keys[kWideE];
#pragma unroll
  for (int e = 0; e < kWideE; ++e) {
    const int64_t i = (int64_t)slice * kWideSlice + e * kTopkThreads + tid;
    const float b = pkv_expf(lg[e] - g) * vv[e];
    keys[e] = 0ull;
    if (i < n_cand) {
      ben[i] = b;
      acc = acc + b;
      keys[e] = ((uint64_t)pkv_ordered_u32(b) << 32) | (uint64_t)(~(uint32_t)i);
    }
  }
  const float ssum = block_tree_sum_1024(acc, s_part);
  if (tid == 0) ws_sum[(int64_t)row * (n_slices + 1) + slice] = ssum;
  wide_hist_slice(WideBinning{52, 0.f, 0.f}, keys, n_cand, slice, s_bins, ctl + (int64_t)row * kWideRowWords);
}

__global__ __launch_bounds__(kTopkThreads) void pkv_adk_compact_kernel(const float *__restrict__ ws_ben, int64_t n_cand,
                                                                       int64_t k_out, uint32_t *__restrict__ ctl,
                                                                       uint64_t *__restrict__ list_a,
                                                                       uint64_t *__restrict__ list_b) {
  __shared__ uint32_t s_tmp[24];
  const int row = blockIdx.y;
  uint64_t keys[kWideE];
  wide_load_keys(BenefitKeys{ws_ben + (int64_t)row * n_cand}, n_cand, blockIdx.x, keys);
  wide_compact_slice(WideBinning{52, 0.f, 0.f}, keys, n_cand, blockIdx.x, (uint32_t)k_out,
                         ctl + (int64_t)row * kWideRowWords, list_a + (int64_t)row * k_out,
                         list_b + (int64_t)row * n_cand, s_tmp);
}

// grid rows; dynamic LDS: lds_bytes_sort(P).
__global__ __launch_bounds__(kTopkThreads) void pkv_adk_finish_kernel(
    const int64_t *__restrict__ cand_ids, int64_t n_cand, int n_slices, float threshold, int64_t k_out, int P,
    const float *__restrict__ ws_sum, const uint32_t *__restrict__ ctl, const uint64_t *__restrict__ list_a,
    const uint64_t *__restrict__ list_b, int64_t *__restrict__ adaptive_k, int64_t *__restrict__ topk_ids, AdkClamp cl) {
  extern __shared__ uint64_t s_keys[];
  __shared__ float s_part[16];
  __shared__ SelSmem sm;
  const int row = blockIdx.x;
  // the sums left by the benefit launch are requested now and added up after the selection
  const float *ss = ws_sum + (int64_t)row * (n_slices + 1);
  const int lane = pkv_lane();
  const float first = lane < n_slices ? ss[lane] : 0.f;
  const float sl_benefit = ss[n_slices];
  uint64_t *s_tmp = P <= kCountingSortMaxP ? s_keys + (P < 1024 ? 1024 : P) : nullptr;
  const bool sorted = wide_finish_keys((uint32_t)k_out, P, ctl + (int64_t)row * kWideRowWords,
                                       list_a + (int64_t)row * k_out, list_b + (int64_t)row * n_cand, n_cand, s_keys,
                                       s_tmp, sm);
  const float total = sl_benefit + combine_slices(ss, n_slices, first, s_part);
  adaptive_tail(s_keys, P, k_out, sl_benefit, total, threshold, cand_ids + (int64_t)row * n_cand, n_cand,
                adaptive_k + row, topk_ids + (int64_t)row * k_out, cl, row, sm, sorted);
}

// uniform_k[r] = max over all rows of adaptive_k, row_keys[r] = base + that maximum: the dense form of the
// adaptive-k step, where every row keeps as many ids as the greediest one
// (polar_cache_atten_value_indices_adaptive_k.py:1462-1499 sizes its gather and attention by max(adaptive_k)).
// One workgroup of 1024 threads.
__global__ __launch_bounds__(kTopkThreads) void pkv_uniform_k_kernel(const int64_t *__restrict__ adaptive_k, int rows,
                                                                    int64_t *__restrict__ uniform_k,
                                                                    int32_t *__restrict__ row_keys, int64_t base) {
  __shared__ int64_t s_max[kTopkThreads / PKV_WAVE];
  int64_t m = 0;
  for (int r = threadIdx.x; r < rows; r += kTopkThreads) m = adaptive_k[r] > m ? adaptive_k[r] : m;
#pragma unroll
  for (int o = PKV_WAVE / 2; o > 0; o >>= 1) {
    const int64_t other = __shfl_xor(m, o, PKV_WAVE);
    m = other > m ? other : m;
  }
  if (pkv_lane() == 0) s_max[threadIdx.x / PKV_WAVE] = m;
  __syncthreads();
  m = s_max[0];
#pragma unroll
  for (int w = 1; w < kTopkThreads / PKV_WAVE; ++w) m = s_max[w] > m ? s_max[w] : m;
  for (int r = threadIdx.x; r < rows; r += kTopkThreads) {
    uniform_k[r] = m;
    if (row_keys) row_keys[r] = (int32_t)(base + m);
  }
}

// Logits of the dense (sink / local / buffer) rows against the group-mean query
// (polar_cache_adaptivek_varlen.py:1418-1419, :1731): out[(b,h)][r] = dtype(mean_g q . K[r]) widened to fp32,
// times scale.  16 lanes per key row, 8 dims per lane: a lane adds its 8 products in order, the 16 partial
// sums meet in a pairwise tree (lane ^ 1, 2, 4, 8).  grid (ceil(n_rows / 16), bs * H) x 256 threads.
constexpr int kDenseLogitThreads = 256;

template <bool BF16>
__global__ __launch_bounds__(kDenseLogitThreads) void pkv_dense_logits_kernel(
    const void *__restrict__ q, int n_kv_heads, int group, const void *__restrict__ k, int64_t k_stride_b,
    int64_t k_stride_h, int64_t n_rows, float scale, float *__restrict__ out, int64_t out_stride) {
  const int bh = blockIdx.y, b = bh / n_kv_heads, h = bh % n_kv_heads;
  const int s = threadIdx.x & 15;
  const int64_t row = (int64_t)blockIdx.x * (kDenseLogitThreads / 16) + (threadIdx.x >> 4);
  float qa[8];
  pkv_query_group_mean_t<BF16>(q, b, h, n_kv_heads, group, qa);
  const int64_t r = row < n_rows ? row : n_rows - 1;
  const int64_t at = (int64_t)b * k_stride_b + (int64_t)h * k_stride_h + r * 128 + 8 * s;
  float kv[8];
  if (BF16) {
    const pkv_u32x4 w = *(const pkv_u32x4 *)((const uint16_t *)k + at);
    const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      kv[2 * p] = __uint_as_float(ww[p] << 16);
      kv[2 * p + 1] = __uint_as_float(ww[p] & 0xffff0000u);
    }
  } else {
    const float4 lo = *(const float4 *)((const float *)k + at), hi = *(const float4 *)((const float *)k + at + 4);
    kv[0] = lo.x, kv[1] = lo.y, kv[2] = lo.z, kv[3] = lo.w, kv[4] = hi.x, kv[5] = hi.y, kv[6] = hi.z, kv[7] = hi.w;
  }
  float acc = qa[0] * kv[0];
#pragma unroll
  for (int j = 1; j < 8; ++j) acc = acc + qa[j] * kv[j];
  acc = acc + pkv_lane_xor_f<1>(acc);
  acc = acc + pkv_lane_xor_f<2>(acc);
  acc = acc + pkv_lane_xor_f<4>(acc);
  acc = acc + pkv_lane_xor_f<8>(acc);
  if (s == 0 && row < n_rows)
    out[(int64_t)bh * out_stride + row] = pkv_rdt(acc, BF16 ? PKV_DTYPE_BF16 : PKV_DTYPE_F32) * scale;
}

static size_t lds_bytes(int P) { return (size_t)(P < 1024 ? 1024 : P) * 8; }
// with room for the counting sort's second copy of the winners where the kernels use it
static size_t lds_bytes_sort(int P) { return lds_bytes(P) * (P <= kCountingSortMaxP ? 2 : 1); }

static int pow2_ceil(int64_t v) {
  int p = 1;
  while (p < v) p <<= 1;
  return p;
}

}  // namespace

int pkv_launch_select(const uint8_t *cnt_u8, int64_t cnt_stride, const uint32_t *row_suf, const uint16_t *chunk_suf,
                      int chunk_keys, int rows,
                      int64_t n_keys, int64_t k, int64_t *out, hipStream_t s) {
  PKV_REQUIRE(k >= 1 && k < n_keys, "select needs 1 <= k < n_keys (k=%lld n=%lld)", (long long)k,
              (long long)n_keys);
  PKV_REQUIRE(cnt_stride % 16 == 0 && cnt_stride >= n_keys && pkv_aligned(cnt_u8, 16),
              "count rows must be 16-byte aligned and padded");
  const int64_t n_chunks = (n_keys + chunk_keys - 1) / chunk_keys;
  dim3 grid((unsigned)n_chunks, (unsigned)rows);
  hipLaunchKernelGGL(pkv_select_kernel, grid, dim3(kSelThreads), 0, s, cnt_u8, cnt_stride, row_suf, chunk_suf, chunk_keys,
                     n_keys, k, out);
  PKV_LAUNCH_CHECK("pkv_select_kernel");
  return PKV_OK;
}

int pkv_launch_select_rerank(const uint8_t *cnt_u8, int64_t cnt_stride, const uint32_t *row_suf,
                             const uint16_t *chunk_suf, int chunk_keys, int bs,
                             int n_kv_heads, int64_t n_keys, int64_t k, const uint8_t *nib, int64_t ns_b, int64_t ns_h,
                             int64_t ns_key, const uint16_t *weight, int64_t ws_b, int64_t ws_h, int64_t ws_key,
                             const float *qhat, const float *qnorm, const float *centers, int64_t *cand, float *scores,
                             hipStream_t s, int64_t extra_off, float *extra_out, uint32_t *range_slots,
                             int64_t range_row_stride, int sub_blocks) {
  PKV_REQUIRE(!extra_out || (extra_off >= 0 && extra_off % 4 == 0 && extra_off + 4 <= ns_key),
              "the extra word must lie inside the key's record (offset %lld, record %lld bytes)", (long long)extra_off,
              (long long)ns_key);
  PKV_REQUIRE(k >= 1 && k < n_keys && k < ((int64_t)1 << 31), "select needs 1 <= k < n_keys (k=%lld n=%lld)", (long long)k,
              (long long)n_keys);
  PKV_REQUIRE(cnt_stride % 16 == 0 && cnt_stride >= n_keys && pkv_aligned(cnt_u8, 16),
              "count rows must be 16-byte aligned and padded");
  PKV_REQUIRE(pkv_aligned(nib, 16) && pkv_aligned(weight, 16) && ns_b % 16 == 0 && ns_h % 16 == 0 && ws_b % 8 == 0 &&
                  ws_h % 8 == 0 && ns_key >= 64 && ns_key % 16 == 0 && ws_key >= 16 && ws_key % 8 == 0 &&
                  ns_key < (1 << 20) && ws_key < (1 << 20),
              "key-major nibbles / weights must be 16-byte aligned, 64 bytes / 16 weights per key");
  const int64_t n_chunks = (n_keys + chunk_keys - 1) / chunk_keys;
  dim3 grid((unsigned)n_chunks, (unsigned)(bs * n_kv_heads));
  if (sub_blocks > 1) {
    const int piece_keys = chunk_keys / sub_blocks;
    PKV_REQUIRE(sub_blocks % 2 == 0 && chunk_keys % sub_blocks == 0 && piece_keys % 16 == 0 && 2 * piece_keys <= kSelKeysPerIter &&
                    n_chunks * sub_blocks <= kSelMaxPieces,
                "select + rerank: %d pieces of a %d-key chunk, %lld chunks per row not supported", sub_blocks, chunk_keys,
                (long long)n_chunks);
    hipLaunchKernelGGL(pkv_select_rerank_pieces_kernel, grid, dim3(kSelThreads), 0, s, cnt_u8, cnt_stride, row_suf, chunk_suf,
                       piece_keys, sub_blocks, n_kv_heads, n_keys, k, nib, ns_b, ns_h, (int)ns_key, weight, ws_b, ws_h,
                       (int)ws_key, qhat, qnorm, centers, cand, scores, (int)extra_off, extra_out, range_slots,
                       range_row_stride);
    PKV_LAUNCH_CHECK("pkv_select_rerank_pieces_kernel");
    return PKV_OK;
  }
  hipLaunchKernelGGL(pkv_select_rerank_kernel, grid, dim3(kSelThreads), 0, s, cnt_u8, cnt_stride, row_suf, chunk_suf,
                     chunk_keys,
                     n_kv_heads, n_keys, k, nib, ns_b, ns_h, (int)ns_key, weight, ws_b, ws_h, (int)ws_key, qhat, qnorm,
                     centers, cand, scores, (int)extra_off, extra_out,
                     range_slots, range_row_stride);
  PKV_LAUNCH_CHECK("pkv_select_rerank_kernel");
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
                             size_t &off_row, size_t &total) {
  chunk_keys = pkv_pick_chunk_keys(rows, len);
  cnt_stride = (int64_t)pkv_align_up((size_t)len, 16);
  const int64_t n_chunks = (len + chunk_keys - 1) / chunk_keys;
  off_hist = pkv_align_up((size_t)rows * (size_t)cnt_stride, 256);
  off_row = off_hist + pkv_align_up((size_t)rows * (size_t)n_chunks * 128 * sizeof(uint16_t), 256);
  total = off_row + pkv_align_up((size_t)rows * 128 * sizeof(uint32_t), 256);
}

extern "C" size_t pkv_bucket_topk_ws_bytes(int rows, int64_t len) {
  if (rows <= 0 || len <= 0) return 256;
  int ck;
  int64_t cs;
  size_t oh, orow, tot;
  bucket_ws_layout(rows, len, ck, cs, oh, orow, tot);
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
  size_t oh, orow, tot;
  bucket_ws_layout(rows, len, ck, cs, oh, orow, tot);
  if (!ws || ws_bytes < tot || !pkv_aligned(ws, 256)) {
    pkv_set_error("pkv_bucket_topk: workspace of %zu bytes (256-aligned) required, got %zu", tot, ws_bytes);
    return PKV_ENOMEM;
  }
  uint8_t *cnt = (uint8_t *)ws;
  uint16_t *hist = (uint16_t *)((char *)ws + oh);
  uint32_t *row_suf = (uint32_t *)((char *)ws + orow);
  const int64_t n_chunks = (len + ck - 1) / ck;
  // two launches: counts -> clamped bytes + chunk suffix histograms, then the select, which adds the chunks'
  // histograms up for the row totals itself (no atomics, so nothing has to be cleared first)
  (void)row_suf;
  hipLaunchKernelGGL(pkv_counts_to_u8_kernel, dim3((unsigned)n_chunks, (unsigned)rows), dim3(256), 0, s, x, x_stride,
                     len, cnt, cs, (uint32_t *)nullptr, hist, ck);
  PKV_LAUNCH_CHECK("pkv_counts_to_u8_kernel");
  return pkv_launch_select(cnt, cs, nullptr, hist, ck, rows, len, k, out, s);
}

// Wide rows (len > 8192): control blocks, list A [rows][k], list B [rows][len].
struct WideWs {
  size_t ctl, list_a, list_b, total;
};
static WideWs wide_ws_layout(int rows, int64_t len, int64_t k, size_t off) {
  WideWs w;
  w.ctl = off = pkv_align_up(off, 256);
  off += (size_t)rows * kWideRowWords * sizeof(uint32_t);
  w.list_a = off = pkv_align_up(off, 256);
  off += (size_t)rows * (size_t)k * sizeof(uint64_t);
  w.list_b = off = pkv_align_up(off, 256);
  off += (size_t)rows * (size_t)len * sizeof(uint64_t);
  w.total = pkv_align_up(off, 256);
  return w;
}

// Words at the start of pkv_topk_f32's workspace that must be zero when its first launch starts (0: none).
// (Handing the range to the one-workgroup kernel as well was measured: its min/max pass is cheaper than the
// producer's extra epilogue, +0.6 us on the step at 32 rows x 4096 candidates.)
int64_t pkv_topk_ctl_words(int rows, int64_t len) { return len > kTopkMaxSort ? (int64_t)rows * kWideRowWords : 0; }
// Where a producer's workgroups leave their (max, ~min) in that area, and the distance between rows in words.
uint32_t *pkv_topk_range_slots(uint32_t *ctl, int64_t len, int64_t *row_stride) {
  (void)len;
  *row_stride = (int64_t)kWideRowWords;
  return ctl + kWideCtlSlots;
}

size_t pkv_topk_ws_bytes_impl(int rows, int64_t len, int64_t k) {
  if (rows <= 0 || len <= kTopkMaxSort || k <= 0) return 256;
  return wide_ws_layout(rows, len, k, 0).total;
}

extern "C" size_t pkv_topk_f32_ws_bytes(int rows, int64_t len, int64_t k) {
  return pkv_topk_ws_bytes_impl(rows, len, k);
}

int pkv_launch_topk_f32(const float *x, int64_t x_stride, const int64_t *ids, int64_t ids_stride, int rows,
                        int64_t len, int64_t k, int64_t *out_ids, float *out_vals, void *ws, size_t ws_bytes,
                        hipStream_t s, bool any_order, bool ctl_ready) {
  PKV_REQUIRE(x && out_ids, "pkv_topk_f32: null pointer");
  PKV_REQUIRE(k > 0, "k must be positive");
  PKV_REQUIRE(k <= len, "k cannot exceed sequence length");
  PKV_REQUIRE(rows > 0 && rows <= 65535 && len < ((int64_t)1 << 31), "bad shape rows=%d len=%lld", rows, (long long)len);
  if (len <= kTopkMaxSort && pow2_ceil(k) * 2 <= pow2_ceil(len) && pow2_ceil(len) >= 2048) {
    const int P = pow2_ceil(k);
    const int ein = pow2_ceil(len) / kTopkThreads;
#define PKV_SEL(EIN, SORTED)                                                                                      \
  hipLaunchKernelGGL((pkv_topk_select_sort_kernel<EIN, SORTED>), dim3((unsigned)rows), dim3(kTopkThreads),        \
                     lds_bytes(P), s, x, x_stride, ids, ids_stride, (int)len, P, k, out_ids, out_vals)
#define PKV_SEL_E(SORTED)             \
  do {                                \
    if (ein <= 2) PKV_SEL(2, SORTED); \
    else if (ein == 4) PKV_SEL(4, SORTED); \
    else PKV_SEL(8, SORTED);          \
  } while (0)
    if (any_order) PKV_SEL_E(false); else PKV_SEL_E(true);
#undef PKV_SEL_E
#undef PKV_SEL
    PKV_LAUNCH_CHECK("pkv_topk_select_sort_kernel");
  } else if (len <= kTopkMaxSort) {
    const int P = pow2_ceil(len);
    hipLaunchKernelGGL(pkv_topk_sort_kernel, dim3((unsigned)rows), dim3(kTopkThreads), lds_bytes(P), s, x, x_stride,
                       ids, ids_stride, (int)len, P, k, out_ids, out_vals);
    PKV_LAUNCH_CHECK("pkv_topk_sort_kernel");
  } else {
    PKV_REQUIRE(k <= kTopkMaxSort, "k up to %d supported when len > %d (got %lld)", kTopkMaxSort, kTopkMaxSort,
                (long long)k);
    const size_t need = pkv_topk_ws_bytes_impl(rows, len, k);
    if (!ws || ws_bytes < need || !pkv_aligned(ws, 256)) {
      pkv_set_error("pkv_topk_f32: rows of more than %d keys need a workspace of %zu bytes (256-aligned), got %zu",
                    kTopkMaxSort, need, ws_bytes);
      return PKV_ENOMEM;
    }
    const WideWs w = wide_ws_layout(rows, len, k, 0);
    uint32_t *ctl = (uint32_t *)((char *)ws + w.ctl);
    uint64_t *list_a = (uint64_t *)((char *)ws + w.list_a), *list_b = (uint64_t *)((char *)ws + w.list_b);
    const int P = pow2_ceil(k);
    const dim3 grid((unsigned)((len + kWideSlice - 1) / kWideSlice), (unsigned)rows);
    // a row of at most kWideRangeSlots slices: every slice leaves its range in a slot of its own and the first one
    // clears the control block, which saves the clearing launch
    const bool own_slots = !ctl_ready && grid.x <= (unsigned)kWideRangeSlots;
    if (!ctl_ready) {  // else: earlier launches of the caller's step cleared the control blocks and left the rows' score ranges
      if (!own_slots) {
        hipLaunchKernelGGL(pkv_zero_u32_kernel, dim3((unsigned)((rows * kWideRowWords + 255) / 256)), dim3(256), 0, s,
                           ctl, (int64_t)rows * kWideRowWords);
        PKV_LAUNCH_CHECK("pkv_zero_u32_kernel");
      }
      hipLaunchKernelGGL(pkv_topk_wide_range_kernel, grid, dim3(kTopkThreads), 0, s, x, x_stride, len, ctl,
                         own_slots ? 1 : 0);
      PKV_LAUNCH_CHECK("pkv_topk_wide_range_kernel");
    }
    const int n_range_slots = (ctl_ready || own_slots) ? kWideRangeSlots : 0;  // per-workgroup score ranges
    hipLaunchKernelGGL(pkv_topk_wide_hist_kernel, grid, dim3(kTopkThreads), 0, s, x, x_stride, ids, ids_stride, len, ctl,
                       n_range_slots);
    PKV_LAUNCH_CHECK("pkv_topk_wide_hist_kernel");
    hipLaunchKernelGGL(pkv_topk_wide_compact_kernel, grid, dim3(kTopkThreads), 0, s, x, x_stride, ids, ids_stride, len, k,
                       ctl, list_a, list_b, n_range_slots);
    PKV_LAUNCH_CHECK("pkv_topk_wide_compact_kernel");
    hipLaunchKernelGGL(pkv_topk_wide_finish_kernel, dim3((unsigned)rows), dim3(kTopkThreads), lds_bytes_sort(P), s, len, P, k,
                       ctl, list_a, list_b, out_ids, out_vals);
    PKV_LAUNCH_CHECK("pkv_topk_wide_finish_kernel");
  }
  return PKV_OK;
}

extern "C" int pkv_topk_f32(const float *x, int64_t x_stride, const int64_t *ids, int64_t ids_stride, int rows,
                            int64_t len, int64_t k, int64_t *out_ids, float *out_vals, void *ws, size_t ws_bytes,
                            void *stream) {
  return pkv_launch_topk_f32(x, x_stride, ids, ids_stride, rows, len, k, out_ids, out_vals, ws, ws_bytes,
                             (hipStream_t)stream, false);
}

struct AdkWs {
  size_t ben, vn, smax, ssum;
  WideWs wide;
  size_t total;
};
static AdkWs adk_ws_layout(int rows, int64_t n_cand, int64_t k_out) {
  AdkWs w;
  const size_t n_slices = (size_t)((n_cand + kWideSlice - 1) / kWideSlice);
  size_t off = 0;
  w.ben = off;
  off = pkv_align_up(off + (size_t)rows * (size_t)n_cand * sizeof(float), 256);
  w.vn = off;
  off = pkv_align_up(off + (size_t)rows * (size_t)n_cand * sizeof(float), 256);
  w.smax = off;
  off = pkv_align_up(off + (size_t)rows * (size_t)((n_cand + kAdkPart - 1) / kAdkPart) * sizeof(float), 256);
  w.ssum = off;
  off = pkv_align_up(off + (size_t)rows * (n_slices + 1) * sizeof(float), 256);  // slice sums, then the dense tokens' sum
  w.wide = wide_ws_layout(rows, n_cand, k_out, off);
  w.total = w.wide.total;
  return w;
}

extern "C" size_t pkv_adaptive_topk_ws_bytes(int rows, int64_t n_cand, int64_t k_out) {
  if (rows <= 0 || n_cand <= kTopkMaxSort || k_out <= 0) return 256;
  return adk_ws_layout(rows, n_cand, k_out).total;
}

extern "C" int pkv_adaptive_topk(const float *sl_logits, int64_t sl_stride, const float *sl_vnorm, int64_t slv_stride,
                                 int64_t sl, const void *cand_scores, int cand_dtype, float cand_scale,
                                 const float *cand_vnorm, const float *value_norm, int64_t vn_stride, int64_t vn_offset,
                                 int64_t vn_pos_stride, const int64_t *cand_ids, int64_t n_cand, float threshold,
                                 int64_t k_out, int rows,
                                 int64_t *adaptive_k, int64_t *topk_ids, int64_t k_min, int64_t k_max,
                                 int32_t *row_keys, int64_t row_keys_base, void *ws, size_t ws_bytes, void *stream) {
  PKV_REQUIRE(k_max <= 0 || (k_min >= 0 && k_min <= k_max), "pkv_adaptive_topk: clamp [%lld, %lld] is empty",
              (long long)k_min, (long long)k_max);
  const AdkClamp cl{k_min, k_max, row_keys, row_keys_base};
  PKV_REQUIRE(cand_scores && cand_ids && adaptive_k && topk_ids && (cand_vnorm || value_norm),
              "pkv_adaptive_topk: null pointer");
  PKV_REQUIRE(sl >= 0 && (sl == 0 || (sl_logits && sl_vnorm)), "pkv_adaptive_topk: dense logits missing");
  if (vn_pos_stride <= 0) vn_pos_stride = 1;
  PKV_REQUIRE(cand_vnorm || (vn_stride > 0 && vn_stride % vn_pos_stride == 0),
              "pkv_adaptive_topk: value_norm needs its row stride (vn_stride), a multiple of the position stride");
  PKV_REQUIRE(cand_dtype == PKV_DTYPE_F32 || cand_dtype == PKV_DTYPE_BF16, "unknown candidate score dtype %d", cand_dtype);
  PKV_REQUIRE(rows > 0 && rows <= 65535 && n_cand > 0 && n_cand < ((int64_t)1 << 31) && k_out > 0 && k_out <= n_cand,
              "need 0 < k_out <= n_cand (k_out=%lld n_cand=%lld rows=%d)", (long long)k_out, (long long)n_cand, rows);
  PKV_REQUIRE(k_out <= kTopkMaxSort, "k_out up to %d supported (got %lld)", kTopkMaxSort, (long long)k_out);
  hipStream_t s = (hipStream_t)stream;
  const int P = pow2_ceil(k_out);
  if (n_cand <= kTopkMaxSort) {  // one workgroup per row, no workspace
    const int ein = pow2_ceil(n_cand) / kTopkThreads;
#define PKV_ADK(EIN)                                                                                                  \
  hipLaunchKernelGGL((pkv_adaptive_topk_kernel<EIN>), dim3((unsigned)rows), dim3(kTopkThreads), lds_bytes_sort(P), s,      \
                     sl_logits, sl_stride, sl_vnorm, slv_stride, sl, cand_scores, cand_dtype, cand_scale, cand_vnorm, \
                     value_norm, vn_stride, vn_offset, vn_pos_stride, cand_ids, (int)n_cand, threshold, k_out, P,     \
                     adaptive_k, topk_ids, cl)
    if (ein <= 1) PKV_ADK(1); else if (ein == 2) PKV_ADK(2); else if (ein == 4) PKV_ADK(4); else PKV_ADK(8);
#undef PKV_ADK
    PKV_LAUNCH_CHECK("pkv_adaptive_topk_kernel");
    return PKV_OK;
  }
  const AdkWs w = adk_ws_layout(rows, n_cand, k_out);
  if (!ws || ws_bytes < w.total || !pkv_aligned(ws, 256)) {
    pkv_set_error("pkv_adaptive_topk: workspace of %zu bytes (256-aligned) required, got %zu", w.total, ws_bytes);
    return PKV_ENOMEM;
  }
  char *base = (char *)ws;
  float *ben = (float *)(base + w.ben), *smax = (float *)(base + w.smax), *ssum = (float *)(base + w.ssum);
  uint32_t *ctl = (uint32_t *)(base + w.wide.ctl);
  uint64_t *list_a = (uint64_t *)(base + w.wide.list_a), *list_b = (uint64_t *)(base + w.wide.list_b);
  float *gathered = (float *)(base + w.vn);
  const int n_slices = (int)((n_cand + kWideSlice - 1) / kWideSlice);
  const int n_parts = (int)((n_cand + kAdkPart - 1) / kAdkPart);
  const dim3 grid((unsigned)n_slices, (unsigned)rows);
  hipLaunchKernelGGL(pkv_adk_max_gather_kernel, dim3((unsigned)n_parts, (unsigned)rows), dim3(kAdkPartThreads), 0, s,
                     sl_logits, sl_stride, sl, cand_scores, cand_dtype, cand_scale, cand_vnorm ? nullptr : value_norm,
                     vn_stride, vn_offset, vn_pos_stride, cand_ids, n_cand, smax, gathered, ctl);
  PKV_LAUNCH_CHECK("pkv_adk_max_gather_kernel");
  hipLaunchKernelGGL(pkv_adk_benefit_kernel, dim3((unsigned)n_slices + 1, (unsigned)rows), dim3(kTopkThreads), 0, s,
                     sl_logits, sl_stride, sl_vnorm, slv_stride, sl, cand_scores, cand_dtype, cand_scale,
                     cand_vnorm ? cand_vnorm : gathered, n_cand, smax, n_parts, ben, ssum, ctl);
  PKV_LAUNCH_CHECK("pkv_adk_benefit_kernel");
  hipLaunchKernelGGL(pkv_adk_compact_kernel, grid, dim3(kTopkThreads), 0, s, ben, n_cand, k_out, ctl, list_a, list_b);
  PKV_LAUNCH_CHECK("pkv_adk_compact_kernel");
  hipLaunchKernelGGL(pkv_adk_finish_kernel, dim3((unsigned)rows), dim3(kTopkThreads), lds_bytes_sort(P), s, cand_ids,
                     n_cand, n_slices, threshold, k_out, P, ssum, ctl, list_a, list_b, adaptive_k, topk_ids, cl);
  PKV_LAUNCH_CHECK("pkv_adk_finish_kernel");
  return PKV_OK;
}

extern "C" int pkv_dense_logits(const void *q, int dtype, int bs, int n_kv_heads, int group, const void *k,
                                int64_t k_stride_b, int64_t k_stride_h, int64_t n_rows, float scale, float *out,
                                int64_t out_stride, void *stream) {
  PKV_REQUIRE(q && k && out, "pkv_dense_logits: null pointer");
  PKV_REQUIRE(dtype == PKV_DTYPE_F32 || dtype == PKV_DTYPE_BF16, "pkv_dense_logits: unknown dtype %d", dtype);
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && group > 0 && (int64_t)bs * n_kv_heads <= 65535 && n_rows > 0 &&
                  out_stride >= n_rows,
              "pkv_dense_logits: bad shape bs=%d heads=%d group=%d rows=%lld", bs, n_kv_heads, group, (long long)n_rows);
  PKV_REQUIRE(k_stride_b % 8 == 0 && k_stride_h % 8 == 0 && pkv_aligned(q, 16) && pkv_aligned(k, 16),
              "pkv_dense_logits: rows must be 16-byte aligned");
  constexpr int rows_per_wg = kDenseLogitThreads / 16;
  const dim3 grid((unsigned)((n_rows + rows_per_wg - 1) / rows_per_wg), (unsigned)(bs * n_kv_heads));
  if (dtype == PKV_DTYPE_BF16)
    hipLaunchKernelGGL(pkv_dense_logits_kernel<true>, grid, dim3(kDenseLogitThreads), 0, (hipStream_t)stream, q,
                       n_kv_heads, group, k, k_stride_b, k_stride_h, n_rows, scale, out, out_stride);
  else
    hipLaunchKernelGGL(pkv_dense_logits_kernel<false>, grid, dim3(kDenseLogitThreads), 0, (hipStream_t)stream, q,
                       n_kv_heads, group, k, k_stride_b, k_stride_h, n_rows, scale, out, out_stride);
  PKV_LAUNCH_CHECK("pkv_dense_logits_kernel");
  return PKV_OK;
}

extern "C" int pkv_uniform_k(const int64_t *adaptive_k, int rows, int64_t *uniform_k, int32_t *row_keys,
                             int64_t row_keys_base, void *stream) {
  PKV_REQUIRE(adaptive_k && uniform_k && rows > 0, "pkv_uniform_k: bad arguments");
  hipLaunchKernelGGL(pkv_uniform_k_kernel, dim3(1), dim3(kTopkThreads), 0, (hipStream_t)stream, adaptive_k, rows,
                     uniform_k, row_keys, row_keys_base);
  PKV_LAUNCH_CHECK("pkv_uniform_k_kernel");
  return PKV_OK;
}
