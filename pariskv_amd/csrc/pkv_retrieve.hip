// One layer's retrieval for one decode step as a fixed sequence of launches on
// the caller's stream: query prep + vote table -> collision scan (+ chunk
// histograms) -> candidate select fused with the 4-bit rerank -> exact top-k ->
// optional gather of the selected K/V rows (5 launches).  The adaptive-k step
// replaces the exact top-k by the dense logits and the adaptive selection.
//
// Reference: cache_hub/polar_cache.py:1126-1162 (collision_based_topk_batch),
// :1207-1231, :1244-1304 and the gather at :1075-1095.
#include "pkv_common.h"

#include <mutex>

PKV_INTERNAL int pkv_launch_identity_fill(int64_t *out, int64_t len, int64_t k, int rows, hipStream_t s);
PKV_INTERNAL int pkv_launch_qk_norm_rope_table(const void *qkv, int64_t stride_b, int bs, int n_q_heads, int n_kv_heads,
                                  const void *q_weight, const void *k_weight, float eps, const void *cos_row,
                                  const void *sin_row, void *q_out, void *k_out, const float *signs, const int32_t *cc,
                                  const PkvTiers &tiers, float *qhat, float *qnorm, uint8_t *lut, uint32_t *row_suf,
                                  uint32_t *zero_ptr, int64_t zero_words, const pkv_kv_append *append, hipStream_t s);
PKV_INTERNAL size_t pkv_fused_sync_bytes(int rows, int64_t n_chunks);
PKV_INTERNAL bool pkv_fused_usable(int rows, int64_t n_keys, int chunk_keys, hipStream_t s);
PKV_INTERNAL int pkv_launch_fused_retrieve(const void *q, int dtype, int bs, int n_kv_heads, int group, const float *signs,
                              const int32_t *cc, int64_t cc_b, int64_t cc_h, const PkvTiers &tiers, float *qhat,
                              float *qnorm, uint8_t *lut, const uint8_t *codes, int64_t cs_b, int64_t cs_h,
                              int64_t n_keys, int chunk_keys, uint8_t *cnt_u8, int64_t cnt_stride, uint32_t *row_suf,
                              uint16_t *chunk_suf, void *sync_area, uint32_t *zero_ptr, int64_t zero_row_words,
                              int64_t zero_row_stride, int64_t k, const uint8_t *nib, int64_t ns_b, int64_t ns_h,
                              int64_t ns_key, const uint16_t *weight, int64_t ws_b, int64_t ws_h, int64_t ws_key,
                              const float *centers, int64_t *cand, float *scores, int64_t extra_off, float *extra_out,
                              uint32_t *range_slots, int64_t range_row_stride, hipStream_t s);

namespace {

struct WsLayout {
  size_t qhat, qnorm, lut, cnt, hist, rowsuf, cand, scores, cand_extra, topk, topk_bytes, sync, sync_bytes, total;
  int64_t cnt_stride;
  int chunk_keys;
  int64_t n_chunks;
  int sub_blocks;  // pieces per chunk of the scan -> select + rerank pair (one suffix histogram each)
};

WsLayout layout(int rows, int64_t n_keys, int64_t n_cand, int64_t k) {
  WsLayout w;
  size_t off = 0;
  auto take = [&](size_t bytes) {
    size_t o = off;
    off += pkv_align_up(bytes, 256);
    return o;
  };
  w.chunk_keys = pkv_pick_chunk_keys(rows, n_keys);
  w.n_chunks = (n_keys + w.chunk_keys - 1) / w.chunk_keys;
  w.cnt_stride = (int64_t)pkv_align_up((size_t)n_keys, 16);
  w.qhat = take((size_t)rows * 128 * sizeof(float));
  w.qnorm = take((size_t)rows * sizeof(float));
  w.lut = take((size_t)rows * 4096);
  w.cnt = take((size_t)rows * (size_t)w.cnt_stride);
  w.sub_blocks = pkv_pick_sub_blocks(w.chunk_keys, w.n_chunks);
  w.hist = take((size_t)rows * (size_t)w.n_chunks * w.sub_blocks * 128 * sizeof(uint16_t));
  w.rowsuf = take((size_t)rows * 128 * sizeof(uint32_t));
  w.cand = take((size_t)rows * (size_t)n_cand * sizeof(int64_t));
  w.scores = take((size_t)rows * (size_t)n_cand * sizeof(float));
  w.cand_extra = take((size_t)rows * (size_t)n_cand * sizeof(float));  // record word passed through per candidate
  // the top-k's control area (range slots; for wide rows the control blocks and lists of the multi-workgroup form)
  w.topk_bytes = pkv_topk_ws_bytes_impl(rows, n_cand, k);
  const size_t ctl_bytes = pkv_align_up((size_t)pkv_topk_ctl_words(rows, n_cand) * 4, 256);
  if (w.topk_bytes < ctl_bytes) w.topk_bytes = ctl_bytes;
  w.topk = take(w.topk_bytes);
  // flags and status word of the one-launch form of the first three stages
  w.sync_bytes = pkv_fused_sync_bytes(rows, w.n_chunks);
  w.sync = take(w.sync_bytes);
  w.total = off;
  return w;
}

bool shape_ok(int rows, int64_t n_keys, int64_t n_cand, int64_t k) {
  return rows > 0 && rows <= 65535 && n_keys > 0 && n_keys <= PKV_MAX_KEYS_PER_ROW && n_cand > 0 &&
         n_cand <= n_keys && k > 0 && k <= n_cand;
}

}  // namespace

extern "C" size_t pkv_retrieve_ws_bytes(int rows, int64_t n_keys, int64_t n_cand, int64_t k) {
  if (!shape_ok(rows, n_keys, n_cand, k)) return 0;
  return layout(rows, n_keys, n_cand, k).total;
}

extern "C" int pkv_retrieve_ws_view(void *ws, int rows, int64_t n_keys, int64_t n_cand, int64_t k, const char *name,
                                    void **ptr, size_t *bytes) {
  PKV_REQUIRE(ws && name && ptr && bytes && shape_ok(rows, n_keys, n_cand, k), "pkv_retrieve_ws_view: bad arguments");
  const WsLayout w = layout(rows, n_keys, n_cand, k);
  char *base = (char *)ws;
  if (!strcmp(name, "qhat")) {
    *ptr = base + w.qhat, *bytes = (size_t)rows * 128 * 4;
  } else if (!strcmp(name, "qnorm")) {
    *ptr = base + w.qnorm, *bytes = (size_t)rows * 4;
  } else if (!strcmp(name, "lut")) {
    *ptr = base + w.lut, *bytes = (size_t)rows * 4096;
  } else if (!strcmp(name, "cnt_u8")) {
    *ptr = base + w.cnt, *bytes = (size_t)rows * (size_t)w.cnt_stride;
  } else if (!strcmp(name, "chunk_suffix_hist")) {
    *ptr = base + w.hist, *bytes = (size_t)rows * (size_t)w.n_chunks * w.sub_blocks * 256;
  } else if (!strcmp(name, "row_suffix_hist")) {
    *ptr = base + w.rowsuf, *bytes = (size_t)rows * 512;
  } else if (!strcmp(name, "cand")) {
    *ptr = base + w.cand, *bytes = (size_t)rows * (size_t)n_cand * 8;
  } else if (!strcmp(name, "scores")) {
    *ptr = base + w.scores, *bytes = (size_t)rows * (size_t)n_cand * 4;
  } else if (!strcmp(name, "topk_control")) {
    *ptr = base + w.topk, *bytes = w.topk_bytes;
  } else if (!strcmp(name, "handover_status")) {
    // one word at the end of the hand-over area: workgroups of one-launch retrievals that gave up a wait (0 = none)
    *ptr = base + w.sync + w.sync_bytes - 256, *bytes = 4;
  } else if (!strcmp(name, "cand_record_word")) {
    *ptr = base + w.cand_extra, *bytes = (size_t)rows * (size_t)n_cand * 4;
  } else {
    pkv_set_error("unknown workspace segment '%s'", name);
    return PKV_EINVAL;
  }
  return PKV_OK;
}

static int retrieve_impl(const pkv_retrieve_args *a, void *ws, size_t ws_bytes, void *stream) {
  PKV_REQUIRE(a != nullptr, "pkv_retrieve: null args");
  PKV_REQUIRE(a->q && a->signs && a->centers && a->cluster_counts && a->codes && a->nib && a->weight,
              "pkv_retrieve: null pointer");
  PKV_REQUIRE(a->dtype == PKV_DTYPE_F32 || a->dtype == PKV_DTYPE_BF16, "unknown dtype %d", a->dtype);
  PKV_REQUIRE(a->bs > 0 && a->n_kv_heads > 0 && a->group > 0, "bad shape bs=%d kv_heads=%d group=%d", a->bs,
              a->n_kv_heads, a->group);
  const int rows = a->bs * a->n_kv_heads;
  PKV_REQUIRE(shape_ok(rows, a->n_keys, a->n_cand, a->k),
              "need 0 < k <= n_cand <= n_keys <= 2^24 (k=%lld n_cand=%lld n_keys=%lld rows=%d)", (long long)a->k,
              (long long)a->n_cand, (long long)a->n_keys, rows);
  PKV_REQUIRE(a->key0 >= 0 && a->key0 + a->n_keys <= a->cap, "retrieval zone [%lld,+%lld) exceeds capacity %lld",
              (long long)a->key0, (long long)a->n_keys, (long long)a->cap);
  PKV_REQUIRE(a->n_tiers >= 1 && a->n_tiers <= PKV_MAX_TIERS, "n_tiers must be in [1,%d]", PKV_MAX_TIERS);
  PKV_REQUIRE(pkv_aligned(a->codes, 16) && pkv_aligned(a->nib, 16) && pkv_aligned(a->weight, 16) &&
                  pkv_aligned(a->q, 16),
              "queries / codes / nib / weight must be 16-byte aligned");
  const WsLayout w = layout(rows, a->n_keys, a->n_cand, a->k);
  if (!ws || ws_bytes < w.total || !pkv_aligned(ws, 256)) {
    pkv_set_error("pkv_retrieve: workspace of %zu bytes (256-aligned) required, got %zu", w.total, ws_bytes);
    return PKV_ENOMEM;
  }
  hipStream_t s = (hipStream_t)stream;
  char *base = (char *)ws;
  float *qhat = (float *)(base + w.qhat);
  float *qnorm = (float *)(base + w.qnorm);
  uint8_t *lut = (uint8_t *)(base + w.lut);
  uint8_t *cnt = (uint8_t *)(base + w.cnt);
  uint16_t *hist = (uint16_t *)(base + w.hist);
  uint32_t *rowsuf = (uint32_t *)(base + w.rowsuf);
  int64_t *cand = (int64_t *)(base + w.cand);
  float *scores = (float *)(base + w.scores);

  PkvTiers t;
  memset(&t, 0, sizeof t);
  t.n = a->n_tiers;
  for (int i = 0; i < a->n_tiers; ++i) t.t[i] = a->tier_counts[i];

  const int H = a->n_kv_heads;
  // bytes from one key's nibbles / weights to the next key's: packed arrays, or both inside one wider record
  const int64_t nk = a->nib_key_stride ? a->nib_key_stride : 64;
  const int64_t wk = (a->weight_key_stride ? a->weight_key_stride : 32) / 2;  // in bf16 elements
  PKV_REQUIRE(nk >= 64 && nk % 16 == 0 && wk >= 16 && wk % 8 == 0,
              "key strides of %lld / %lld bytes: nibbles need >= 64, weights >= 32, multiples of 16",
              (long long)a->nib_key_stride, (long long)a->weight_key_stride);
  // the top-k takes the rows' score ranges from its control area (and a multi-workgroup top-k, more than 8192
  // candidates, wants its control blocks cleared): the first launch of the step clears, the select + rerank launch
  // leaves the ranges
  const int64_t ctl_words = a->out_ids && a->n_cand != a->n_keys ? pkv_topk_ctl_words(rows, a->n_cand) : 0;
  uint32_t *topk_ctl = ctl_words ? (uint32_t *)(base + w.topk) : nullptr;
  int64_t range_stride = 0;
  uint32_t *range_slots = topk_ctl ? pkv_topk_range_slots(topk_ctl, a->n_cand, &range_stride) : nullptr;
  const uint8_t *codes = a->codes + a->key0 * 16;
  const uint8_t *nib = a->nib + a->key0 * nk;
  const uint16_t *weight = a->weight + a->key0 * wk;
  int rc;
  if (a->n_cand != a->n_keys && a->launch_plan == PKV_PLAN_ONE_LAUNCH && pkv_fused_usable(rows, a->n_keys, w.chunk_keys, s)) {
    // query prep, scan and select + rerank as one launch
    rc = pkv_launch_fused_retrieve(a->q, a->dtype, a->bs, H, a->group, a->signs, a->cluster_counts, (int64_t)H * 4096, 4096,
                                   t, qhat, qnorm, lut, codes, (int64_t)H * a->cap * 16, a->cap * 16, a->n_keys,
                                   w.chunk_keys, a->skip_vote_counts ? nullptr : cnt, w.cnt_stride, rowsuf, hist,
                                   base + w.sync, topk_ctl, topk_ctl ? ctl_words / rows : 0, topk_ctl ? ctl_words / rows : 0,
                                   a->n_cand, nib, (int64_t)H * a->cap * nk, a->cap * nk, nk, weight,
                                   (int64_t)H * a->cap * wk, a->cap * wk, wk, a->centers, cand, scores,
                                   a->record_word_offset,
                                   a->record_word_offset > 0 ? (float *)(base + w.cand_extra) : nullptr, range_slots,
                                   range_stride, s);
  } else {
    // table_ready: pkv_qk_norm_rope_table already left the rotated query, its norm and the vote table of these
    // queries in the workspace and cleared what this launch would clear
    rc = a->table_ready ? PKV_OK
                        : pkv_launch_query_prep_lut(a->q, a->dtype, a->bs, H, a->group, a->signs, a->cluster_counts,
                                                    (int64_t)H * 4096, 4096, t, qhat, qnorm, lut, nullptr, rowsuf, s, topk_ctl,
                                                    ctl_words);
    if (rc) return rc;
    if (a->n_cand == a->n_keys) {
      rc = pkv_launch_identity_fill(cand, a->n_keys, a->n_cand, rows, s);
      if (rc) return rc;
      rc = pkv_launch_rerank(cand, a->bs, H, a->n_cand, a->n_keys, nib, (int64_t)H * a->cap * nk, a->cap * nk, nk, 4,
                             weight, (int64_t)H * a->cap * wk, a->cap * wk, wk, 1, qhat, qnorm, a->centers, scores,
                             nullptr, s);
    } else {
      rc = pkv_launch_scan(codes, (int64_t)H * a->cap * 16, a->cap * 16, 16, 1, a->bs, H, a->n_keys, lut, cnt,
                           w.cnt_stride, nullptr, rowsuf, hist, w.chunk_keys, s, w.sub_blocks);
      if (rc) return rc;
      rc = pkv_launch_select_rerank(cnt, w.cnt_stride, rowsuf, hist, w.chunk_keys, a->bs, H, a->n_keys, a->n_cand, nib,
                                    (int64_t)H * a->cap * nk, a->cap * nk, nk, weight, (int64_t)H * a->cap * wk, a->cap * wk,
                                    wk, qhat, qnorm, a->centers, cand, scores, s, a->record_word_offset,
                                    a->record_word_offset > 0 ? (float *)(base + w.cand_extra) : nullptr,
                                    range_slots, range_stride, w.sub_blocks);
    }
  }
  if (rc) return rc;
  if (!a->out_ids) return PKV_OK;  // candidates only: the caller reads them out of the workspace
  rc = pkv_launch_topk_f32(scores, a->n_cand, cand, a->n_cand, rows, a->n_cand, a->k, a->out_ids, a->out_scores,
                           (char *)ws + w.topk, w.topk_bytes, s, a->any_order != 0, topk_ctl != nullptr);
  if (rc) return rc;
  if (a->src_k) {
    PKV_REQUIRE(a->src_v && a->dst_k && a->dst_v, "pkv_retrieve: gather needs src_v, dst_k, dst_v");
    const void *sk = a->src_k, *sv = a->src_v;
    if (a->gather_from_host) {
      void *dk = nullptr, *dv = nullptr;
      rc = pkv_host_device_pointer(a->src_k, &dk);
      if (rc) return rc;
      rc = pkv_host_device_pointer(a->src_v, &dv);
      if (rc) return rc;
      sk = dk, sv = dv;
    }
    rc = pkv_launch_gather(sk, sv, a->src_len, a->out_ids, a->k, a->idx_offset, a->dst_k, a->dst_v, a->dst_len,
                           a->dst_row0, rows, a->row_bytes, s);
  }
  return rc;
}

extern "C" int pkv_qk_norm_rope_table(const void *qkv, int64_t stride_b, int n_q_heads, const void *q_weight,
                                      const void *k_weight, float eps, const void *cos_row, const void *sin_row, void *q_out,
                                      void *k_out, const pkv_retrieve_args *a, void *ws, size_t ws_bytes,
                                      const pkv_kv_append *append, void *stream) {
  PKV_REQUIRE(a != nullptr, "pkv_qk_norm_rope_table: null retrieval arguments");
  PKV_REQUIRE(a->dtype == PKV_DTYPE_BF16 && a->bs > 0 && a->n_kv_heads > 0 && a->group > 0 &&
                  n_q_heads == a->n_kv_heads * a->group,
              "pkv_qk_norm_rope_table: bf16 queries of %d x %d heads expected, got %d query heads", a->n_kv_heads, a->group,
              n_q_heads);
  PKV_REQUIRE(a->signs && a->cluster_counts && a->n_tiers >= 1 && a->n_tiers <= PKV_MAX_TIERS,
              "pkv_qk_norm_rope_table: the retrieval's signs / cluster counts / tiers are missing");
  const int rows = a->bs * a->n_kv_heads;
  PKV_REQUIRE(shape_ok(rows, a->n_keys, a->n_cand, a->k), "pkv_qk_norm_rope_table: bad retrieval shape");
  const WsLayout w = layout(rows, a->n_keys, a->n_cand, a->k);
  if (!ws || ws_bytes < w.total || !pkv_aligned(ws, 256)) {
    pkv_set_error("pkv_qk_norm_rope_table: workspace of %zu bytes (256-aligned) required, got %zu", w.total, ws_bytes);
    return PKV_ENOMEM;
  }
  char *base = (char *)ws;
  PkvTiers t;
  memset(&t, 0, sizeof t);
  t.n = a->n_tiers;
  for (int i = 0; i < a->n_tiers; ++i) t.t[i] = a->tier_counts[i];
  const int64_t ctl_words = a->out_ids && a->n_cand != a->n_keys ? pkv_topk_ctl_words(rows, a->n_cand) : 0;
  return pkv_launch_qk_norm_rope_table(qkv, stride_b, a->bs, n_q_heads, a->n_kv_heads, q_weight, k_weight, eps, cos_row,
                                       sin_row, q_out, k_out, a->signs, a->cluster_counts, t, (float *)(base + w.qhat),
                                       (float *)(base + w.qnorm), (uint8_t *)(base + w.lut), (uint32_t *)(base + w.rowsuf),
                                       ctl_words ? (uint32_t *)(base + w.topk) : nullptr, ctl_words, append,
                                       (hipStream_t)stream);
}

extern "C" int pkv_retrieve(const pkv_retrieve_args *a, void *ws, size_t ws_bytes, void *stream) {
  return retrieve_impl(a, ws, ws_bytes, stream);
}

// ---- the same retrieval for callers that cannot allocate: the workspace is a fixed array of the library ----

// Scratch of the no-allocation entry point: the segments pkv_retrieve lays out in its caller's workspace
// (rotated query, vote table, vote counts, chunk histograms, candidate list, scores, lists of the wide top-k).
// One copy per GPU, held from the load of the library's code object on that GPU until the process ends.
static __device__ __align__(256) unsigned char scratch[PKV_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices];  // per device: the address of that GPU's copy of `scratch`

// Device address of the calling thread's current GPU's scratch array (looked up once per device).
int scratch_for_current_device(void **out) {
  int dev = -1;
  PKV_HIP(hipGetDevice(&dev));
  PKV_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal %d outside [0,%d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void *p = nullptr;
    PKV_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    PKV_REQUIRE(p != nullptr && pkv_aligned(p, 256), "the scratch array of device %d has no usable address", dev);
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return PKV_OK;
}
}  // namespace

extern "C" size_t pkv_retrieve_noalloc_max_bytes(void) { return (size_t)PKV_NOALLOC_SCRATCH_BYTES; }

extern "C" int pkv_retrieve_noalloc_prepare(void) {
  void *ws = nullptr;
  return scratch_for_current_device(&ws);
}

extern "C" int pkv_retrieve_noalloc(const pkv_retrieve_args *a, void *stream) {
  PKV_REQUIRE(a != nullptr, "pkv_retrieve_noalloc: null args");
  PKV_REQUIRE(a->out_ids != nullptr,
              "pkv_retrieve_noalloc: the candidates-only form (out_ids == NULL) leaves its results in the workspace, "
              "which here is the library's own scratch; use pkv_retrieve");
  const int rows = a->bs * a->n_kv_heads;
  PKV_REQUIRE(a->bs > 0 && a->n_kv_heads > 0 && shape_ok(rows, a->n_keys, a->n_cand, a->k),
              "need 0 < k <= n_cand <= n_keys <= 2^24 (k=%lld n_cand=%lld n_keys=%lld rows=%d)", (long long)a->k,
              (long long)a->n_cand, (long long)a->n_keys, rows);
  const size_t need = layout(rows, a->n_keys, a->n_cand, a->k).total;
  if (need > (size_t)PKV_NOALLOC_SCRATCH_BYTES) {
    pkv_set_error("pkv_retrieve_noalloc: this shape needs %zu bytes of scratch, the fixed array holds %zu "
                  "(rows=%d n_keys=%lld n_cand=%lld k=%lld); use pkv_retrieve with a workspace of the caller's",
                  need, (size_t)PKV_NOALLOC_SCRATCH_BYTES, rows, (long long)a->n_keys, (long long)a->n_cand,
                  (long long)a->k);
    return PKV_ENOMEM;
  }
  // the scratch array is the current device's: a stream of another GPU would be handed the wrong copy's address
  int cur = -1;
  hipDevice_t sdev = -1;
  PKV_HIP(hipGetDevice(&cur));
  if (stream != nullptr && hipStreamGetDevice((hipStream_t)stream, &sdev) == hipSuccess) {
    PKV_REQUIRE((int)sdev == cur, "pkv_retrieve_noalloc: the stream belongs to device %d, the calling thread's current device is %d",
                (int)sdev, cur);
  } else {
    (void)hipGetLastError();
  }
  void *ws = nullptr;
  const int rc = scratch_for_current_device(&ws);
  if (rc) return rc;
  return retrieve_impl(a, ws, (size_t)PKV_NOALLOC_SCRATCH_BYTES, stream);
}

extern "C" int pkv_decode_step(const pkv_retrieve_args *retrieve, void *ws, size_t ws_bytes,
                               const pkv_attn_args *attention, void *stream) {
  PKV_REQUIRE(retrieve && attention, "pkv_decode_step: null args");
  int rc = pkv_retrieve(retrieve, ws, ws_bytes, stream);
  if (rc) return rc;
  return pkv_decode_attention(retrieve->q, retrieve->dtype, retrieve->bs, retrieve->n_kv_heads, retrieve->group,
                              attention->segments, attention->n_segments, attention->row_keys, attention->scale,
                              attention->out, attention->ws, attention->ws_bytes, stream);
}

extern "C" int pkv_adaptive_decode_step(const pkv_retrieve_args *retrieve, void *ws, size_t ws_bytes,
                                        const pkv_adaptive_args *ad, const pkv_attn_args *attention, void *stream) {
  PKV_REQUIRE(retrieve && ad && attention, "pkv_adaptive_decode_step: null args");
  PKV_REQUIRE(!retrieve->out_ids && !retrieve->src_k,
              "pkv_adaptive_decode_step: the retrieval must be in its candidates-only form (no out_ids, no gather)");
  PKV_REQUIRE(ad->row_keys && attention->row_keys == ad->row_keys,
              "pkv_adaptive_decode_step: the attention must read the row_keys the adaptive stage writes");
  PKV_REQUIRE(ad->dense_rows > 0 && ad->dense_rows <= ad->dense_vnorm_stride && ad->dense_rows <= ad->dense_logits_stride,
              "pkv_adaptive_decode_step: %lld dense rows exceed the norm / logit rows (%lld, %lld)",
              (long long)ad->dense_rows, (long long)ad->dense_vnorm_stride, (long long)ad->dense_logits_stride);
  int rc = pkv_retrieve(retrieve, ws, ws_bytes, stream);
  if (rc) return rc;
  const int rows = retrieve->bs * retrieve->n_kv_heads;
  const WsLayout w = layout(rows, retrieve->n_keys, retrieve->n_cand, retrieve->k);
  const int64_t *cand = (const int64_t *)((char *)ws + w.cand);
  const float *scores = (const float *)((char *)ws + w.scores);
  // the candidates' value norms came out of the rerank with the scores when the caller keeps them in the key
  // records (not on the all-keys-are-candidates path, which reranks without the fused kernel)
  const bool norms_emitted = retrieve->record_word_offset > 0 && retrieve->n_cand != retrieve->n_keys;
  const float *cand_vnorm = norms_emitted ? (const float *)((char *)ws + w.cand_extra) : nullptr;
  rc = pkv_dense_logits(retrieve->q, retrieve->dtype, retrieve->bs, retrieve->n_kv_heads, retrieve->group, ad->dense_k,
                        ad->dense_stride_b, ad->dense_stride_h, ad->dense_rows, ad->scale, ad->dense_logits,
                        ad->dense_logits_stride, stream);
  if (rc) return rc;
  rc = pkv_adaptive_topk(ad->dense_logits, ad->dense_logits_stride, ad->dense_vnorm, ad->dense_vnorm_stride,
                         ad->dense_rows, scores, PKV_DTYPE_F32, ad->scale, cand_vnorm, ad->value_norm, ad->vn_stride,
                         ad->vn_offset, ad->vn_pos_stride, cand, retrieve->n_cand, ad->threshold, ad->k_out, rows, ad->adaptive_k,
                         ad->topk_ids, ad->k_min, ad->k_max, ad->row_keys, ad->row_keys_base, ad->ws, ad->ws_bytes, stream);
  if (rc) return rc;
  if (ad->uniform_k) {
    rc = pkv_uniform_k(ad->adaptive_k, rows, ad->uniform_k, ad->row_keys, ad->row_keys_base, stream);
    if (rc) return rc;
  }
  rc = pkv_gather_uva_ragged(ad->src_k, ad->src_v, ad->src_len, ad->topk_ids, ad->k_out,
                             ad->uniform_k ? ad->uniform_k : ad->adaptive_k, ad->idx_offset,
                             ad->dst_k, ad->dst_v, ad->dst_len, ad->dst_row0, retrieve->bs, retrieve->n_kv_heads,
                             ad->row_bytes, stream);
  if (rc) return rc;
  return pkv_decode_attention(retrieve->q, retrieve->dtype, retrieve->bs, retrieve->n_kv_heads, retrieve->group,
                              attention->segments, attention->n_segments, attention->row_keys, attention->scale,
                              attention->out, attention->ws, attention->ws_bytes, stream);
}
