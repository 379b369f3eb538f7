// Dense decode attention over the gathered key set: softmax(q k^T * scale) v for ONE
// query token per sequence, GQA (the G query heads of a KV head share its keys), over
// up to four row segments of head_dim 128 (sink | update buffer | gathered top-k |
// local window), non-causal.
//
// Reference: cache_hub/polar_cache.py:1084-1105 (torch.cat of the segments, then
// flash_attn_func on [bs, S, H, D]); here the segments are read where they lie.
//
// HBM-bound: 512 B (one K row + one V row, bf16) per key and KV head, read once for
// all G query heads.  Split over the key axis (flash-decoding): grid (n_splits, R);
// every split keeps a running (max, sum, output) per query head and the partial
// results are merged by a second small launch.
//   bf16: four waves per split on the matrix cores (v_mfma_f32_16x16x32_bf16), merged through LDS, see below.
//   fp32: 256 threads per split, every 16 lanes own one key at a time (a wave
//         instruction moves four whole rows), fp32 FMA and lane-exchange reductions.
//
// Arithmetic: products and sums in fp32 (bf16 path: bf16 x bf16 products accumulated in
// fp32, probabilities rounded to bf16 before P.V as flash-attn does), exp2 with the scale
// folded in; the output is rounded to the input dtype.  Not bit-reproducible against another summation order -
// the tolerance of this row is 2e-2 absolute in bf16.
#include "pkv_common.h"

// Fused multiply-add is welcome here (the rest of the library forbids it because integer results are
// derived from its float steps; this kernel's only contract is the 2e-2 tolerance).
#pragma clang fp contract(fast)

namespace {

constexpr int kAttThreads = 256;
constexpr int kAttKeysPerIter = kAttThreads / 16;  // 16 keys per workgroup step
constexpr int kAttUnroll = 2;                      // keys per 16-lane group per step
constexpr float kNegBig = -1.0e30f;

struct AttSegs {
  const void *k[PKV_ATTN_MAX_SEGMENTS];
  const void *v[PKV_ATTN_MAX_SEGMENTS];
  int64_t stride_b[PKV_ATTN_MAX_SEGMENTS], stride_h[PKV_ATTN_MAX_SEGMENTS];
  int64_t row0[PKV_ATTN_MAX_SEGMENTS];
  int64_t end[PKV_ATTN_MAX_SEGMENTS];  // exclusive end of the segment in the concatenated key order
  const int64_t *idx[PKV_ATTN_MAX_SEGMENTS];  // per segment: selected rows (relative to row0) or nullptr
  int64_t idx_stride[PKV_ATTN_MAX_SEGMENTS], idx_limit[PKV_ATTN_MAX_SEGMENTS];
  int n;
};

// Row (inside the (b, h) slab of its segment, row0 included) and segment of concatenated key jj, packed as
// row | segment << 29.  Indexed segments cost one dependent 8-byte load.
__device__ __forceinline__ uint32_t att_resolve_row(const AttSegs &segs, int row, uint32_t jj) {
  int s = 0;
  uint32_t first = 0;
#pragma unroll
  for (int t = 1; t < PKV_ATTN_MAX_SEGMENTS; ++t)
    if (t < segs.n && jj >= (uint32_t)segs.end[t - 1]) s = t, first = (uint32_t)segs.end[t - 1];
  const int64_t *ip = segs.idx[0];
  int64_t stride = segs.idx_stride[0], limit = segs.idx_limit[0], row0 = segs.row0[0];
#pragma unroll
  for (int t = 1; t < PKV_ATTN_MAX_SEGMENTS; ++t)
    if (s == t) ip = segs.idx[t], stride = segs.idx_stride[t], limit = segs.idx_limit[t], row0 = segs.row0[t];
  int64_t r = jj - first;
  if (ip) {
    r = ip[(int64_t)row * stride + r];
    r = r < 0 ? 0 : (r >= limit ? limit - 1 : r);
  }
  return (uint32_t)(r + row0) | ((uint32_t)s << 29);
}

// Eight consecutive elements as loaded (16 B of bf16, or 32 B of fp32) and their fp32 values.  Kept
// apart so that a load can be issued a whole step before its data is touched.
template <bool BF16>
struct Raw8 {
  pkv_u32x4 a;
  pkv_u32x4 b[BF16 ? 0 : 1];
};

template <bool BF16>
__device__ __forceinline__ void load_raw8(const void *base, int64_t elem_off, Raw8<BF16> &r) {
  if (BF16) {
    r.a = __builtin_nontemporal_load((const pkv_u32x4 *)((const uint16_t *)base + elem_off));
  } else {
    r.a = __builtin_nontemporal_load((const pkv_u32x4 *)((const float *)base + elem_off));
    r.b[BF16 ? -1 : 0] = __builtin_nontemporal_load((const pkv_u32x4 *)((const float *)base + elem_off + 4));
  }
}

template <bool BF16>
__device__ __forceinline__ void expand8(const Raw8<BF16> &r, float (&x)[8]) {
  const uint32_t ww[4] = {r.a.x, r.a.y, r.a.z, r.a.w};
  if (BF16) {
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      x[2 * p] = __uint_as_float(ww[p] << 16);
      x[2 * p + 1] = __uint_as_float(ww[p] & 0xffff0000u);
    }
  } else {
    const pkv_u32x4 hi = r.b[BF16 ? -1 : 0];
    x[0] = __uint_as_float(ww[0]), x[1] = __uint_as_float(ww[1]), x[2] = __uint_as_float(ww[2]);
    x[3] = __uint_as_float(ww[3]), x[4] = __uint_as_float(hi.x), x[5] = __uint_as_float(hi.y);
    x[6] = __uint_as_float(hi.z), x[7] = __uint_as_float(hi.w);
  }
}

template <bool BF16>
__device__ __forceinline__ void load8(const void *base, int64_t elem_off, float (&x)[8]) {
  Raw8<BF16> r;
  load_raw8<BF16>(base, elem_off, r);
  expand8<BF16>(r, x);
}

// Partial results layout: ws[((row * n_splits + split) * G + g) * 130 + {0: max, 1: sum, 2..129: output}].
constexpr int kPartStride = 130;

template <bool BF16, int G, bool INDEXED>
__global__ __launch_bounds__(kAttThreads) void pkv_attn_partial_kernel(const void *__restrict__ q, int n_kv_heads,
                                                                       int group, int g0, int g_count, AttSegs segs,
                                                                       int64_t total, const int32_t *__restrict__ row_keys,
                                                                       int64_t per_split, float scale_log2e,
                                                                       float *__restrict__ ws) {
  const int split = blockIdx.x, row = blockIdx.y;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  const int tid = threadIdx.x;
  const int lane16 = tid & 15;        // owns dims 8*lane16 .. +7
  const int grp = tid >> 4;           // 16 key slots per workgroup step

  if (row_keys) {  // ragged rows: this (b, h) attends to its first row_keys[row] keys only
    const int64_t rk = row_keys[row];
    total = rk < total ? (rk > 0 ? rk : 1) : total;
  }
  const int64_t j0 = (int64_t)split * per_split;
  const int64_t j1 = (j0 + per_split < total) ? j0 + per_split : total;
  // per segment: byte address of this lane's 16 bytes of "concatenated key 0" (may lie before the tensor);
  // with indexed segments: of row 0 of the (b, h) slab
  const int esz = BF16 ? 2 : 4;
  const char *kb[PKV_ATTN_MAX_SEGMENTS], *vb[PKV_ATTN_MAX_SEGMENTS];
#pragma unroll
  for (int s = 0; s < PKV_ATTN_MAX_SEGMENTS; ++s) {
    const int64_t first = s == 0 ? 0 : segs.end[s - 1];
    const int64_t off = ((int64_t)b * segs.stride_b[s] + (int64_t)h * segs.stride_h[s] +
                         (INDEXED ? 0 : (segs.row0[s] - first) * 128) + 8 * lane16) * esz;
    kb[s] = (const char *)segs.k[s] + off;
    vb[s] = (const char *)segs.v[s] + off;
  }
  // K/V rows of the step after the current one are requested before the current one is consumed
  float kx[kAttUnroll][8], vx[kAttUnroll][8];
  Raw8<BF16> kn[kAttUnroll], vn[kAttUnroll];
  auto fetch = [&](int64_t jb, Raw8<BF16> (&kd)[kAttUnroll], Raw8<BF16> (&vd)[kAttUnroll]) {
#pragma unroll
    for (int u = 0; u < kAttUnroll; ++u) {
      const int64_t j = jb + u * kAttKeysPerIter + grp;
      const uint32_t jj = (uint32_t)(j < j1 ? j : j1 - 1);  // fewer than 2^24 keys
      const char *kp = kb[0], *vp = vb[0];
      uint32_t rownum = jj;
      if (INDEXED) {
        const uint32_t packed = att_resolve_row(segs, row, jj);
        rownum = packed & 0x1fffffffu;
#pragma unroll
        for (int s = 1; s < PKV_ATTN_MAX_SEGMENTS; ++s)
          if ((packed >> 29) == (uint32_t)s) kp = kb[s], vp = vb[s];
      } else {
#pragma unroll
        for (int s = 1; s < PKV_ATTN_MAX_SEGMENTS; ++s)
          if (s < segs.n && jj >= (uint32_t)segs.end[s - 1]) kp = kb[s], vp = vb[s];
      }
      const uint64_t boff = (uint64_t)rownum * (uint32_t)(128 * esz);
      load_raw8<BF16>(kp + boff, 0, kd[u]);
      load_raw8<BF16>(vp + boff, 0, vd[u]);
    }
  };
  if (j0 < j1) fetch(j0, kn, vn);  // before the queries: nothing here waits for them

  float qv[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {  // query heads g0 .. g0 + g_count - 1 of the KV head (g_count <= G; surplus slots idle)
    load8<BF16>(q, ((int64_t)row * group + g0 + (g < g_count ? g : 0)) * 128 + 8 * lane16, qv[g]);
#pragma unroll
    for (int d = 0; d < 8; ++d) qv[g][d] *= scale_log2e;  // scores come out in units of log2(e)
  }
  float m[G], l[G], o[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    m[g] = kNegBig, l[g] = 0.f;
#pragma unroll
    for (int d = 0; d < 8; ++d) o[g][d] = 0.f;
  }

  for (int64_t jb = j0; jb < j1; jb += kAttKeysPerIter * kAttUnroll) {
    bool valid[kAttUnroll];
#pragma unroll
    for (int u = 0; u < kAttUnroll; ++u) {
      valid[u] = jb + u * kAttKeysPerIter + grp < j1;
      expand8<BF16>(kn[u], kx[u]);
      expand8<BF16>(vn[u], vx[u]);
    }
    if (jb + kAttKeysPerIter * kAttUnroll < j1) fetch(jb + kAttKeysPerIter * kAttUnroll, kn, vn);
    float s[G][kAttUnroll];
#pragma unroll
    for (int g = 0; g < G; ++g) {
#pragma unroll
      for (int u = 0; u < kAttUnroll; ++u) {
        float acc = qv[g][0] * kx[u][0];
#pragma unroll
        for (int d = 1; d < 8; ++d) acc += qv[g][d] * kx[u][d];
        acc += pkv_lane_xor_f<1>(acc);
        acc += pkv_lane_xor_f<2>(acc);
        acc += pkv_lane_xor_f<4>(acc);
        acc += pkv_lane_xor_f<8>(acc);
        s[g][u] = valid[u] ? acc : kNegBig;
      }
    }
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float mn = m[g];
#pragma unroll
      for (int u = 0; u < kAttUnroll; ++u) mn = fmaxf(mn, s[g][u]);
      const float corr = exp2f(m[g] - mn);
      m[g] = mn;
      float p[kAttUnroll], psum = 0.f;
#pragma unroll
      for (int u = 0; u < kAttUnroll; ++u) {
        p[u] = valid[u] ? exp2f(s[g][u] - mn) : 0.f;
        psum += p[u];
      }
      l[g] = l[g] * corr + psum;
#pragma unroll
      for (int d = 0; d < 8; ++d) {
        float acc = o[g][d] * corr;
#pragma unroll
        for (int u = 0; u < kAttUnroll; ++u) acc += p[u] * vx[u][d];
        o[g][d] = acc;
      }
    }
  }

  // merge the 16 key slots of the workgroup through LDS
  __shared__ float s_m[16][G], s_l[16][G], s_o[16][G][128 + 4];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    if (lane16 == 0) s_m[grp][g] = m[g], s_l[grp][g] = l[g];
    *(float4 *)&s_o[grp][g][8 * lane16] = float4{o[g][0], o[g][1], o[g][2], o[g][3]};
    *(float4 *)&s_o[grp][g][8 * lane16 + 4] = float4{o[g][4], o[g][5], o[g][6], o[g][7]};
  }
  __syncthreads();
  float *part = ws + (((int64_t)row * gridDim.x + split) * group + g0) * kPartStride;
  for (int e = tid; e < g_count * 128; e += kAttThreads) {
    const int g = e >> 7, d = e & 127;
    float mn = s_m[0][g];
#pragma unroll
    for (int w = 1; w < 16; ++w) mn = fmaxf(mn, s_m[w][g]);
    float ls = 0.f, os = 0.f;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const float c = exp2f(s_m[w][g] - mn);
      ls += s_l[w][g] * c;
      os += s_o[w][g][d] * c;
    }
    part[g * kPartStride + 2 + d] = os;
    if (d == 0) part[g * kPartStride] = mn, part[g * kPartStride + 1] = ls;
  }
}

// ---- bf16 inputs: the same partial step on the matrix cores ----
//
// Each wave: 32 keys per step, v_mfma_f32_16x16x32_bf16 throughout.
//   scores:  S^T[key][head] = K[key][dim] . Q^T[dim][head]: A = 16 keys x 32 dims (lane (r, j) holds dims
//            32c + 8j .. +7 of key r: one 128-bit load), B = the query heads (zero columns past `group`),
//            4 instructions per 16 keys.  Lane (n, j) receives the scores of head n for keys 4j .. 4j+3 of the
//            tile - which is exactly where the next product wants the probabilities, so nothing is moved.
//   output:  O[head][dim] += P[head][key] . V[key][dim] over the 32 keys of two tiles: lane (n, j) supplies its
//            8 probabilities as A; for B it loads dims 8n .. 8n+7 of its 8 keys (rows read whole, 16 lanes per
//            row) and regroups them with byte permutes so that instruction m covers the dims 8n + m.
// The running maximum of head n lives in the lanes n, n+16, n+32, n+48; the output rows of head h live in lanes
// with j == h / 4.  group <= 16, all heads of the KV head in one pass.
typedef __bf16 pkv_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pkv_f32x4 __attribute__((ext_vector_type(4)));
constexpr int kMfmaStepKeys = 32;

__device__ __forceinline__ pkv_f32x4 mfma_bf16(pkv_u32x4 a, pkv_u32x4 b, pkv_f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(pkv_bf16x8, a), __builtin_bit_cast(pkv_bf16x8, b), c,
                                                 0, 0, 0);
}

__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return (uint32_t)pkv_f32_to_bf16_bits(lo) | ((uint32_t)pkv_f32_to_bf16_bits(hi) << 16);
}

constexpr int kMfmaWaves = 4;  // waves per workgroup: each takes a quarter of the split, merged through LDS

template <bool INDEXED>
__global__ __launch_bounds__(kMfmaWaves * PKV_WAVE) void pkv_attn_partial_mfma_kernel(
    const void *__restrict__ q, int n_kv_heads, int group, AttSegs segs, int64_t total,
    const int32_t *__restrict__ row_keys, int64_t per_split, float scale_log2e, float *__restrict__ ws) {
  const int split = blockIdx.x, row = blockIdx.y;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  const int lane = threadIdx.x & (PKV_WAVE - 1), wave = threadIdx.x / PKV_WAVE;
  const int n = lane & 15, j = lane >> 4;
  if (row_keys) {
    const int64_t rk = row_keys[row];
    total = rk < total ? (rk > 0 ? rk : 1) : total;
  }
  const int64_t per_wave = per_split / kMfmaWaves;  // a multiple of the 32 keys of one step
  const int64_t j0 = (int64_t)split * per_split + (int64_t)wave * per_wave;
  const int64_t j1 = (j0 + per_wave < total) ? j0 + per_wave : total;  // j1 <= j0: nothing left for this wave

  // per segment: byte address of "concatenated key 0" for this (b, h); with indexed segments: of row 0 of the slab
  const char *kb[PKV_ATTN_MAX_SEGMENTS], *vb[PKV_ATTN_MAX_SEGMENTS];
#pragma unroll
  for (int s = 0; s < PKV_ATTN_MAX_SEGMENTS; ++s) {
    const int64_t first = s == 0 ? 0 : segs.end[s - 1];
    const int64_t off = ((int64_t)b * segs.stride_b[s] + (int64_t)h * segs.stride_h[s] +
                         (INDEXED ? 0 : (segs.row0[s] - first) * 128)) * 2;
    kb[s] = (const char *)segs.k[s] + off;
    vb[s] = (const char *)segs.v[s] + off;
  }
  // INDEXED: lane l holds the resolved row of key blk0 + l for the current block of 64 keys (two steps);
  // the rows a lane needs are then fetched from the owning lanes, so the index loads are one per key.
  uint32_t my_row = 0;
  int64_t blk0 = j0;
  auto row_ptr = [&](const char *const (&base)[PKV_ATTN_MAX_SEGMENTS], int64_t key) {
    const uint32_t jj = (uint32_t)(key < j1 ? key : j1 - 1);
    const char *p = base[0];
    if (INDEXED) {
      const uint32_t packed = (uint32_t)__shfl((int)my_row, (int)(jj - (uint32_t)blk0), PKV_WAVE);
#pragma unroll
      for (int s = 1; s < PKV_ATTN_MAX_SEGMENTS; ++s)
        if ((packed >> 29) == (uint32_t)s) p = base[s];
      return p + (uint64_t)(packed & 0x1fffffffu) * 256u;
    }
#pragma unroll
    for (int s = 1; s < PKV_ATTN_MAX_SEGMENTS; ++s)
      if (s < segs.n && jj >= (uint32_t)segs.end[s - 1]) p = base[s];
    return p + jj * 256u;
  };

  const pkv_u32x4 zero4 = {0u, 0u, 0u, 0u};
  pkv_u32x4 qb[4];
#pragma unroll
  for (int c = 0; c < 4; ++c)
    qb[c] = n < group ? *(const pkv_u32x4 *)((const uint16_t *)q + ((int64_t)row * group + n) * 128 + 32 * c + 8 * j) : zero4;

  float m_run = kNegBig, l_part = 0.f;
  pkv_f32x4 o[8];
#pragma unroll
  for (int m = 0; m < 8; ++m) o[m] = pkv_f32x4{0.f, 0.f, 0.f, 0.f};

  for (int64_t jb = j0; jb < j1; jb += kMfmaStepKeys) {
    if (INDEXED && ((jb - j0) & (PKV_WAVE - 1)) == 0) {
      blk0 = jb;
      const int64_t key = jb + lane;
      my_row = att_resolve_row(segs, row, (uint32_t)(key < j1 ? key : j1 - 1));
    }
    // K: two tiles of 16 keys, lane (n, j) reads dims 32c + 8j .. +7 of key jb + 16t + n
    pkv_u32x4 ka[2][4], vr[8];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const char *kp = row_ptr(kb, jb + 16 * t + n) + 16 * j;
#pragma unroll
      for (int c = 0; c < 4; ++c) ka[t][c] = __builtin_nontemporal_load((const pkv_u32x4 *)(kp + 64 * c));
    }
    // V: dims 8n .. 8n+7 of the 8 keys whose probabilities this lane will hold
#pragma unroll
    for (int e = 0; e < 8; ++e)
      vr[e] = __builtin_nontemporal_load((const pkv_u32x4 *)(row_ptr(vb, jb + 16 * (e >> 2) + 4 * j + (e & 3)) + 16 * n));

    pkv_f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      s0 = mfma_bf16(ka[0][c], qb[c], s0);
      s1 = mfma_bf16(ka[1][c], qb[c], s1);
    }
    float sc[8];
    bool valid[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      valid[e] = jb + 16 * (e >> 2) + 4 * j + (e & 3) < j1;
      const float raw = (e < 4) ? s0[e & 3] : s1[e & 3];
      sc[e] = valid[e] ? raw * scale_log2e : kNegBig;
    }
    float mx = sc[0];
#pragma unroll
    for (int e = 1; e < 8; ++e) mx = fmaxf(mx, sc[e]);
    mx = fmaxf(mx, __shfl_xor(mx, 16, PKV_WAVE));
    mx = fmaxf(mx, __shfl_xor(mx, 32, PKV_WAVE));
    const float m_new = fmaxf(m_run, mx);
    const float corr = exp2f(m_run - m_new);
    m_run = m_new;
    float p[8], psum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      p[e] = valid[e] ? exp2f(sc[e] - m_new) : 0.f;
      psum += p[e];
    }
    l_part = l_part * corr + psum;
    const pkv_u32x4 pa = {pack_bf16x2(p[0], p[1]), pack_bf16x2(p[2], p[3]), pack_bf16x2(p[4], p[5]),
                          pack_bf16x2(p[6], p[7])};
    // the output rows of this lane belong to heads 4j .. 4j+3: fetch their correction factors
    float cr[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) cr[i] = __shfl(corr, 4 * j + i, PKV_WAVE);
#pragma unroll
    for (int m = 0; m < 8; ++m) {
      // element m of each of the eight V vectors: dword m/2, half m%2
      const uint32_t sel = (m & 1) ? 0x07060302u : 0x05040100u;
      pkv_u32x4 bm;
      bm.x = __builtin_amdgcn_perm(vr[1][m >> 1], vr[0][m >> 1], sel);
      bm.y = __builtin_amdgcn_perm(vr[3][m >> 1], vr[2][m >> 1], sel);
      bm.z = __builtin_amdgcn_perm(vr[5][m >> 1], vr[4][m >> 1], sel);
      bm.w = __builtin_amdgcn_perm(vr[7][m >> 1], vr[6][m >> 1], sel);
      pkv_f32x4 acc = o[m];
      acc.x *= cr[0], acc.y *= cr[1], acc.z *= cr[2], acc.w *= cr[3];
      o[m] = mfma_bf16(pa, bm, acc);
    }
  }

  l_part += __shfl_xor(l_part, 16, PKV_WAVE);
  l_part += __shfl_xor(l_part, 32, PKV_WAVE);
  // merge the waves of the workgroup: every wave leaves (max, sum, output) of its keys in LDS, then the
  // workgroup's 256 threads combine them, one (head, dim) pair at a time.  group <= 8.
  __shared__ float s_m[kMfmaWaves][8], s_l[kMfmaWaves][8], s_o[kMfmaWaves][8][128 + 4];
  if (j == 0 && n < group) s_m[wave][n] = m_run, s_l[wave][n] = l_part;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int head = 4 * j + i;
    if (head < group) {
      *(float4 *)&s_o[wave][head][8 * n] = float4{o[0][i], o[1][i], o[2][i], o[3][i]};
      *(float4 *)&s_o[wave][head][8 * n + 4] = float4{o[4][i], o[5][i], o[6][i], o[7][i]};
    }
  }
  __syncthreads();
  float *part = ws + ((int64_t)row * gridDim.x + split) * group * kPartStride;
  for (int e = threadIdx.x; e < group * 128; e += kMfmaWaves * PKV_WAVE) {
    const int g = e >> 7, d = e & 127;
    float mn = s_m[0][g];
#pragma unroll
    for (int w = 1; w < kMfmaWaves; ++w) mn = fmaxf(mn, s_m[w][g]);
    float ls = 0.f, os = 0.f;
#pragma unroll
    for (int w = 0; w < kMfmaWaves; ++w) {
      const float c = exp2f(s_m[w][g] - mn);
      ls += s_l[w][g] * c;
      os += s_o[w][g][d] * c;
    }
    part[g * kPartStride + 2 + d] = os;
    if (d == 0) part[g * kPartStride] = mn, part[g * kPartStride + 1] = ls;
  }
}

// grid R, G*128 threads: merge the splits (at most 64) and normalise.
template <bool BF16>
__global__ void pkv_attn_merge_kernel(const float *__restrict__ ws, int n_splits, int G, void *__restrict__ out) {
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const int g = tid >> 7, d = tid & 127;
  __shared__ float s_w[8][64];   // weight of split s for head g, already divided by the total
  const float *rowp = ws + (int64_t)row * n_splits * G * kPartStride;
  // the first 16 splits' partial outputs are requested before the weights are known: one memory round trip
  // instead of two for the usual case (a few thousand keys)
  constexpr int kEarly = 16;
  const float *po = rowp + (int64_t)g * kPartStride + 2 + d;
  float early[kEarly];
#pragma unroll
  for (int s = 0; s < kEarly; ++s) early[s] = s < n_splits ? po[(int64_t)s * G * kPartStride] : 0.f;
  if (d < PKV_WAVE) {  // one wave per head: lane = split
    const bool live = d < n_splits;
    const float *p = rowp + ((int64_t)(live ? d : 0) * G + g) * kPartStride;
    const float mi = live ? p[0] : kNegBig, li = live ? p[1] : 0.f;
    float mn = mi;
#pragma unroll
    for (int x = 1; x < PKV_WAVE; x <<= 1) mn = fmaxf(mn, __shfl_xor(mn, x, PKV_WAVE));
    const float c = exp2f(mi - mn);
    float tot = li * c;
#pragma unroll
    for (int x = 1; x < PKV_WAVE; x <<= 1) tot += __shfl_xor(tot, x, PKV_WAVE);
    s_w[g][d] = c / tot;
  }
  __syncthreads();
  float os = 0.f;
#pragma unroll
  for (int s = 0; s < kEarly; ++s) os += early[s] * (s < n_splits ? s_w[g][s] : 0.f);
#pragma unroll 8
  for (int s = kEarly; s < n_splits; ++s) os += po[(int64_t)s * G * kPartStride] * s_w[g][s];
  const int64_t oi = ((int64_t)row * G + g) * 128 + d;
  if (BF16)
    ((uint16_t *)out)[oi] = pkv_f32_to_bf16_bits(os);
  else
    ((float *)out)[oi] = os;
}

int pick_splits(int rows, int64_t total) {
  // One round of workgroups: with four query heads the kernel holds 3 workgroups per CU (768 on the chip);
  // a few more would run as a second round and double the launch's duration.
  int64_t s = 768 / rows;
  const int64_t max_by_len = (total + 63) / 64;  // at least 64 keys per split
  if (s > max_by_len) s = max_by_len;
  if (s > 64) s = 64;
  if (s < 1) s = 1;
  return (int)s;
}

// Matrix-core path: four waves per workgroup, one 32-key step per wave while that keeps the split count within
// the 64 the merge kernel takes (every load of the workgroup is then in flight at once); longer key sets give
// each wave more steps.
int pick_splits_mfma(int rows, int64_t total) {
  (void)rows;
  int64_t s = (total + kMfmaWaves * kMfmaStepKeys - 1) / (kMfmaWaves * kMfmaStepKeys);
  if (s > 64) s = 64;
  if (s < 1) s = 1;
  return (int)s;
}

}  // namespace

extern "C" size_t pkv_decode_attention_ws_bytes(int bs, int n_kv_heads, int group, int64_t total_keys) {
  if (bs <= 0 || n_kv_heads <= 0 || group <= 0 || total_keys <= 0) return 256;
  // room for the largest split count either path uses (64), whatever the key count and dtype
  return pkv_align_up((size_t)bs * n_kv_heads * 64 * group * kPartStride * sizeof(float), 256);
}

extern "C" int pkv_decode_attention(const void *q, int dtype, int bs, int n_kv_heads, int group,
                                    const pkv_attn_segment *segments, int n_segments, const int32_t *row_keys,
                                    float scale, void *out, void *ws, size_t ws_bytes, void *stream) {
  PKV_REQUIRE(q && segments && out && ws, "pkv_decode_attention: null pointer");
  PKV_REQUIRE(dtype == PKV_DTYPE_F32 || dtype == PKV_DTYPE_BF16, "unknown dtype %d", dtype);
  PKV_REQUIRE(bs > 0 && n_kv_heads > 0 && (int64_t)bs * n_kv_heads <= 65535, "bad shape bs=%d kv_heads=%d", bs,
              n_kv_heads);
  PKV_REQUIRE(group >= 1 && group <= 8, "GQA group must be in [1, 8] (got %d)", group);
  PKV_REQUIRE(n_segments >= 1 && n_segments <= PKV_ATTN_MAX_SEGMENTS, "1..%d key segments", PKV_ATTN_MAX_SEGMENTS);
  PKV_REQUIRE(pkv_aligned(q, 16) && pkv_aligned(out, 4), "q must be 16-byte aligned");
  const int64_t vec = dtype == PKV_DTYPE_BF16 ? 8 : 4;
  AttSegs sg;
  memset(&sg, 0, sizeof sg);
  int64_t total = 0;
  bool indexed = false;
  for (int i = 0; i < n_segments; ++i) {
    const pkv_attn_segment &s = segments[i];
    PKV_REQUIRE(s.n_rows >= 0 && s.row0 >= 0, "segment %d: negative extent", i);
    if (s.n_rows == 0) continue;
    PKV_REQUIRE(s.k && s.v, "segment %d: null K/V", i);
    PKV_REQUIRE(pkv_aligned(s.k, 16) && pkv_aligned(s.v, 16) && s.stride_b % vec == 0 && s.stride_h % vec == 0,
                "segment %d: K/V must be 16-byte aligned with 16-byte-multiple strides", i);
    sg.k[sg.n] = s.k, sg.v[sg.n] = s.v;
    sg.stride_b[sg.n] = s.stride_b, sg.stride_h[sg.n] = s.stride_h;
    sg.row0[sg.n] = s.row0;
    if (s.idx) {
      PKV_REQUIRE(pkv_aligned(s.idx, 8) && s.idx_stride >= s.n_rows && s.idx_limit > 0 &&
                      s.row0 + s.idx_limit < ((int64_t)1 << 29),
                  "segment %d: indexed rows need idx_stride >= n_rows and 0 < idx_limit (row0 + idx_limit < 2^29)", i);
      sg.idx[sg.n] = s.idx, sg.idx_stride[sg.n] = s.idx_stride, sg.idx_limit[sg.n] = s.idx_limit;
      indexed = true;
    }
    total += s.n_rows;
    sg.end[sg.n] = total;
    ++sg.n;
  }
  PKV_REQUIRE(total > 0, "pkv_decode_attention: no keys");
  PKV_REQUIRE(total < ((int64_t)1 << 23), "pkv_decode_attention: at most 2^23 - 1 keys (got %lld)", (long long)total);
  const int rows = bs * n_kv_heads;
  const bool bf = dtype == PKV_DTYPE_BF16;
  const int n_splits = bf ? pick_splits_mfma(rows, total) : pick_splits(rows, total);
  const size_t need = (size_t)rows * n_splits * group * kPartStride * sizeof(float);
  if (ws_bytes < need || !pkv_aligned(ws, 16)) {
    pkv_set_error("pkv_decode_attention: workspace of %zu bytes required, got %zu", need, ws_bytes);
    return PKV_ENOMEM;
  }
  const int step = bf ? kMfmaWaves * kMfmaStepKeys : kAttKeysPerIter * kAttUnroll;
  int64_t per_split = (total + n_splits - 1) / n_splits;
  per_split = (per_split + step - 1) / step * step;
  const float scale_log2e = scale * 1.4426950408889634f;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)n_splits, (unsigned)rows);
  if (bf) {
    if (indexed)
      hipLaunchKernelGGL(pkv_attn_partial_mfma_kernel<true>, grid, dim3(kMfmaWaves * PKV_WAVE), 0, s, q, n_kv_heads, group, sg, total,
                         row_keys, per_split, scale_log2e, (float *)ws);
    else
      hipLaunchKernelGGL(pkv_attn_partial_mfma_kernel<false>, grid, dim3(kMfmaWaves * PKV_WAVE), 0, s, q, n_kv_heads, group, sg, total,
                         row_keys, per_split, scale_log2e, (float *)ws);
  } else {
#define PKV_ATT(GG, G0, GC, IDX)                                                                                  \
  hipLaunchKernelGGL((pkv_attn_partial_kernel<false, GG, IDX>), grid, dim3(kAttThreads), 0, s, q, n_kv_heads, group, G0, \
                     GC, sg, total, row_keys, per_split, scale_log2e, (float *)ws)
#define PKV_ATT_G(G0, GC, IDX)            \
  do {                                    \
    if (GC == 1) PKV_ATT(1, G0, GC, IDX); \
    else if (GC == 2) PKV_ATT(2, G0, GC, IDX); \
    else PKV_ATT(4, G0, GC, IDX);         \
  } while (0)
    for (int g0 = 0; g0 < group; g0 += 4) {  // four query heads per launch: more would not fit the registers
      const int gc = group - g0 < 4 ? group - g0 : 4;
      if (indexed) PKV_ATT_G(g0, gc, true); else PKV_ATT_G(g0, gc, false);
    }
#undef PKV_ATT_G
#undef PKV_ATT
  }
  PKV_LAUNCH_CHECK("pkv_attn_partial_kernel");
  if (bf)
    hipLaunchKernelGGL(pkv_attn_merge_kernel<true>, dim3((unsigned)rows), dim3(group * 128), 0, s, (const float *)ws,
                       n_splits, group, out);
  else
    hipLaunchKernelGGL(pkv_attn_merge_kernel<false>, dim3((unsigned)rows), dim3(group * 128), 0, s, (const float *)ws,
                       n_splits, group, out);
  PKV_LAUNCH_CHECK("pkv_attn_merge_kernel");
  return PKV_OK;
}
