// Dense decode attention over the gathered key set: softmax(q k^T * scale) v for ONE
// query token per sequence, GQA (the G query heads of a KV head share its keys), over
// up to four row segments of head_dim 128 (sink | update buffer | gathered top-k |
// local window), non-causal.
//
// Reference: cache_hub/polar_cache.py:1084-1105 (torch.cat of the segments, then
// flash_attn_func on [bs, S, H, D]); here the segments are read where they lie.
//
// HBM-bound: 512 B (one K row + one V row, bf16) per key and KV head, read once for
// all G query heads.  Split over the key axis (flash-decoding): grid (n_splits, R),
// every 16 lanes own one key at a time (16 B of K and of V per lane, so a wave
// instruction moves four whole rows), keep a running (max, sum, output) per query
// head, and the partial results are merged first inside the workgroup, then across
// splits by a second small launch.
//
// Arithmetic: products and sums in fp32, exp2 with the scale folded in; the output is
// rounded to the input dtype.  Not bit-reproducible against another summation order -
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
  int n;
};

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

template <bool BF16, int G>
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
  // per segment: byte address of this lane's 16 bytes of "concatenated key 0" (may lie before the tensor)
  const int esz = BF16 ? 2 : 4;
  const char *kb[PKV_ATTN_MAX_SEGMENTS], *vb[PKV_ATTN_MAX_SEGMENTS];
#pragma unroll
  for (int s = 0; s < PKV_ATTN_MAX_SEGMENTS; ++s) {
    const int64_t first = s == 0 ? 0 : segs.end[s - 1];
    const int64_t off = ((int64_t)b * segs.stride_b[s] + (int64_t)h * segs.stride_h[s] +
                         (segs.row0[s] - first) * 128 + 8 * lane16) * esz;
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
#pragma unroll
      for (int s = 1; s < PKV_ATTN_MAX_SEGMENTS; ++s)
        if (s < segs.n && jj >= (uint32_t)segs.end[s - 1]) kp = kb[s], vp = vb[s];
      const uint32_t boff = jj * (uint32_t)(128 * esz);
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

  if (j0 < j1) fetch(j0, kn, vn);
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

// grid R, G*128 threads: merge the splits (at most 64) and normalise.
template <bool BF16>
__global__ void pkv_attn_merge_kernel(const float *__restrict__ ws, int n_splits, int G, void *__restrict__ out) {
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const int g = tid >> 7, d = tid & 127;
  __shared__ float s_w[8][64];   // weight of split s for head g, already divided by the total
  const float *rowp = ws + (int64_t)row * n_splits * G * kPartStride;
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
  const float *po = rowp + (int64_t)g * kPartStride + 2 + d;
#pragma unroll 8
  for (int s = 0; s < n_splits; ++s) os += po[(int64_t)s * G * kPartStride] * s_w[g][s];
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

}  // namespace

extern "C" size_t pkv_decode_attention_ws_bytes(int bs, int n_kv_heads, int group, int64_t total_keys) {
  if (bs <= 0 || n_kv_heads <= 0 || group <= 0 || total_keys <= 0) return 256;
  const int rows = bs * n_kv_heads;
  return pkv_align_up((size_t)rows * pick_splits(rows, total_keys) * group * kPartStride * sizeof(float), 256);
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
    total += s.n_rows;
    sg.end[sg.n] = total;
    ++sg.n;
  }
  PKV_REQUIRE(total > 0, "pkv_decode_attention: no keys");
  PKV_REQUIRE(total < ((int64_t)1 << 23), "pkv_decode_attention: at most 2^23 - 1 keys (got %lld)", (long long)total);
  const int rows = bs * n_kv_heads;
  const int n_splits = pick_splits(rows, total);
  const size_t need = (size_t)rows * n_splits * group * kPartStride * sizeof(float);
  if (ws_bytes < need || !pkv_aligned(ws, 16)) {
    pkv_set_error("pkv_decode_attention: workspace of %zu bytes required, got %zu", need, ws_bytes);
    return PKV_ENOMEM;
  }
  const int step = kAttKeysPerIter * kAttUnroll;
  int64_t per_split = (total + n_splits - 1) / n_splits;
  per_split = (per_split + step - 1) / step * step;
  const float scale_log2e = scale * 1.4426950408889634f;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)n_splits, (unsigned)rows);
#define PKV_ATT(BF, GG, G0, GC)                                                                                  \
  hipLaunchKernelGGL((pkv_attn_partial_kernel<BF, GG>), grid, dim3(kAttThreads), 0, s, q, n_kv_heads, group, G0, GC, \
                     sg, total, row_keys, per_split, scale_log2e, (float *)ws)
  const bool bf = dtype == PKV_DTYPE_BF16;
  for (int g0 = 0; g0 < group; g0 += 4) {  // four query heads per launch: more would not fit the registers
    const int gc = group - g0 < 4 ? group - g0 : 4;
    if (gc == 1) { if (bf) PKV_ATT(true, 1, g0, gc); else PKV_ATT(false, 1, g0, gc); }
    else if (gc == 2) { if (bf) PKV_ATT(true, 2, g0, gc); else PKV_ATT(false, 2, g0, gc); }
    else { if (bf) PKV_ATT(true, 4, g0, gc); else PKV_ATT(false, 4, g0, gc); }
  }
#undef PKV_ATT
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
