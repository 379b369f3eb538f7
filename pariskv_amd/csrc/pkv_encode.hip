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
//
// The kernel is bound by vector-instruction issue, not by HBM.  fp32 keys take
// enc_key_exact (correctly rounded divisions and roots, about 700 instructions
// per lane and key); bf16 keys take enc_key_fast (about 300), which reaches the
// same bits through reciprocals, a table for the magnitude code and centre, and
// lane-crossing adds folded into one instruction, and hands a wave over to
// enc_key_exact when one of its keys is outside the range where that is proven.
#include "pkv_common.h"

namespace {

constexpr int kEncThreads = 256;
constexpr int kEncKeysPerIter = kEncThreads / 16;  // 16
constexpr int kEncKeysPerWg = 256;

__constant__ float c_thresholds[7] = {0.08447265625f, 0.169921875f, 0.2578125f, 0.349609375f,
                                      0.44921875f,    0.55859375f,  0.69140625f};
__constant__ float c_centers[8] = {0.0419921875f, 0.126953125f, 0.212890625f, 0.302734375f,
                                   0.396484375f,  0.5f,         0.6171875f,   0.76171875f};

// Adds a workgroup's 16 x 256 histogram to a row's cluster sizes.  Two neighbouring counters travel in one 64-bit
// atomic where the row is 8-byte aligned (a counter would have to pass 2^32 to carry into its neighbour; they
// count keys of one sequence), which halves the atomics the launch sends to L2.
__device__ __forceinline__ void pkv_flush_cluster_hist(const uint32_t *s_hist, int32_t *cc, int tid, int n_threads) {
  if (((uintptr_t)cc & 7) == 0) {
    for (int i = tid; i < 16 * 256 / 2; i += n_threads) {
      const uint64_t v = (uint64_t)s_hist[2 * i] | ((uint64_t)s_hist[2 * i + 1] << 32);
      if (v) atomicAdd((unsigned long long *)cc + i, (unsigned long long)v);
    }
  } else {
    for (int i = tid; i < 16 * 256; i += n_threads) {
      const uint32_t v = s_hist[i];
      if (v) atomicAdd(&cc[i], (int32_t)v);
    }
  }
}

struct EncOut {
  uint32_t code;    // sign code of the lane's block
  uint32_t packed;  // eight 4-bit (sign, magnitude) codes
  uint32_t wbits;   // rerank weight, bf16 bits
};

// One key's block, every operation in the reference's order with correctly rounded division and square root.
// BF16 = the rounding chain of the reference's bf16 tensors (compile-time, so that no rounding point branches).
template <bool BF16>
__device__ __forceinline__ void enc_key_exact(const float (&x)[8], const float (&sg)[8], int s, bool rerank,
                                              const float *s_centers, EncOut &o) {
  constexpr int dtype = BF16 ? PKV_DTYPE_BF16 : PKV_DTYPE_F32;
  float y[8];
  const float n = pkv_normalize_rotate_16(x, sg, s, dtype, y);
  uint32_t code = 0;
#pragma unroll
  for (int j = 0; j < 8; ++j) code |= (y[j] >= 0.0f) ? (1u << j) : 0u;
  o.code = code;
  if (!rerank) return;
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
  o.packed = packed;
  o.wbits = pkv_f32_to_bf16_bits((r / alpha) * n);
}

// ---- bf16 keys: the same results from reciprocals -----------------------------------------------------------
//
// Both division families of the bf16 chain divide a bf16 value by a bf16 value and round the fp32 quotient to
// bf16.  Write the operands as mx * 2^a and md * 2^b with integer significands in [128, 255].  A rounding
// boundary of bf16 (the midpoint of two neighbouring bf16 numbers) has a 9-bit significand, so
//   | mx / md - boundary | = | mx * 2^k - o * md | / (md * 2^k)   with k = 8 or 9 and o odd,
// which is zero only if md is a power of two (then the quotient is itself a bf16 number, not a boundary) and is
// otherwise at least 1 / (255 * 512): a relative distance above 2^-18 from every boundary.  x * rcp(d) with the
// hardware reciprocal (1 ulp) is within 2^-22 of the quotient, and so is the correctly rounded fp32 quotient:
// both round to the same bf16.  This holds while the quotient is a normal number, which the range checks below
// guarantee; a key that fails them is encoded by enc_key_exact instead.  The two square roots have no such
// structure: the hardware square root (1 ulp) is used unless it lands within 4 ulp of a bf16 rounding boundary.

constexpr int kMagTableBits = 10;                    // bf16 patterns 0x3C00 .. 0x3FFF: 2^-7 <= |u| < 2
constexpr uint32_t kMagTableLo = 0x3C000000u, kMagTableHi = 0x3FFF0000u;

template <int CTRL>
__device__ __forceinline__ float enc_dpp(float v) {  // bound_ctrl set, so that the move folds into the add that uses it
  return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float enc_flip(float v, uint32_t sign_mask) {
  return __uint_as_float(__float_as_uint(v) ^ sign_mask);
}

// v + (value of lane ^ 4): banks 0 and 2 of a row of 16 lanes read four lanes up, banks 1 and 3 four lanes down.
// The leading wait covers the two states the hardware needs between a vector write and a lane-crossing read of
// the same register.
__device__ __forceinline__ float enc_sum_xor4(float v) {
  float d;
  asm("s_nop 1\n\t"
      "v_add_f32_dpp %0, %1, %1 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_add_f32_dpp %0, %1, %1 row_shr:4 row_mask:0xf bank_mask:0xa"
      : "=&v"(d)
      : "v"(v));
  return d;
}

// Walsh-Hadamard stage across lane ^ 4 for eight values: lanes with bit 2 clear get t + other, the rest other - t.
__device__ __forceinline__ void enc_butterfly_xor4(float (&t)[8]) {
  float d[8];
  asm("s_nop 1\n\t"
      "v_add_f32_dpp %0, %8, %8 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_sub_f32_dpp %0, %8, %8 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %1, %9, %9 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_sub_f32_dpp %1, %9, %9 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %2, %10, %10 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_sub_f32_dpp %2, %10, %10 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %3, %11, %11 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_sub_f32_dpp %3, %11, %11 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %4, %12, %12 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_sub_f32_dpp %4, %12, %12 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %5, %13, %13 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_sub_f32_dpp %5, %13, %13 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %6, %14, %14 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_sub_f32_dpp %6, %14, %14 row_shr:4 row_mask:0xf bank_mask:0xa\n\t"
      "v_add_f32_dpp %7, %15, %15 row_shl:4 row_mask:0xf bank_mask:0x5\n\t"
      "v_sub_f32_dpp %7, %15, %15 row_shr:4 row_mask:0xf bank_mask:0xa"
      : "=&v"(d[0]), "=&v"(d[1]), "=&v"(d[2]), "=&v"(d[3]), "=&v"(d[4]), "=&v"(d[5]), "=&v"(d[6]), "=&v"(d[7])
      : "v"(t[0]), "v"(t[1]), "v"(t[2]), "v"(t[3]), "v"(t[4]), "v"(t[5]), "v"(t[6]), "v"(t[7]));
#pragma unroll
  for (int j = 0; j < 8; ++j) t[j] = d[j];
}

// bf16(sqrt(a)) from the hardware square root (1 ulp); where the fp32 root lies within 4 ulp of a bf16 rounding
// boundary the correctly rounded root decides.
__device__ __forceinline__ float enc_sqrt_bf16(float a) {
  float r = __builtin_amdgcn_sqrtf(a);
  if ((__float_as_uint(r) & 0xffffu) - 0x7ffcu < 9u) {
    asm volatile("" ::: "memory");  // keeps the rare case a branch: without it both roots are computed every time
    r = sqrtf(a);
  }
  return pkv_bf16_round(r);
}

__device__ __forceinline__ float enc_min_abs8(const float (&v)[8]) {
  float m = __builtin_fminf(__builtin_fminf(fabsf(v[0]), fabsf(v[1])), fabsf(v[2]));
  m = __builtin_fminf(__builtin_fminf(m, fabsf(v[3])), fabsf(v[4]));
  m = __builtin_fminf(__builtin_fminf(m, fabsf(v[5])), fabsf(v[6]));
  return __builtin_fminf(m, fabsf(v[7]));
}

// The bf16 chain of enc_key_exact without a division.  w[] = the lane's eight bf16 components as loaded (two per
// word), sgw[] = the SRHT sign bits in the same packing.  Returns true when this lane's key needs enc_key_exact
// (norm or radius outside [1e-8, 2^60], or a component below 2^-40 in magnitude, zero included); o is then
// unspecified.  sm1/sm2/sm8 = the sign bit where the lane's block index has bit 0/1/3 set.  s_mag[p - 0x3C00] =
// {magnitude code, magnitude centre} for the bf16 pattern p of |u|; s_spread[c] = bit j of the sign code c moved to
// bit 4j + 3.
__device__ __forceinline__ bool enc_key_fast(const uint32_t (&w)[4], const uint32_t (&sgw)[4], uint32_t sm1,
                                             uint32_t sm2, uint32_t sm8, bool rerank, const uint2 *s_mag,
                                             const uint32_t *s_spread, EncOut &o) {
  float x[8];  // components times their SRHT sign: the sign commutes with the division and its rounding
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    const uint32_t v = w[p] ^ sgw[p];
    x[2 * p] = __uint_as_float(v << 16);
    x[2 * p + 1] = __uint_as_float(v & 0xffff0000u);
  }
  // the square of a bf16 value of magnitude in [2^-40, 2^60] is exact in fp32 (16 significant bits, a normal
  // number), so a fused multiply-add rounds once, to the same bits as the product and the sum rounded in turn; a key
  // with a component outside that range is handed to enc_key_exact whatever is computed here
  float acc = x[0] * x[0];
#pragma unroll
  for (int j = 1; j < 8; ++j) acc = __builtin_fmaf(x[j], x[j], acc);
  acc = enc_dpp<0xB1>(acc) + acc;   // lane ^ 1
  acc = enc_dpp<0x4E>(acc) + acc;   // lane ^ 2
  acc = enc_sum_xor4(acc);
  acc = enc_dpp<0x128>(acc) + acc;  // lane ^ 8
  const float n = enc_sqrt_bf16(acc);
  bool bad = !(n >= 1e-8f) || n > 0x1p60f;
  bad |= enc_min_abs8(x) < 0x1p-40f;
  const float n_inv = __builtin_amdgcn_rcpf(n);
  float t[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) t[j] = pkv_bf16_round(x[j] * n_inv);
#pragma unroll
  for (int hh = 1; hh < 8; hh <<= 1) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if ((i & hh) == 0) {
        const float a = t[i], c = t[i + hh];
        t[i] = a + c;
        t[i + hh] = a - c;
      }
    }
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) t[j] = enc_dpp<0xB1>(t[j]) + enc_flip(t[j], sm1);
#pragma unroll
  for (int j = 0; j < 8; ++j) t[j] = enc_dpp<0x4E>(t[j]) + enc_flip(t[j], sm2);
  enc_butterfly_xor4(t);
#pragma unroll
  for (int j = 0; j < 8; ++j) t[j] = enc_dpp<0x128>(t[j]) + enc_flip(t[j], sm8);
  float y[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = pkv_bf16_round(t[j] * PKV_HADAMARD_SCALE);
  bad |= enc_min_abs8(y) < 0x1p-40f;  // no zeros from here on: y >= 0 is the sign bit
  uint32_t sneg = 0;
#pragma unroll
  for (int j = 7; j >= 0; --j) sneg = __builtin_amdgcn_alignbit(sneg, __float_as_uint(y[j]), 31);
  o.code = ~sneg & 0xffu;
  if (!rerank) return bad;

  float r2 = y[0] * y[0];  // y: bf16 values, magnitudes checked above: exact squares again
#pragma unroll
  for (int j = 1; j < 8; ++j) r2 = __builtin_fmaf(y[j], y[j], r2);
  const float r = enc_sqrt_bf16(r2);
  bad |= !(r >= 1e-8f) || r > 0x1p60f;
  const float r_inv = __builtin_amdgcn_rcpf(r);
  float au[8];
  uint2 e[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    au[j] = fabsf(pkv_bf16_round(y[j] * r_inv));
    const float cl = __builtin_amdgcn_fmed3f(au[j], __uint_as_float(kMagTableLo), __uint_as_float(kMagTableHi));
    const uint32_t byte_off = __builtin_amdgcn_ubfe(__float_as_uint(cl), 13, kMagTableBits + 3);  // 8 * (pattern - 0x3C00)
    e[j] = *(const uint2 *)((const char *)s_mag + byte_off);
  }
  uint32_t mags = 0;
  float alpha = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    mags = __builtin_amdgcn_alignbit(e[j].x, mags, 4);  // the code enters at the top nibble; after 8 steps code j sits in nibble j
    const float p = pkv_bf16_round(__uint_as_float(e[j].y) * au[j]);
    alpha = (j == 0) ? p : alpha + p;
  }
  if (alpha < 1e-6f) alpha = 1e-6f;
  o.packed = (mags & 0x77777777u) | s_spread[o.code];  // bit 3 of nibble j = bit j of the sign code
  // (r / alpha) * n: both forms are within 2^-22 of the exact value, at most 6 ulp apart; the reciprocal form
  // decides the bf16 rounding unless it lies within 8 ulp of a rounding boundary
  float wt = (r * __builtin_amdgcn_rcpf(alpha)) * n;
  if ((__float_as_uint(wt) & 0xffffu) - 0x7ff8u < 17u) wt = (r / alpha) * n;
  o.wbits = pkv_f32_to_bf16_bits(wt);
  return bad;
}

template <bool BF16>
__global__ __launch_bounds__(kEncThreads) __attribute__((amdgpu_waves_per_eu(6, 6))) void pkv_encode_kernel(
    const void *__restrict__ keys, int n_kv_heads, int64_t n_keys, int64_t k_stride_b, int64_t k_stride_h,
    int64_t k_stride_key, const float *__restrict__ signs, uint8_t *__restrict__ codes, int64_t cs_b, int64_t cs_h,
    int64_t cs_key, int64_t cs_sub, uint8_t *__restrict__ nib, int64_t ns_b, int64_t ns_h, int64_t ns_key,
    int64_t ns_sub, uint16_t *__restrict__ weight, int64_t ws_b, int64_t ws_h, int64_t ws_key, int64_t ws_sub,
    int32_t *__restrict__ cluster_counts, int64_t cc_b, int64_t cc_h, int keys_per_wg) {
  const int row = blockIdx.y;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  const int tid = threadIdx.x;
  const int s = tid & 15;   // block (subspace) owned by this lane
  const int kq = tid >> 4;  // key slot inside the iteration

  __shared__ uint32_t s_hist[16 * 256];
  __shared__ uint2 s_mag[BF16 ? (1 << kMagTableBits) : 1];
  __shared__ float s_centers[8];  // magnitude centres, looked up by code (an LDS read instead of a load from constant memory)
  __shared__ uint32_t s_spread[BF16 ? 256 : 1];
  if (tid < 8) s_centers[tid] = c_centers[tid];
  if (BF16) {
    uint32_t sp = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) sp |= ((uint32_t)(tid >> j) & 1u) << (4 * j + 3);
    s_spread[tid] = sp;  // kEncThreads == 256: one entry per thread
  }
  if (BF16) {
    for (int i = tid; i < (1 << kMagTableBits); i += kEncThreads) {
      const float v = __uint_as_float(kMagTableLo + ((uint32_t)i << 16));
      int t = 0;
#pragma unroll
      for (int k = 0; k < 7; ++k) t += (c_thresholds[k] < v) ? 1 : 0;
      s_mag[i] = make_uint2((uint32_t)t, __float_as_uint(c_centers[t]));
    }
  }
  if (cluster_counts)
    for (int i = tid; i < 16 * 256; i += kEncThreads) s_hist[i] = 0;
  __syncthreads();

  float sg[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) sg[j] = signs[8 * s + j];
  uint32_t sgw[4];  // the signs' sign bits, packed like a loaded word of two bf16
#pragma unroll
  for (int p = 0; p < 4; ++p)
    sgw[p] = ((__float_as_uint(sg[2 * p]) >> 16) & 0x8000u) | (__float_as_uint(sg[2 * p + 1]) & 0x80000000u);
  const uint32_t sm1 = (s & 1) ? 0x80000000u : 0u, sm2 = (s & 2) ? 0x80000000u : 0u, sm8 = (s & 8) ? 0x80000000u : 0u;
  const bool rerank = nib || weight;

  // every pointer advances by one iteration's 16 keys; lanes past the end of a ragged last block reload its last
  // key (all lanes take part in the shuffles) and store nothing
  const int64_t key_begin = (int64_t)blockIdx.x * keys_per_wg;  // < n_keys by the grid's construction
  const int last = (int)((n_keys - key_begin < keys_per_wg) ? n_keys - key_begin : keys_per_wg) - 1;
  constexpr int esize = BF16 ? 2 : 4;
  const char *krow = (const char *)keys + ((int64_t)b * k_stride_b + (int64_t)h * k_stride_h + key_begin * k_stride_key + 8 * s) * esize;
  const char *kp = krow + (int64_t)kq * k_stride_key * esize;
  const char *kp_last = krow + (int64_t)last * k_stride_key * esize;
  uint8_t *cp = codes + (int64_t)b * cs_b + (int64_t)h * cs_h + (key_begin + kq) * cs_key + (int64_t)s * cs_sub;
  uint8_t *np = nib ? nib + (int64_t)b * ns_b + (int64_t)h * ns_h + (key_begin + kq) * ns_key + (int64_t)s * ns_sub : nullptr;
  uint16_t *wp = weight ? weight + (int64_t)b * ws_b + (int64_t)h * ws_h + (key_begin + kq) * ws_key + (int64_t)s * ws_sub : nullptr;
  const int64_t k_step = (int64_t)kEncKeysPerIter * k_stride_key * esize, c_step = (int64_t)kEncKeysPerIter * cs_key,
                n_step = (int64_t)kEncKeysPerIter * ns_key, w_step = (int64_t)kEncKeysPerIter * ws_key;
  pkv_u32x4 raw[BF16 ? 1 : 2];  // the next iteration's key, loaded one iteration ahead
  {
    const char *src = kq <= last ? kp : kp_last;
    raw[0] = *(const pkv_u32x4 *)src;
    if (!BF16) raw[BF16 ? 0 : 1] = *(const pkv_u32x4 *)(src + 16);
  }
  for (int rel = kq; rel - kq <= last; rel += kEncKeysPerIter, cp += c_step, np += n_step, wp += w_step) {
    const bool active = rel <= last;
    pkv_u32x4 cur[BF16 ? 1 : 2];
    cur[0] = raw[0];
    if (!BF16) cur[BF16 ? 0 : 1] = raw[BF16 ? 0 : 1];
    kp += k_step;
    if (rel - kq + kEncKeysPerIter <= last) {  // uniform: another iteration follows
      const char *src = rel + kEncKeysPerIter <= last ? kp : kp_last;
      raw[0] = *(const pkv_u32x4 *)src;
      if (!BF16) raw[BF16 ? 0 : 1] = *(const pkv_u32x4 *)(src + 16);
    }
    EncOut o;
    bool exact = true;
    float x[8];
    if (BF16) {
      const uint32_t w[4] = {cur[0].x, cur[0].y, cur[0].z, cur[0].w};
      exact = __builtin_amdgcn_ballot_w64(enc_key_fast(w, sgw, sm1, sm2, sm8, rerank, s_mag, s_spread, o)) != 0;
      if (exact) {
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          x[2 * p] = __uint_as_float(w[p] << 16);
          x[2 * p + 1] = __uint_as_float(w[p] & 0xffff0000u);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[j] = __uint_as_float(cur[0][j]);
        x[4 + j] = __uint_as_float(cur[BF16 ? 0 : 1][j]);
      }
    }
    if (exact) {  // the whole wave: every lane takes part in the shuffles
      if (BF16) {  // rare: the signs are fetched again instead of being held in registers across the loop
#pragma unroll
        for (int j = 0; j < 8; ++j) sg[j] = signs[8 * s + j];
      }
      enc_key_exact<BF16>(x, sg, s, rerank, s_centers, o);
    }

    if (active) {
      *cp = (uint8_t)o.code;
      if (cluster_counts) atomicAdd(&s_hist[s * 256 + o.code], 1u);
      if (nib) *(uint32_t *)np = o.packed;
      if (weight) *wp = (uint16_t)o.wbits;
    }
  }
  if (cluster_counts) {
    __syncthreads();
    pkv_flush_cluster_hist(s_hist, cluster_counts + (int64_t)b * cc_b + (int64_t)h * cc_h, tid, kEncThreads);
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
  pkv_flush_cluster_hist(s_hist, cluster_counts + (int64_t)b * cc_b + (int64_t)h * cc_h, threadIdx.x, 256);
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
  // 256 keys per workgroup: measured against 64 .. 1024 and against one resident set of larger workgroups, this
  // balances the per-workgroup set-up (tables, histogram flush) against the partial last round of workgroups.
  const int64_t rows = (int64_t)bs * n_kv_heads;
  const int64_t per_wg = kEncKeysPerWg;
  dim3 grid((unsigned)((n_keys + per_wg - 1) / per_wg), (unsigned)rows);
#define PKV_ENC(BF)                                                                                                  \
  hipLaunchKernelGGL(pkv_encode_kernel<BF>, grid, dim3(kEncThreads), 0, (hipStream_t)stream, keys, n_kv_heads, n_keys, \
                     k_stride_b, k_stride_h, k_stride_key, signs, codes, cs_b, cs_h, cs_key, cs_sub, nib, ns_b, ns_h,  \
                     ns_key, ns_sub, weight, ws_b, ws_h, ws_key, ws_sub, cluster_counts, cc_b, cc_h, (int)per_wg)
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
