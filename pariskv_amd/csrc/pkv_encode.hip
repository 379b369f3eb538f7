// Encode-on-append: normalise, SRHT rotate, sign code per 8-dim block, 3-bit
// magnitude code per dim, per-block rerank weight, cluster-size histogram.
//
// Reference: cache_hub/polar_cache.py:924-978 (batch_encode: ~15 torch launches,
// three permute copies and [.,S,16,8] intermediates) and :980-996
// (_count_cluster_keys: bincount per batch element).
//
// One key is handled by 16 lanes, each owning the 8 dims of one block, so four
// keys share a wave64.  The 128-point Walsh-Hadamard transform is three in-lane
// butterfly stages plus four cross-lane stages (block xor 1,2,4,8); everything
// after the rotation is lane-local.  256 B read + 112 B written per key.
//
// Block s (bits s3 s2 s1 s0) sits in lane s0*1 ^ s1*2 ^ s2*7 ^ s3*15 of its
// row of 16, so that the partner of every cross-lane stage is one
// data-parallel-primitive move away (quad_perm [1,0,3,2], [2,3,0,1],
// row_half_mirror, row_mirror) and the move folds into the arithmetic
// instruction that uses it.
//
// The order of every floating-point operation is fixed (and contraction into
// FMA is disabled at build time) because the integer outputs must be
// reproducible bit for bit:
//   sum of squares: sequential inside a block, then a pairwise tree over blocks.
//
// The kernel sits between vector-instruction issue and the memory system (about
// 3.5 TB/s of mixed traffic: 256 B read, 16 + 96 B written in pieces, 64 B of
// histogram atomics per key): forty more instructions per key cost 5 - 10 %, a
// quarter fewer gained 5 %; without the record stores it takes 90, without any
// store and without the histogram 70 us per 2^20 keys, with everything 120 - 126.
// enc_key_exact is the chain as written (correctly rounded divisions and roots,
// about 660 vector instructions per lane and key).  bf16 keys take enc_key_fast
// (about 225), which reaches the same bits through reciprocals, a table for the
// magnitude code and its term of the weight, and lane-crossing butterflies of
// one instruction per value; fp32 keys take enc_key_fast_f32 (about 345): the
// compiler's own division sequence with the reciprocal refinement shared by the
// eight quotients of a denominator and without its range scaling, the same
// butterflies, and a small banded table for the magnitude code.  Either hands a
// wave over to enc_key_exact when one of its keys is outside the range where
// that is proven.
#include "pkv_common.h"

namespace {

// 256 threads with four workgroups per CU (LDS: 16 KB histogram + 16 KB table each) and 512 threads with three measure
// the same; eight waves per SIMD need 64 registers and run a third slower.
constexpr int kEncThreads = 256;
constexpr int kEncWavesPerSimd = 4;
constexpr int kEncKeysPerIter = kEncThreads / 16;
constexpr int kEncKeysPerWg = 16 * kEncKeysPerIter;
// iterations whose keys a wave has in flight (bf16 keys, 1 / 2 / 4: 132 / 127 / 125 us per 1M key-heads); an fp32
// key takes two 16-byte words per lane, so half as many iterations hold the same bytes in as many registers
constexpr int kEncAheadBf16 = 4, kEncAheadF32 = 2;

#define PKV_ENC_THRESHOLDS 0.08447265625f, 0.169921875f, 0.2578125f, 0.349609375f, 0.44921875f, 0.55859375f, 0.69140625f
#define PKV_ENC_CENTERS 0.0419921875f, 0.126953125f, 0.212890625f, 0.302734375f, 0.396484375f, 0.5f, 0.6171875f, 0.76171875f
__constant__ float c_thresholds[7] = {PKV_ENC_THRESHOLDS};
__constant__ float c_centers[8] = {PKV_ENC_CENTERS};
constexpr float kEncThresholds[7] = {PKV_ENC_THRESHOLDS};
constexpr float kEncCenters[8] = {PKV_ENC_CENTERS};

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
// Block owned by lane l of a row of 16 (the inverse of l = s0*1 ^ s1*2 ^ s2*7 ^ s3*15).
__device__ __forceinline__ int enc_block_of_lane(int l) { return l ^ ((l & 4) ? 3 : 0) ^ ((l & 8) ? 4 : 0); }
constexpr int kEncLaneXor4 = 7, kEncLaneXor8 = 15;  // lane distance to the blocks s ^ 4 and s ^ 8

template <bool BF16>
__device__ __forceinline__ void enc_key_exact(const float (&x)[8], const float (&sg)[8], int s, bool rerank,
                                              const float *s_centers, EncOut &o) {
  constexpr int dtype = BF16 ? PKV_DTYPE_BF16 : PKV_DTYPE_F32;
  float y[8];
  const float n = pkv_normalize_rotate_16<kEncLaneXor4, kEncLaneXor8>(x, sg, s, dtype, y);
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

// What the bf16 chain does with one component u of a block's direction depends on the bf16 pattern of |u| alone:
// its magnitude code t (the number of thresholds below |u|) and its term of the weight's denominator,
// bf16(centre[t] * |u|).  Both come from one 8-byte table entry indexed by the low 11 bits of the pattern, which
// covers 2^-15 <= |u| < 2 (patterns 0x3800 .. 0x3FFF); |u| never reaches 2, and a wave that holds a smaller |u|
// recomputes those terms by the formula (code 0, centre[0]).  The table is a constant of the library's device image;
// a workgroup copies its 16 KB into LDS.
constexpr int kMagTableBits = 11;
constexpr int kMagEntries = 1 << kMagTableBits;
constexpr uint32_t kMagTableLo = 0x38000000u;  // 2^-15
constexpr float kMagTableLoF = 0x1p-15f;

constexpr uint32_t enc_cx_bf16_round_bits(float f) {  // round to nearest even; positive normal numbers
  uint32_t b = __builtin_bit_cast(uint32_t, f);
  b += 0x7fffu + ((b >> 16) & 1u);
  return b & 0xffff0000u;
}
// fp32 keys: |u| is not a pattern one can index by, but thresholds lie further apart than 0.08, so a band of that
// width holds at most one of them: entry k, for k = floor(12.5 |u|) (<= 12 as |u| <= 1 up to rounding; 16 entries, the
// index is masked), names the number of thresholds below the band, the one threshold inside it (or infinity) and the
// centres on either side of that threshold.  The code is the count plus one comparison.  The product 12.5 |u| is
// rounded, so a |u| next to a band's edge may land in the neighbouring band: every entry is valid for the band widened
// by kMagBandSlop on both sides (checked below: still at most one threshold).
constexpr int kMagBands = 16;
constexpr float kMagBandsPerUnit = 12.5f, kMagBandSlop = 1e-4f;
struct EncTables {
  uint32_t mag[2 * kMagEntries];  // {magnitude code, bf16(centre * |u|) as fp32 bits} for pattern kMagTableLo >> 16 + i
  uint32_t spread[256];           // bit j of the index moved to bit 4j + 3
  uint32_t band[4 * kMagBands];   // {thresholds below the band, threshold inside it, centre below it, centre above it}
  bool bands_ok;
  constexpr EncTables() : mag{}, spread{}, band{}, bands_ok(true) {
    for (int k = 0; k < kMagBands; ++k) {
      const float lo = (float)k / kMagBandsPerUnit - kMagBandSlop, hi = (float)(k + 1) / kMagBandsPerUnit + kMagBandSlop;
      int below = 0, inside = 0;
      float th = __builtin_huge_valf();
      for (int i = 0; i < 7; ++i) {
        if (kEncThresholds[i] <= lo) ++below;
        else if (kEncThresholds[i] < hi) ++inside, th = kEncThresholds[i];
      }
      if (inside > 1) bands_ok = false;
      band[4 * k] = (uint32_t)below;
      band[4 * k + 1] = __builtin_bit_cast(uint32_t, th);
      band[4 * k + 2] = __builtin_bit_cast(uint32_t, kEncCenters[below]);
      band[4 * k + 3] = __builtin_bit_cast(uint32_t, kEncCenters[below + (inside ? 1 : 0)]);
    }
    for (int i = 0; i < kMagEntries; ++i) {
      const float v = __builtin_bit_cast(float, kMagTableLo + ((uint32_t)i << 16));
      int t = 0;
      for (int k = 0; k < 7; ++k) t += (kEncThresholds[k] < v) ? 1 : 0;
      mag[2 * i] = (uint32_t)t;
      mag[2 * i + 1] = enc_cx_bf16_round_bits(kEncCenters[t] * v);
    }
    for (int c = 0; c < 256; ++c) {
      uint32_t sp = 0;
      for (int j = 0; j < 8; ++j) sp |= ((uint32_t)(c >> j) & 1u) << (4 * j + 3);
      spread[c] = sp;
    }
  }
};
__device__ __align__(16) const EncTables g_enc_tables = EncTables();
static_assert(EncTables().bands_ok, "a band of |u| holds two magnitude thresholds");

template <int CTRL>
__device__ __forceinline__ float enc_dpp(float v) {  // bound_ctrl set, so that the move folds into the add that uses it
  return __uint_as_float((uint32_t)__builtin_amdgcn_update_dpp(0, (int)__float_as_uint(v), CTRL, 0xf, 0xf, true));
}
// One Walsh-Hadamard stage across lanes in one instruction per value: held' = held(partner) * c + held with
// c = +1 in the lanes whose block index has the stage's bit clear and -1 in the others.  Where c = +1 that is the
// stage's own sum; where c = -1 it is own - partner, the NEGATIVE of the stage's partner - own (negation commutes
// with rounding to nearest).  A lane therefore carries its value times (-1)^(number of set bits among the stages
// done so far), the same factor in both lanes of every later pair, and the factor left after the four stages, the
// parity of the block index, is taken out by the sign of the lane's final scale.  (A difference that is exactly zero
// keeps +0 where the negated form would hold -0; zeros that reach the result send the key to enc_key_exact.)
// The compiler does not fold the move into a fused multiply-add, hence the assembly: the four stages of eight values.
// The leading wait covers the two states the hardware needs between a vector write and a lane-crossing read of the
// same register; inside the block a value is read eight instructions after it was written.
#define PKV_ENC_STAGE(CTL, C)                                   \
  "v_fmac_f32_dpp %0, %0, " C " " CTL " row_mask:0xf bank_mask:0xf\n\t" \
  "v_fmac_f32_dpp %1, %1, " C " " CTL " row_mask:0xf bank_mask:0xf\n\t" \
  "v_fmac_f32_dpp %2, %2, " C " " CTL " row_mask:0xf bank_mask:0xf\n\t" \
  "v_fmac_f32_dpp %3, %3, " C " " CTL " row_mask:0xf bank_mask:0xf\n\t" \
  "v_fmac_f32_dpp %4, %4, " C " " CTL " row_mask:0xf bank_mask:0xf\n\t" \
  "v_fmac_f32_dpp %5, %5, " C " " CTL " row_mask:0xf bank_mask:0xf\n\t" \
  "v_fmac_f32_dpp %6, %6, " C " " CTL " row_mask:0xf bank_mask:0xf\n\t" \
  "v_fmac_f32_dpp %7, %7, " C " " CTL " row_mask:0xf bank_mask:0xf\n\t"
__device__ __forceinline__ void enc_lane_stages(float (&t)[8], float c1, float c2, float c4, float c8) {
  asm("s_nop 1\n\t"
      PKV_ENC_STAGE("quad_perm:[1,0,3,2]", "%8")
      PKV_ENC_STAGE("quad_perm:[2,3,0,1]", "%9")
      PKV_ENC_STAGE("row_half_mirror", "%10")
      PKV_ENC_STAGE("row_mirror", "%11")
      : "+v"(t[0]), "+v"(t[1]), "+v"(t[2]), "+v"(t[3]), "+v"(t[4]), "+v"(t[5]), "+v"(t[6]), "+v"(t[7])
      : "v"(c1), "v"(c2), "v"(c4), "v"(c8));
}
#undef PKV_ENC_STAGE

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

// fp32 keys.  a / d as the compiler's own expansion of a correctly rounded division computes it (reciprocal, one
// Newton step on it, quotient, two residual corrections), without the operand scaling and the special-case fix-up
// around it: both are the identity while d and a are normal, 1 / d is normal and the quotient and its residuals
// stay clear of the denormals, which the callers' range checks see to.  The refined reciprocal depends on d alone
// and is shared by the eight quotients of one key and lane.
struct EncRcp {
  float neg_d, y;
};
__device__ __forceinline__ EncRcp enc_rcp_refined(float d) {
  EncRcp r;
  const float y0 = __builtin_amdgcn_rcpf(d);
  r.neg_d = -d;
  r.y = __builtin_fmaf(__builtin_fmaf(r.neg_d, y0, 1.0f), y0, y0);
  return r;
}
__device__ __forceinline__ float enc_div_shared(float a, const EncRcp &r) {
  float q = a * r.y;
  q = __builtin_fmaf(__builtin_fmaf(r.neg_d, q, a), r.y, q);
  return __builtin_fmaf(__builtin_fmaf(r.neg_d, q, a), r.y, q);
}
// sqrt(a), correctly rounded, for 2^-90 <= a <= 2^120: the hardware root (1 ulp) moved to a neighbour where the
// residuals say so, again the compiler's expansion without its scaling of tiny arguments and its special cases.
__device__ __forceinline__ float enc_sqrt_rn(float a) {
  const float s = __builtin_amdgcn_sqrtf(a);
  const float dn = __uint_as_float(__float_as_uint(s) - 1u), up = __uint_as_float(__float_as_uint(s) + 1u);
  const float r_dn = __builtin_fmaf(-dn, s, a), r_up = __builtin_fmaf(-up, s, a);
  float r = (0.0f >= r_dn) ? dn : s;
  r = (0.0f < r_up) ? up : r;
  return r;
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
// unspecified.  c1/c2/c4/c8 = -1 where the lane's block index has bit 0/1/2/3 set, else +1; scale = 1/sqrt(128)
// with the sign (-1)^(set bits of the block index).  s_mag / s_spread = the workgroup's copy of g_enc_tables.
__device__ __forceinline__ bool enc_key_fast(const uint32_t (&w)[4], const uint32_t (&sgw)[4], float c1, float c2,
                                             float c4, float c8, float scale, bool rerank, const uint2 *s_mag,
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
  acc = enc_dpp<0xB1>(acc) + acc;   // block ^ 1: lane ^ 1
  acc = enc_dpp<0x4E>(acc) + acc;   // block ^ 2: lane ^ 2
  acc = enc_dpp<0x141>(acc) + acc;  // block ^ 4: lane ^ 7 (row_half_mirror)
  acc = enc_dpp<0x140>(acc) + acc;  // block ^ 8: lane ^ 15 (row_mirror)
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
  enc_lane_stages(t, c1, c2, c4, c8);
  float y[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = pkv_bf16_round(t[j] * scale);
  // y >= 0 is read off the sign bit, which is wrong for a zero: a key with |y| < 2^-40 somewhere, zero included, goes
  // to enc_key_exact.  With the rerank outputs that test is made further down, and only in waves that need it.
  uint32_t sneg = 0;
#pragma unroll
  for (int j = 7; j >= 0; --j) sneg = __builtin_amdgcn_alignbit(sneg, __float_as_uint(y[j]), 31);
  o.code = ~sneg & 0xffu;
  if (!rerank) return bad | (enc_min_abs8(y) < 0x1p-40f);

  // y: bf16 values.  Their squares are exact again unless a |y| is below 2^-40, and such a y has |u| = |y| / r below
  // 2^-15 (r <= 2^-24 is sent to enc_key_exact as well), which the test on |u| below catches.
  float r2 = y[0] * y[0];
#pragma unroll
  for (int j = 1; j < 8; ++j) r2 = __builtin_fmaf(y[j], y[j], r2);
  const float r = enc_sqrt_bf16(r2);
  bad |= !(r >= 0x1p-24f) || r > 0x1p60f;
  const float r_inv = __builtin_amdgcn_rcpf(r);
  float u[8];
  uint2 e[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    u[j] = pkv_bf16_round(y[j] * r_inv);
    const uint32_t byte_off = __builtin_amdgcn_ubfe(__float_as_uint(u[j]), 13, kMagTableBits + 3);  // 8 * (pattern & 0x7ff)
    e[j] = *(const uint2 *)((const char *)s_mag + byte_off);
  }
  if (__builtin_amdgcn_ballot_w64(enc_min_abs8(u) < kMagTableLoF) != 0) {  // about one wave in thirty
    bad |= enc_min_abs8(y) < 0x1p-40f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float au = fabsf(u[j]);
      if (au < kMagTableLoF) e[j] = make_uint2(0u, __float_as_uint(pkv_bf16_round(kEncCenters[0] * au)));
    }
  }
  uint32_t mags = 0;
  float alpha = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    mags = __builtin_amdgcn_alignbit(e[j].x, mags, 4);  // the code enters at the top nibble; after 8 steps code j sits in nibble j
    const float p = __uint_as_float(e[j].y);
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

// The fp32 chain of enc_key_exact in fewer instructions, same bits: the sixteen quotients of a key and lane share
// two refined reciprocals (enc_div_shared), the roots skip the compiler's range scaling (enc_sqrt_rn), the
// lane-crossing butterflies take one instruction per value (enc_lane_stages), signs are read off the sign bit and
// the weight's division is done only near a bf16 rounding boundary.  Sums, products and comparisons are the exact
// path's own.  xr[] = the lane's eight components as loaded, sg[] = the SRHT signs of its block.  Returns true when
// this lane's key needs enc_key_exact (norm or radius outside [1e-8, 2^60], or a component of the key or of its
// rotation below 2^-40 in magnitude, zero included); o is then unspecified.  A zero whose sign differs from the
// exact path's (the butterflies' negated differences) can only end as a zero of the rotation, which that test sees.
__device__ __forceinline__ bool enc_key_fast_f32(const float (&xr)[8], const float (&sg)[8], float c1, float c2,
                                                 float c4, float c8, float scale, bool rerank,
                                                 const pkv_u32x4 *s_band, const uint32_t *s_spread, EncOut &o) {
  float x[8];  // components times their SRHT sign (+-1): the sign commutes with the division and its rounding
#pragma unroll
  for (int j = 0; j < 8; ++j) x[j] = xr[j] * sg[j];
  float acc = x[0] * x[0];
#pragma unroll
  for (int j = 1; j < 8; ++j) acc = acc + x[j] * x[j];
  acc = enc_dpp<0xB1>(acc) + acc;   // block ^ 1: lane ^ 1
  acc = enc_dpp<0x4E>(acc) + acc;   // block ^ 2: lane ^ 2
  acc = enc_dpp<0x141>(acc) + acc;  // block ^ 4: lane ^ 7 (row_half_mirror)
  acc = enc_dpp<0x140>(acc) + acc;  // block ^ 8: lane ^ 15 (row_mirror)
  const float n = enc_sqrt_rn(acc);  // acc outside the root's range gives an n outside the range tested next
  bool bad = !(n >= 1e-8f) || n > 0x1p60f;
  bad |= enc_min_abs8(x) < 0x1p-40f;
  const EncRcp n_rcp = enc_rcp_refined(n);
  float t[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) t[j] = enc_div_shared(x[j], n_rcp);
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
  enc_lane_stages(t, c1, c2, c4, c8);
  float y[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) y[j] = t[j] * scale;
  uint32_t sneg = 0;
#pragma unroll
  for (int j = 7; j >= 0; --j) sneg = __builtin_amdgcn_alignbit(sneg, __float_as_uint(y[j]), 31);
  o.code = ~sneg & 0xffu;
  bad |= enc_min_abs8(y) < 0x1p-40f;
  if (!rerank) return bad;

  float r2 = y[0] * y[0];
#pragma unroll
  for (int j = 1; j < 8; ++j) r2 = r2 + y[j] * y[j];
  const float r = enc_sqrt_rn(r2);
  bad |= !(r >= 1e-8f) || r > 0x1p60f;
  const EncRcp r_rcp = enc_rcp_refined(r);
  uint32_t mags = 0;
  float alpha = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float au = fabsf(enc_div_shared(y[j], r_rcp));
    // 16 bytes per band: floor(200 |u|) without its low four bits = 16 floor(12.5 |u|); the mask also bounds the index
    const uint32_t band_off = (uint32_t)(au * (16.0f * kMagBandsPerUnit)) & (16u * (kMagBands - 1));
    const pkv_u32x4 e = *(const pkv_u32x4 *)((const char *)s_band + band_off);
    const bool above = __uint_as_float(e.y) < au;
    const uint32_t tc = e.x + (above ? 1u : 0u);
    mags = __builtin_amdgcn_alignbit(tc, mags, 4);  // the code enters at the top nibble; after 8 steps code j sits in nibble j
    const float p = __uint_as_float(above ? e.w : e.z) * au;
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

// ALL: codes, 4-bit records, weights and cluster sizes are all written (the caller's pointers are all set), so the
// loop body has no branch around a store.  Loads and stores retire through one in-order counter; with a store that
// may or may not have been issued after the load of the next key, the only safe wait for that key is "everything
// outstanding", stores included.  Without the branches the wait names the exact count and the stores stay in flight.
template <bool BF16, bool ALL>
__global__ __launch_bounds__(kEncThreads) __attribute__((amdgpu_waves_per_eu(kEncWavesPerSimd, kEncWavesPerSimd))) void pkv_encode_kernel(
    const void *__restrict__ keys, int n_kv_heads, int64_t n_keys, int64_t k_stride_b, int64_t k_stride_h,
    int64_t k_stride_key, const float *__restrict__ signs, uint8_t *__restrict__ codes, int64_t cs_b, int64_t cs_h,
    int64_t cs_key, int64_t cs_sub, uint8_t *__restrict__ nib, int64_t ns_b, int64_t ns_h, int64_t ns_key,
    int64_t ns_sub, uint16_t *__restrict__ weight, int64_t ws_b, int64_t ws_h, int64_t ws_key, int64_t ws_sub,
    int32_t *__restrict__ cluster_counts, int64_t cc_b, int64_t cc_h, int keys_per_wg) {
  const bool has_nib = ALL || nib, has_weight = ALL || weight, has_hist = ALL || cluster_counts;
  const int row = blockIdx.y;
  const int b = row / n_kv_heads, h = row % n_kv_heads;
  const int tid = threadIdx.x;
  const int s = enc_block_of_lane(tid & 15);  // block (subspace) owned by this lane
  const int kq = tid >> 4;  // key slot inside the iteration

  __shared__ uint32_t s_hist[16 * 256];
  __shared__ __align__(16) uint2 s_mag[BF16 ? kMagEntries : 2];
  __shared__ float s_centers[8];  // magnitude centres, looked up by code (an LDS read instead of a load from constant memory)
  __shared__ uint32_t s_spread[256];
  __shared__ __align__(16) pkv_u32x4 s_band[BF16 ? 1 : kMagBands];
  if (tid < 8) s_centers[tid] = c_centers[tid];
  if (!BF16 && tid < kMagBands) s_band[tid] = ((const pkv_u32x4 *)g_enc_tables.band)[tid];
  if (tid < 256) s_spread[tid] = g_enc_tables.spread[tid];
  if (BF16) {
    const pkv_u32x4 *src = (const pkv_u32x4 *)g_enc_tables.mag;
#pragma unroll
    for (int i = 0; i < kMagEntries / 2 / kEncThreads; ++i)
      ((pkv_u32x4 *)s_mag)[tid + i * kEncThreads] = src[tid + i * kEncThreads];
  }
  if (has_hist)
    for (int i = tid; i < 16 * 256; i += kEncThreads) s_hist[i] = 0;
  __syncthreads();

  float sg[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) sg[j] = signs[8 * s + j];
  uint32_t sgw[4];  // the signs' sign bits, packed like a loaded word of two bf16
#pragma unroll
  for (int p = 0; p < 4; ++p)
    sgw[p] = ((__float_as_uint(sg[2 * p]) >> 16) & 0x8000u) | (__float_as_uint(sg[2 * p + 1]) & 0x80000000u);
  const float c1 = (s & 1) ? -1.f : 1.f, c2 = (s & 2) ? -1.f : 1.f, c4 = (s & 4) ? -1.f : 1.f, c8 = (s & 8) ? -1.f : 1.f;
  const float scale = (__builtin_popcount((unsigned)s) & 1) ? -PKV_HADAMARD_SCALE : PKV_HADAMARD_SCALE;
  const bool rerank = ALL || nib || weight;

  // Addresses are a wave-uniform base, which advances by one iteration's 16 keys through scalar adds, plus a
  // 32-bit lane offset that never changes (the launcher checks that the offsets fit).  Lanes past the end of a
  // ragged last block load its last key (all lanes take part in the lane-crossing steps); they store nothing, or,
  // in the ALL form, that key's results once more.
  const int64_t key_begin = (int64_t)blockIdx.x * keys_per_wg;  // < n_keys by the grid's construction
  const int last = (int)((n_keys - key_begin < keys_per_wg) ? n_keys - key_begin : keys_per_wg) - 1;
  constexpr int esize = BF16 ? 2 : 4;
  const char *k_base = (const char *)keys + ((int64_t)b * k_stride_b + (int64_t)h * k_stride_h + key_begin * k_stride_key) * esize;
  uint8_t *c_base = codes + (int64_t)b * cs_b + (int64_t)h * cs_h + key_begin * cs_key;
  uint8_t *n_base = has_nib ? nib + (int64_t)b * ns_b + (int64_t)h * ns_h + key_begin * ns_key : nullptr;
  char *w_base = has_weight ? (char *)(weight + (int64_t)b * ws_b + (int64_t)h * ws_h + key_begin * ws_key) : nullptr;
  const uint32_t key_bytes = (uint32_t)(k_stride_key * esize), blk_off = (uint32_t)(8 * s * esize);
  const uint32_t k_lane = (uint32_t)kq * key_bytes + blk_off;
  const uint32_t c_lane = (uint32_t)(kq * cs_key + s * cs_sub), n_lane = (uint32_t)(kq * ns_key + s * ns_sub),
                 w_lane = (uint32_t)(2 * (kq * ws_key + s * ws_sub));
  const int64_t k_step = (int64_t)kEncKeysPerIter * k_stride_key * esize, c_step = (int64_t)kEncKeysPerIter * cs_key,
                n_step = (int64_t)kEncKeysPerIter * ns_key, w_step = (int64_t)kEncKeysPerIter * ws_key * 2;
  // A wave keeps the keys of its next kEncAhead iterations in flight, each in a register set of its own: set j holds
  // iterations j, j + kEncAhead, ... and is refilled as soon as its key has been copied out.  (A ring whose sets are
  // copied into each other waits for the newest load at every copy and hides one iteration of latency whatever its
  // depth.)  Loads are never skipped - past the block's end they fetch its last iteration again - because a load that
  // may or may not have been issued makes every later wait of the in-order counter a wait for everything.
  constexpr int kW = BF16 ? 1 : 2;  // 16-byte words per lane and key
  constexpr int kEncAhead = BF16 ? kEncAheadBf16 : kEncAheadF32;
  const int n_iter = last / kEncKeysPerIter + 1;
  pkv_u32x4 raw[kEncAhead][kW];
  auto load_iter = [&](int it, pkv_u32x4 (&reg)[kW]) {
    const int it_c = it < n_iter ? it : n_iter - 1;  // uniform
    const char *base = k_base + (int64_t)it_c * k_step;
    const int lim = last - it_c * kEncKeysPerIter;  // the iteration holds the block's keys 16 it_c .. 16 it_c + lim
    uint32_t off = k_lane;
    if (lim < kEncKeysPerIter - 1) off = kq <= lim ? k_lane : (uint32_t)lim * key_bytes + blk_off;  // uniform: it is ragged
    reg[0] = *(const pkv_u32x4 *)(base + off);
    if (!BF16) reg[kW - 1] = *(const pkv_u32x4 *)(base + off + 16);
  };
  auto iteration = [&](int it, pkv_u32x4 (&reg)[kW]) {
    const int first = it * kEncKeysPerIter;
    const bool active = kq <= last - first;
    pkv_u32x4 cur[kW];
#pragma unroll
    for (int q = 0; q < kW; ++q) cur[q] = reg[q];
    load_iter(it + kEncAhead, reg);
    EncOut o;
    bool exact = true;
    float x[8];
    if (BF16) {
      const uint32_t w[4] = {cur[0].x, cur[0].y, cur[0].z, cur[0].w};
      exact = __builtin_amdgcn_ballot_w64(enc_key_fast(w, sgw, c1, c2, c4, c8, scale, rerank, s_mag, s_spread, o)) != 0;
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
        x[4 + j] = __uint_as_float(cur[kW - 1][j]);
      }
      exact = __builtin_amdgcn_ballot_w64(enc_key_fast_f32(x, sg, c1, c2, c4, c8, scale, rerank, s_band, s_spread, o)) != 0;
    }
    if (exact) {  // the whole wave: every lane takes part in the shuffles
      if (BF16) {  // rare: the signs are fetched again instead of being held in registers across the loop
#pragma unroll
        for (int j = 0; j < 8; ++j) sg[j] = signs[8 * s + j];
      }
      enc_key_exact<BF16>(x, sg, s, rerank, s_centers, o);
    }

    // the empty statement keeps the lane offsets apart from the bases, so that the stores address
    // scalar base + lane offset instead of three 64-bit lane pointers that would each need an add per iteration
    uint8_t *cb = c_base + (int64_t)it * c_step, *nb = n_base + (int64_t)it * n_step;
    char *wb = w_base + (int64_t)it * w_step;
    uint32_t c_off = c_lane, n_off = n_lane, w_off = w_lane;
    if (ALL) {
      // No branch around the stores (see above): a lane past the end of a ragged block holds the block's last key
      // and writes that key's results once more, to the same place.
      if (last - first < kEncKeysPerIter - 1) {  // uniform
        const uint32_t kk = (uint32_t)(kq < last - first ? kq : last - first);
        c_off = kk * (uint32_t)cs_key + (uint32_t)(s * cs_sub);
        n_off = kk * (uint32_t)ns_key + (uint32_t)(s * ns_sub);
        w_off = 2 * (kk * (uint32_t)ws_key + (uint32_t)(s * ws_sub));
      }
      asm volatile("" : "+v"(c_off), "+v"(n_off), "+v"(w_off));
      // written once and not read again by this launch: streaming stores (5 - 8 % on two of three shapes)
      __builtin_nontemporal_store((uint8_t)o.code, cb + c_off);
      __builtin_nontemporal_store(o.packed, (uint32_t *)(nb + n_off));
      __builtin_nontemporal_store((uint16_t)o.wbits, (uint16_t *)(wb + w_off));
      if (active) atomicAdd(&s_hist[s * 256 + o.code], 1u);
    } else if (active) {
      asm volatile("" : "+v"(c_off), "+v"(n_off), "+v"(w_off));
      cb[c_off] = (uint8_t)o.code;
      if (has_hist) atomicAdd(&s_hist[s * 256 + o.code], 1u);
      if (has_nib) *(uint32_t *)(nb + n_off) = o.packed;
      if (has_weight) *(uint16_t *)(wb + w_off) = (uint16_t)o.wbits;
    }
  };
#pragma unroll
  for (int j = 0; j < kEncAhead; ++j) load_iter(j, raw[j]);
  int it = 0;
  for (; it + kEncAhead <= n_iter; it += kEncAhead) {  // whole groups: no branch between the sets' loads and stores
#pragma unroll
    for (int j = 0; j < kEncAhead; ++j) iteration(it + j, raw[j]);
  }
#pragma unroll
  for (int j = 0; j < kEncAhead - 1; ++j)  // what a ragged block leaves: fewer than kEncAhead iterations
    if (it + j < n_iter) iteration(it + j, raw[j]);
  if (has_hist) {
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
  // a lane's byte offsets inside one iteration's keys and 16 blocks are kept in 32 bits
  const int64_t lim = (int64_t)1 << 31;
  PKV_REQUIRE(k_stride_key >= 0 && cs_key >= 0 && cs_sub >= 0 && ns_key >= 0 && ns_sub >= 0 && ws_key >= 0 && ws_sub >= 0,
              "pkv_encode_append: negative key or block strides are not supported");
  PKV_REQUIRE(kEncKeysPerIter * k_stride_key * 4 + 512 < lim && kEncKeysPerIter * cs_key + 16 * cs_sub < lim &&
                  kEncKeysPerIter * ns_key + 16 * ns_sub < lim && 2 * (kEncKeysPerIter * ws_key + 16 * ws_sub) < lim,
              "pkv_encode_append: key or block strides too large (a lane's offsets inside one iteration's keys must stay below 2 GiB)");
  // 256 keys per workgroup: measured against 128 .. 4096, this balances the per-workgroup set-up (tables,
  // histogram flush) against the partial last round of workgroups.
  const int64_t rows = (int64_t)bs * n_kv_heads;
  const int64_t per_wg = kEncKeysPerWg;
  dim3 grid((unsigned)((n_keys + per_wg - 1) / per_wg), (unsigned)rows);
#define PKV_ENC(BF, ALL)                                                                                               \
  hipLaunchKernelGGL((pkv_encode_kernel<BF, ALL>), grid, dim3(kEncThreads), 0, (hipStream_t)stream, keys, n_kv_heads,  \
                     n_keys, k_stride_b, k_stride_h, k_stride_key, signs, codes, cs_b, cs_h, cs_key, cs_sub, nib, ns_b, \
                     ns_h, ns_key, ns_sub, weight, ws_b, ws_h, ws_key, ws_sub, cluster_counts, cc_b, cc_h, (int)per_wg)
  const bool all = nib && weight && cluster_counts;
  if (dtype == PKV_DTYPE_BF16) {
    if (all) PKV_ENC(true, true); else PKV_ENC(true, false);
  } else {
    if (all) PKV_ENC(false, true); else PKV_ENC(false, false);
  }
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
