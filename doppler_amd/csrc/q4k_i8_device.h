// Device pieces shared by the int8 matrix-core Q4_K GEMV kernels (q4k_gemv_i8.hip: one product per
// launch; q4k_gemv_chain.hip: several dependent products per launch): the activation quantiser, the
// layout of its records in LDS, and the arithmetic that turns a work unit's integer digit sums into
// a partial dot product.
//
// Activation format.  A super-block column (256 activations) is quantised per 32-element sub-block:
// X = round(x * 2^E) with E chosen from the sub-block's largest magnitude so that |X| < 2^20, split
// into three 7-bit digits X = x0 * 2^14 + x1 * 2^7 + x2: the top one signed (-64..63), the lower two
// the plain bit fields 0..127 (three instructions per element, against five for balanced digits;
// all are valid int8 operands and the digit sums stay far inside 24 bits).  Every finite f32 activation keeps
// 20 bits below its sub-block's maximum (magnitudes below 2^-127 round to zero, as on flush-to-zero
// hardware).  A sub-block that holds a NaN gets the factor NaN; one that holds an infinity (and no
// NaN) gets the factor +Inf and the digits +-1 at the infinite elements, 0 elsewhere, so that the
// product comes out as (sum of +-w over the infinite elements) * Inf: the sign the exact sum has,
// and NaN where that sum is zero.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

// Bytes of one record (one super-block column of one activation row) and the offsets inside it.
constexpr int kRec = 848;
constexpr int kRecPlane = 256;     // digit plane p at 256 p: byte e = digit p of element e
constexpr int kRecSums = 768;      // 8 floats: sum of the quantised activations of each sub-block (not yet scaled)
constexpr int kRecXinv = 800;      // 8 floats: 2^-E of each sub-block
constexpr int kRecSsq = 832;       // float: the column's sum of squares (RMSNorm prologue)

// Sum over aligned groups of 8 lanes, left in all of them.
__device__ __forceinline__ int sum8_i32(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0xB1, 0xF, 0xF, false);    // quad_perm [1,0,3,2]
  v += __builtin_amdgcn_update_dpp(0, v, 0x4E, 0xF, 0xF, false);    // quad_perm [2,3,0,1]
  v += __builtin_amdgcn_update_dpp(0, v, 0x141, 0xF, 0xF, false);   // row_half_mirror
  return v;
}

// Largest value over aligned groups of 8 lanes, left in all of them.
__device__ __forceinline__ uint32_t max8_u32(uint32_t v) {
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, false));
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, false));
  v = max(v, (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, false));
  return v;
}

// Sum over the four lanes l, l ^ 16, l ^ 32, l ^ 48, left in all of them.
__device__ __forceinline__ float sum_lane_groups(float v) {
  const uint32_t u = __float_as_uint(v);
  auto a = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const uint32_t w = __float_as_uint(v);
  auto b = __builtin_amdgcn_permlane16_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// Lane t of a wave holds elements 4t .. 4t+3 of a column (sub-block t / 8): quantises them and
// writes the lane's share of the record at `rec` (digit planes, and from the first lane of every
// sub-block its sum and factor).  The values are taken as they come: masking past K and the
// RMSNorm weight are the caller's business.
__device__ __forceinline__ void i8_quantise_store(const float (&v)[4], unsigned char* rec, const int lane) {
  uint32_t ab[4];
#pragma unroll
  for (int e = 0; e < 4; e++) ab[e] = __float_as_uint(v[e]) & 0x7FFFFFFFu;
  // as unsigned integers magnitudes order like the floats, infinities above every finite value, NaNs above those
  const uint32_t mb = max8_u32(max(max(ab[0], ab[1]), max(ab[2], ab[3])));
  const int ef = (int)(mb >> 23);
  const bool special = ef == 255;
  const int ex = max(ef - 127, -107);                      // the sub-block's largest magnitude is below 2^(ex+1)
  float sf = __uint_as_float((uint32_t)(127 + 19 - ex) << 23);       // |x| * sf < 2^20
  float xinv = __uint_as_float((uint32_t)(127 - 19 + ex) << 23);
  float q[4] = {v[0], v[1], v[2], v[3]};
  // non-finite values are rare: their handling stays off the common path (one wave-uniform branch)
  if (__builtin_amdgcn_ballot_w64(special) != 0ull) {
    if (special) {
      const bool has_nan = mb > 0x7F800000u;
      sf = 1.0f;
      xinv = __uint_as_float(has_nan ? 0x7FC00000u : 0x7F800000u);
#pragma unroll
      for (int e = 0; e < 4; e++) q[e] = (ab[e] == 0x7F800000u && !has_nan) ? copysignf(1.0f, v[e]) : 0.0f;
    }
  }
  // X = round(x * sf) sits in the low mantissa bits of x * sf + 1.5 * 2^23 (two's complement)
  // (the bit pattern is 0x4B400000 + X: bits 0..6, 7..13 and 14..21 are the digits, the last one as a
  // two's-complement byte)
  uint32_t b[4], d1[4], d0[4];
  uint32_t xs = 0u;
#pragma unroll
  for (int e = 0; e < 4; e++) {
    b[e] = __float_as_uint(fmaf(q[e], sf, 12582912.0f));
    xs += b[e];
    d1[e] = b[e] >> 7;                                                     // byte 0: middle digit and one bit of the top one
    d0[e] = b[e] >> 14;                                                    // byte 0 = top digit
  }
  const uint32_t lo01 = 0x0c0c0400u, hi23 = 0x04000c0cu;   // byte 0 of (src1, src0) -> bytes 0,1 / 2,3
  const uint32_t pk0 = __builtin_amdgcn_perm(d0[1], d0[0], lo01) | __builtin_amdgcn_perm(d0[3], d0[2], hi23);
  const uint32_t pk1 = (__builtin_amdgcn_perm(d1[1], d1[0], lo01) | __builtin_amdgcn_perm(d1[3], d1[2], hi23)) & 0x7F7F7F7Fu;
  const uint32_t pk2 = (__builtin_amdgcn_perm(b[1], b[0], lo01) | __builtin_amdgcn_perm(b[3], b[2], hi23)) & 0x7F7F7F7Fu;
  // sum of the quantised activations of the sub-block (8 lanes x 4 elements, |sum| < 2^25)
  const float sxf = (float)sum8_i32((int)(xs - 4u * 0x4B400000u));
  reinterpret_cast<uint32_t*>(rec)[lane] = pk0;
  reinterpret_cast<uint32_t*>(rec)[64 + lane] = pk1;
  reinterpret_cast<uint32_t*>(rec)[128 + lane] = pk2;
  if ((lane & 7) == 0) {
    reinterpret_cast<float*>(rec)[kRecSums / 4 + (lane >> 3)] = sxf;
    reinterpret_cast<float*>(rec)[kRecXinv / 4 + (lane >> 3)] = xinv;
  }
}

// What lane (weight row j, group kg) of a unit contributes: sub-blocks kg (digit sums da, scale
// sc_a, min mn_a, activation sum and factor sx[0] / xinv[0]) and 4 + kg (db, sc_b, mn_b, sx[1] /
// xinv[1]) of its row's super-block.  The three digit sums are put together as integers first:
// da[0] * 2^14 + da[1] * 2^7 + da[2] IS sum_k q_k X_k, exactly (at most 32 * 15 * 2^20 in magnitude), so
// the dot product of a sub-block meets one rounding when it becomes a float and one when it is scaled.
// Each sub-block is finished in f32 before its factor is applied, which keeps a non-finite factor
// from meeting the other sub-block's terms.
typedef int i8dev_v4i __attribute__((ext_vector_type(4)));
typedef float i8dev_v2f __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float i8_unit_term(const i8dev_v4i da, const i8dev_v4i db, const int sc_a, const int sc_b,
                                              const float mn_a, const float mn_b, const float d, const float dmin,
                                              const i8dev_v2f sx, const i8dev_v2f xinv) {
  const float ta = (float)((((da[0] << 7) + da[1]) << 7) + da[2]);
  const float tb = (float)((((db[0] << 7) + db[1]) << 7) + db[2]);
  const float ca = fmaf(d * (float)sc_a, ta, -(dmin * mn_a) * sx[0]);
  const float cb = fmaf(d * (float)sc_b, tb, -(dmin * mn_b) * sx[1]);
  return fmaf(xinv[0], ca, xinv[1] * cb);
}

}  // namespace
