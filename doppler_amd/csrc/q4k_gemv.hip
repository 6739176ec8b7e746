// Q4_K dequantisation and the dequant-fused GEMV (M = 1..8) for gfx950.
//
// Weight layout is the reference's row layout, untouched: W[N,K] is N*ceil(K/256)
// super-blocks of 144 bytes; a block is {f16 d, f16 dmin, 12 bytes of 6-bit scales/mins,
// 128 bytes of nibbles}; byte j of 32-byte chunk c holds element 64c+j (low nibble,
// sub-block 2c) and 64c+32+j (high nibble, sub-block 2c+1).
//
// Work split used by every GEMV kernel here: four lanes share one super-block, lane c of
// the four owns chunk c = 64 weights = two whole sub-blocks, so each lane needs exactly one
// (scale, min) pair per nibble half, issues three 16-byte loads per block (header + two
// halves of its chunk) and a wave covers 16 consecutive blocks = 2304 contiguous bytes.
// Per sub-block the dot product is factored as  scale * sum(x*q) - min * sum(x)  so the
// inner loop is one byte->float convert and one FMA per weight, and sum(x) per 32-group is
// computed once per activation vector.
#include <algorithm>
#include <cstdlib>

#include "dh_common.h"

namespace {

using dh::kBlockBytes;
using dh::kQK;

__device__ __forceinline__ float f16lo(uint32_t v) {
  return __half2float(__ushort_as_half((unsigned short)(v & 0xffffu)));
}
__device__ __forceinline__ float f16hi(uint32_t v) {
  return __half2float(__ushort_as_half((unsigned short)(v >> 16)));
}

// Scales and mins of sub-blocks 2c and 2c+1 from the 16-byte block header.
// Bytes 4..7 (hdr.y): low 6 bits = scale 0..3, top 2 bits = high bits of scale 4..7.
// Bytes 8..11 (hdr.z): same for mins.  Bytes 12..15 (hdr.w): low nibble = scale 4..7 low
// bits, high nibble = min 4..7 low bits.
__device__ __forceinline__ void q4k_pair_scales(const uint4 hdr, const int c, float& sc_lo,
                                                float& sc_hi, float& mn_lo, float& mn_hi) {
  const float d = f16lo(hdr.x);
  const float dmin = f16hi(hdr.x);
  const int sh = (c & 1) * 16;
  const uint32_t a1 = hdr.y >> sh, a2 = hdr.z >> sh, a3 = hdr.w >> sh;
  uint32_t scp, mnp;
  if (c < 2) {
    scp = a1 & 0x3F3Fu;
    mnp = a2 & 0x3F3Fu;
  } else {
    scp = (a3 & 0x0F0Fu) | ((a1 >> 2) & 0x3030u);
    mnp = ((a3 >> 4) & 0x0F0Fu) | ((a2 >> 2) & 0x3030u);
  }
  sc_lo = d * (float)(scp & 0xFFu);
  sc_hi = d * (float)((scp >> 8) & 0xFFu);
  mn_lo = dmin * (float)(mnp & 0xFFu);
  mn_hi = dmin * (float)((mnp >> 8) & 0xFFu);
}

// ---------------------------------------------------------------------------------------
// Dequantise to f32, bit-exact: w = scale*q - min is the correctly rounded f32 of the exact
// value whichever way it is contracted (scale and scale*q are exact in f32).
// One thread per nibble byte: writes two outputs.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void q4k_dequant_kernel(const uint8_t* __restrict__ W,
                                                          int64_t num_blocks,
                                                          float* __restrict__ out) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t blk = t >> 7;
  if (blk >= num_blocks) return;
  const int byte = (int)(t & 127);
  const int c = byte >> 5, j = byte & 31;
  const uint8_t* b = W + blk * kBlockBytes;
  const uint4 hdr = *reinterpret_cast<const uint4*>(b);
  float sc_lo, sc_hi, mn_lo, mn_hi;
  q4k_pair_scales(hdr, c, sc_lo, sc_hi, mn_lo, mn_hi);
  const uint32_t q = b[16 + byte];
  float* o = out + blk * kQK + c * 64 + j;
  o[0] = sc_lo * (float)(q & 15u) - mn_lo;
  o[32] = sc_hi * (float)(q >> 4) - mn_hi;
}

// ---------------------------------------------------------------------------------------
// Generic GEMV: activations staged in LDS, any K (tail masked by zero activations), any
// blocks-per-row count.  DUAL computes two weight matrices against the same activations
// and combines them as act(g)*u (the fused gate/up projection).
// ---------------------------------------------------------------------------------------

// LDS index of activation k: 4 floats of padding after every 64 so that the 64 lanes of a
// wave, which read 16-byte vectors 256 bytes apart, spread over the banks.
__device__ __forceinline__ int xs_index(int k) { return k + ((k >> 6) << 2); }

struct GemvArgs {
  const float* A;       // [M][K]
  const uint8_t* W;     // Q4_K rows
  const uint8_t* W2;    // second matrix (DUAL) or null
  void* C;              // [M][N] f32 or f16
  const float* residual;
  int M, N, K, nb;
  float alpha;
  int c_f16;
  int rows_per_wave;    // multiple of rows-per-step
  int activation;       // DUAL: DH_ACT_SILU / DH_ACT_GELU
  float clamp_max;      // DUAL + silu: 0 = off
};

__device__ __forceinline__ float act_silu(float x) { return x / (1.0f + __expf(-x)); }
__device__ __forceinline__ float act_gelu(float x) {
  const float inner = 0.7978845608f * (x + 0.044715f * x * x * x);
  return 0.5f * x * (1.0f + tanhf(fminf(fmaxf(inner, -15.0f), 15.0f)));
}

template <int MT>
__device__ __forceinline__ void q4k_block_chunk_dot(const uint8_t* __restrict__ blk_ptr, const int c,
                                                    const float* __restrict__ xs,
                                                    const float* __restrict__ xsum, const int kp,
                                                    const int nsub, const int kb, const int sub0,
                                                    float (&acc)[MT]) {
  const uint4 hdr = *reinterpret_cast<const uint4*>(blk_ptr);
  const uint4 qa = *reinterpret_cast<const uint4*>(blk_ptr + 16 + c * 32);
  const uint4 qb = *reinterpret_cast<const uint4*>(blk_ptr + 32 + c * 32);
  float sc_lo, sc_hi, mn_lo, mn_hi;
  q4k_pair_scales(hdr, c, sc_lo, sc_hi, mn_lo, mn_hi);
  const uint32_t q[8] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w};
  const int xb = xs_index(kb);
#pragma unroll
  for (int m = 0; m < MT; m++) {
    const float* xm = xs + m * kp + xb;
    float dl = 0.f, dh = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float4 xl = *reinterpret_cast<const float4*>(xm + 4 * j);
      const float4 xh = *reinterpret_cast<const float4*>(xm + 32 + 4 * j);
      const uint32_t lo = q[j] & 0x0F0F0F0Fu;
      const uint32_t hi = (q[j] >> 4) & 0x0F0F0F0Fu;
      dl = fmaf(xl.x, (float)(lo & 0xFFu), dl);
      dl = fmaf(xl.y, (float)((lo >> 8) & 0xFFu), dl);
      dl = fmaf(xl.z, (float)((lo >> 16) & 0xFFu), dl);
      dl = fmaf(xl.w, (float)(lo >> 24), dl);
      dh = fmaf(xh.x, (float)(hi & 0xFFu), dh);
      dh = fmaf(xh.y, (float)((hi >> 8) & 0xFFu), dh);
      dh = fmaf(xh.z, (float)((hi >> 16) & 0xFFu), dh);
      dh = fmaf(xh.w, (float)(hi >> 24), dh);
    }
    const float sxl = xsum[m * nsub + sub0];
    const float sxh = xsum[m * nsub + sub0 + 1];
    acc[m] += sc_lo * dl - mn_lo * sxl + sc_hi * dh - mn_hi * sxh;
  }
}

template <int MT, bool DUAL>
__global__ __launch_bounds__(256) void q4k_gemv_lds_kernel(const GemvArgs a) {
  extern __shared__ float smem[];
  const int nb = a.nb;
  const int kpad = nb * kQK;
  const int kp = nb * (kQK + 16);  // padded floats per activation row
  const int nsub = nb * 8;
  float* xs = smem;                       // [MT][kp]
  float* xsum = xs + MT * kp;             // [MT][nsub]
  float* part = xsum + MT * nsub;         // [4 waves][64][MT * (DUAL ? 2 : 1)]
  constexpr int PV = MT * (DUAL ? 2 : 1);

  const int tid = threadIdx.x;
  // ---- stage activations (zero beyond K) and their 32-group sums
  for (int m = 0; m < MT; m++) {
    const float* am = a.A + (int64_t)m * a.K;
    for (int k = tid; k < kpad; k += 256) xs[m * kp + xs_index(k)] = k < a.K ? am[k] : 0.f;
  }
  __syncthreads();
  for (int i = tid; i < MT * nsub; i += 256) {
    const int m = i / nsub, g = i - m * nsub;
    const float* p = xs + m * kp + xs_index(g * 32);
    float s = 0.f;
#pragma unroll
    for (int j = 0; j < 32; j++) s += p[j];
    xsum[i] = s;
  }
  __syncthreads();

  const int wave = tid >> 6, lane = tid & 63;
  const int slot = lane >> 2, c = lane & 3;
  const int lanes_per_row = nb >= 16 ? 64 : nb * 4;
  const int rps = 64 / lanes_per_row;            // rows per step
  const int steps_per_row = nb >= 16 ? (nb + 15) / 16 : 1;
  const int64_t wave_row0 = ((int64_t)blockIdx.x * 4 + wave) * a.rows_per_wave;
  float* mypart = part + (wave * 64) * PV;
  const int64_t row_bytes = (int64_t)nb * kBlockBytes;

  for (int r = 0; r < a.rows_per_wave; r += rps) {
    const int rin = slot / (nb >= 16 ? 16 : nb);   // row within this step (0 when nb >= 16)
    const int64_t row = wave_row0 + r + rin;
    const bool row_ok = rin < rps && row < a.N && (r + rin) < a.rows_per_wave;
    float acc[MT], acc2[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m] = acc2[m] = 0.f;
    for (int s = 0; s < steps_per_row; s++) {
      const int blk = nb >= 16 ? s * 16 + slot : slot - rin * nb;
      if (row_ok && blk < nb) {
        const int64_t off = row * row_bytes + (int64_t)blk * kBlockBytes;
        const int kb = blk * kQK + c * 64;
        q4k_block_chunk_dot<MT>(a.W + off, c, xs, xsum, kp, nsub, kb, blk * 8 + 2 * c, acc);
        if (DUAL) q4k_block_chunk_dot<MT>(a.W2 + off, c, xs, xsum, kp, nsub, kb, blk * 8 + 2 * c, acc2);
      }
    }
    // ---- segmented reduction through this wave's own LDS slice (fixed order: deterministic)
#pragma unroll
    for (int m = 0; m < MT; m++) {
      mypart[lane * PV + m] = acc[m];
      if (DUAL) mypart[lane * PV + MT + m] = acc2[m];
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    for (int o = lane; o < rps * MT; o += 64) {
      const int orow = o / MT, m = o - orow * MT;
      const int64_t row_o = wave_row0 + r + orow;
      if (row_o < a.N && (r + orow) < a.rows_per_wave) {
        float s = 0.f, s2 = 0.f;
        for (int l = 0; l < lanes_per_row; l++) {
          s += mypart[(orow * lanes_per_row + l) * PV + m];
          if (DUAL) s2 += mypart[(orow * lanes_per_row + l) * PV + MT + m];
        }
        float v;
        if (DUAL) {
          const float g = a.activation == DH_ACT_SILU ? act_silu(s) : act_gelu(s);
          v = g * s2 * a.alpha;
          if (a.activation == DH_ACT_SILU && a.clamp_max > 0.f)
            v = fminf(fmaxf(v, -a.clamp_max), a.clamp_max);
        } else {
          v = s * a.alpha;
          if (a.residual) v += a.residual[(int64_t)m * a.N + row_o];
        }
        if (a.c_f16)
          reinterpret_cast<__half*>(a.C)[(int64_t)m * a.N + row_o] = __float2half(v);
        else
          reinterpret_cast<float*>(a.C)[(int64_t)m * a.N + row_o] = v;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// ---------------------------------------------------------------------------------------
// Decode GEMV (one activation row), activations resident in registers.
//
// A wave walks whole rows: LPR lanes cover one row slab per step (LPR = 64: 16 blocks =
// 4096 weights = 2304 contiguous bytes; rows with fewer blocks pack 64/LPR rows per step), so
// a lane always meets the SAME 64 activations x[kb .. kb+63].  They are converted once per
// wave into packed f16 pairs (a high part and a residual low part, scaled by a per-lane power
// of two so the pair carries ~22 bits of x) and stay in 64 VGPRs for every row.
//
// Nibbles never become floats: `w & 0x000F000F` read as two f16 values is (q0, q2) * 2^-24
// (f16 subnormals, which v_dot2_f32_f16 multiplies exactly), `w & 0x00F000F0` is
// (16 q0, 16 q2) * 2^-24 for the high nibbles.  Five integer ops unpack eight weights and one
// v_dot2_f32_f16 per activation part multiplies two of them, accumulating in f32; the
// powers of two are folded into the per-sub-block scale.  Rows longer than one slab are
// split over S waves whose partial sums meet in LDS once per 64 rows.
// ---------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(2))) _Float16 half2_t;

__device__ __forceinline__ half2_t as_h2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }

struct GemvM1Args {
  const float* x;        // [K]
  const uint8_t* W;      // Q4_K rows
  const uint8_t* W2;     // second matrix (DUAL) or null
  void* C;               // [N] f32 or f16
  const float* residual; // [N] or null
  int N, K, nb;
  float alpha;
  int c_f16;
  int activation;
  float clamp_max;
  int steps_per_wave;    // row steps each wave group walks
};

struct XRegs {
  half2_t hi[32];        // [4j+0]=(x[4j],x[4j+2]) [4j+1]=(x[4j+1],x[4j+3]) low-nibble side,
  half2_t lo[32];        // [4j+2],[4j+3] the same for x[32+4j..] (high-nibble side)
  float f_lo, f_hi;      // 2^24/sf and 2^20/sf: undo the subnormal and activation scalings
  float sx_lo, sx_hi;    // sum of the 32 activations of each sub-block (min term)
};

template <bool XLO>
__device__ __forceinline__ void load_x_regs(const float* __restrict__ x, int kb, int K, XRegs& r) {
  float v[64];
#pragma unroll
  for (int i = 0; i < 16; i++) {
    const int k = kb + 4 * i;
    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
    if (k + 3 < K) {
      t = *reinterpret_cast<const float4*>(x + k);
    } else {
      if (k < K) t.x = x[k];
      if (k + 1 < K) t.y = x[k + 1];
      if (k + 2 < K) t.z = x[k + 2];
    }
    v[4 * i] = t.x; v[4 * i + 1] = t.y; v[4 * i + 2] = t.z; v[4 * i + 3] = t.w;
  }
  float amax = 0.f, s0 = 0.f, s1 = 0.f;
#pragma unroll
  for (int i = 0; i < 32; i++) {
    amax = fmaxf(amax, fmaxf(fabsf(v[i]), fabsf(v[32 + i])));
    s0 += v[i];
    s1 += v[32 + i];
  }
  r.sx_lo = s0;
  r.sx_hi = s1;
  // sf = 2^(14 - floor(log2 amax)): the largest |x*sf| lands in [2^14, 2^15), inside f16 range
  int e = (int)((__float_as_uint(amax) >> 23) & 0xFF) - 127;
  e = max(-100, min(100, e));
  if (amax == 0.f) e = 14;
  const float sf = __uint_as_float((uint32_t)(127 + 14 - e) << 23);
  const float inv = __uint_as_float((uint32_t)(127 - 14 + e) << 23);
  r.f_lo = 16777216.0f * inv;
  r.f_hi = 1048576.0f * inv;
  auto pack = [&](float a, float b, half2_t& hi, half2_t& lo) {
    const float as = a * sf, bs = b * sf;
    const _Float16 ah = (_Float16)as, bh = (_Float16)bs;
    hi = half2_t{ah, bh};
    if (XLO) lo = half2_t{(_Float16)(as - (float)ah), (_Float16)(bs - (float)bh)};
  };
#pragma unroll
  for (int j = 0; j < 8; j++) {
    pack(v[4 * j], v[4 * j + 2], r.hi[4 * j], r.lo[4 * j]);
    pack(v[4 * j + 1], v[4 * j + 3], r.hi[4 * j + 1], r.lo[4 * j + 1]);
    pack(v[32 + 4 * j], v[32 + 4 * j + 2], r.hi[4 * j + 2], r.lo[4 * j + 2]);
    pack(v[32 + 4 * j + 1], v[32 + 4 * j + 3], r.hi[4 * j + 3], r.lo[4 * j + 3]);
  }
}

struct BlockChunk {
  uint4 hdr, qa, qb;
};

// Plain 16-byte load (a non-temporal hint measured ~20% slower on this streaming pattern).
__device__ __forceinline__ uint4 load_stream16(const uint8_t* __restrict__ p) {
  return *reinterpret_cast<const uint4*>(p);
}

__device__ __forceinline__ BlockChunk load_chunk(const uint8_t* __restrict__ p, int c) {
  BlockChunk b;
  b.hdr = load_stream16(p);
  b.qa = load_stream16(p + 16 + c * 32);
  b.qb = load_stream16(p + 32 + c * 32);
  return b;
}

template <bool XLO>
__device__ __forceinline__ float chunk_dot_regs(const BlockChunk& b, int c, const XRegs& r) {
  float sc_lo, sc_hi, mn_lo, mn_hi;
  q4k_pair_scales(b.hdr, c, sc_lo, sc_hi, mn_lo, mn_hi);
  const uint32_t q[8] = {b.qa.x, b.qa.y, b.qa.z, b.qa.w, b.qb.x, b.qb.y, b.qb.z, b.qb.w};
  float dl0 = 0.f, dl1 = 0.f, dh0 = 0.f, dh1 = 0.f;
#pragma unroll
  for (int j = 0; j < 8; j++) {
    const uint32_t w = q[j], t = w >> 8;
    const half2_t lo02 = as_h2(w & 0x000F000Fu), hi02 = as_h2(w & 0x00F000F0u);
    const half2_t lo13 = as_h2(t & 0x000F000Fu), hi13 = as_h2(t & 0x00F000F0u);
    dl0 = __builtin_amdgcn_fdot2(lo02, r.hi[4 * j], dl0, false);
    dl1 = __builtin_amdgcn_fdot2(lo13, r.hi[4 * j + 1], dl1, false);
    dh0 = __builtin_amdgcn_fdot2(hi02, r.hi[4 * j + 2], dh0, false);
    dh1 = __builtin_amdgcn_fdot2(hi13, r.hi[4 * j + 3], dh1, false);
    if (XLO) {
      dl0 = __builtin_amdgcn_fdot2(lo02, r.lo[4 * j], dl0, false);
      dl1 = __builtin_amdgcn_fdot2(lo13, r.lo[4 * j + 1], dl1, false);
      dh0 = __builtin_amdgcn_fdot2(hi02, r.lo[4 * j + 2], dh0, false);
      dh1 = __builtin_amdgcn_fdot2(hi13, r.lo[4 * j + 3], dh1, false);
    }
  }
  return (sc_lo * r.f_lo) * (dl0 + dl1) + (sc_hi * r.f_hi) * (dh0 + dh1) - mn_lo * r.sx_lo - mn_hi * r.sx_hi;
}

template <int LPR>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ float gemv_epilogue(float g, float u, bool dual, const GemvM1Args& a, int64_t row) {
  float v;
  if (dual) {
    const float act = a.activation == DH_ACT_SILU ? act_silu(g) : act_gelu(g);
    v = act * u * a.alpha;
    if (a.activation == DH_ACT_SILU && a.clamp_max > 0.f) v = fminf(fmaxf(v, -a.clamp_max), a.clamp_max);
  } else {
    v = g * a.alpha;
    if (a.residual) v += a.residual[row];
  }
  return v;
}

__device__ __forceinline__ void gemv_store(const GemvM1Args& a, int64_t row, float v) {
  if (a.c_f16)
    reinterpret_cast<__half*>(a.C)[row] = __float2half(v);
  else
    reinterpret_cast<float*>(a.C)[row] = v;
}

// LPR lanes per row (4 * blocks handled per wave step), S waves per row (slabs of 16 blocks),
// RG row groups per workgroup.  Requires nb == (LPR / 4) * S.
template <int LPR, int S, int RG, bool DUAL, bool XLO>
__global__ __launch_bounds__(64 * S * RG) void q4k_gemv_m1_kernel(const GemvM1Args a) {
  constexpr int RPS = 64 / LPR;   // rows per wave step
  __shared__ float part_g[S > 1 ? RG * S * 64 : 1];
  __shared__ float part_u[(S > 1 && DUAL) ? RG * S * 64 : 1];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slab = wave % S, rg = wave / S;
  const int c = lane & 3;
  const int blk = slab * 16 + ((lane % LPR) >> 2);
  const int rin = lane / LPR;
  XRegs xr;
  load_x_regs<XLO>(a.x, blk * kQK + c * 64, a.K, xr);

  const int64_t row_bytes = (int64_t)a.nb * kBlockBytes;
  const int64_t group_row0 = ((int64_t)blockIdx.x * RG + rg) * a.steps_per_wave * RPS;
  const int64_t lane_off = (int64_t)blk * kBlockBytes;
  float batch_g = 0.f, batch_u = 0.f;

  BlockChunk cur, cur2, nxt, nxt2;
  {
    const int64_t row = min(group_row0 + rin, (int64_t)a.N - 1);
    cur = load_chunk(a.W + row * row_bytes + lane_off, c);
    if (DUAL) cur2 = load_chunk(a.W2 + row * row_bytes + lane_off, c);
  }
  for (int st = 0; st < a.steps_per_wave; st++) {
    const int64_t row = group_row0 + (int64_t)st * RPS + rin;
    if (st + 1 < a.steps_per_wave) {
      const int64_t nrow = min(row + RPS, (int64_t)a.N - 1);   // clamped: loads stay in bounds
      nxt = load_chunk(a.W + nrow * row_bytes + lane_off, c);
      if (DUAL) nxt2 = load_chunk(a.W2 + nrow * row_bytes + lane_off, c);
    }
    float g = group_sum<LPR>(chunk_dot_regs<XLO>(cur, c, xr));
    float u = 0.f;
    if (DUAL) u = group_sum<LPR>(chunk_dot_regs<XLO>(cur2, c, xr));
    if (S == 1) {
      if ((lane % LPR) == 0 && row < a.N) gemv_store(a, row, gemv_epilogue(g, u, DUAL, a, row));
    } else {
      // LPR == 64 here: one row per step; lane (st % 64) keeps this row's partial sum
      if (lane == (st & 63)) { batch_g = g; batch_u = u; }
      if ((st & 63) == 63 || st + 1 == a.steps_per_wave) {
        part_g[(rg * S + slab) * 64 + lane] = batch_g;
        if (DUAL) part_u[(rg * S + slab) * 64 + lane] = batch_u;
        __syncthreads();
        if (slab == 0) {
          const int64_t orow = group_row0 + (st & ~63) + lane;
          if (lane <= (st & 63) && orow < a.N) {
            float sg = 0.f, su = 0.f;
#pragma unroll
            for (int s2 = 0; s2 < S; s2++) {
              sg += part_g[(rg * S + s2) * 64 + lane];
              if (DUAL) su += part_u[(rg * S + s2) * 64 + lane];
            }
            gemv_store(a, orow, gemv_epilogue(sg, su, DUAL, a, orow));
          }
        }
        __syncthreads();
      }
    }
    cur = nxt;
    if (DUAL) cur2 = nxt2;
  }
}

template <int LPR, int S, int RG, bool DUAL>
int launch_m1(GemvM1Args a, const char* op) {
  constexpr int RPS = 64 / LPR;
  // target ~2 waves per SIMD across the chip: 2048 waves = 2048 / S wave groups
  static int env_steps = -1;
  if (env_steps < 0) {
    const char* e = getenv("DH_GEMV_STEPS");
    env_steps = e ? atoi(e) : 0;
  }
  const int64_t total_steps = dh::ceil_div(a.N, RPS);
  int steps = env_steps > 0 ? env_steps : (int)std::max<int64_t>(4, dh::ceil_div(total_steps, 2048 / S));
  a.steps_per_wave = steps;
  const int grid = (int)dh::ceil_div(total_steps, (int64_t)steps * RG);
  hipLaunchKernelGGL((q4k_gemv_m1_kernel<LPR, S, RG, DUAL, true>), dim3(grid), dim3(64 * S * RG), 0, dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  return 0;
}

// Returns -1 when the shape is not served by the register-resident kernel.
template <bool DUAL>
int dispatch_m1(const GemvM1Args& a, const char* op) {
  switch (a.nb) {
    case 1: return launch_m1<4, 1, 4, DUAL>(a, op);
    case 2: return launch_m1<8, 1, 4, DUAL>(a, op);
    case 4: return launch_m1<16, 1, 4, DUAL>(a, op);
    case 8: return launch_m1<32, 1, 4, DUAL>(a, op);
    case 16: return launch_m1<64, 1, 4, DUAL>(a, op);
    case 32: return launch_m1<64, 2, 2, DUAL>(a, op);
    case 48: return launch_m1<64, 3, 2, DUAL>(a, op);
    case 64: return launch_m1<64, 4, 1, DUAL>(a, op);
    default: return -1;
  }
}

// ---------------------------------------------------------------------------------------
// GEMV on the matrix cores, M = 1..8 activation rows in one pass over the weights.
//
// v_mfma_f32_32x32x16_f16 computes D[32][32] += A[32][16] . B[16][32].  Here B is a tile of 32
// weight rows x 16 weights of one sub-block, A holds the activations for the same 16 k as up
// to 32 "x-columns": each activation row m contributes two, a high f16 part and the f16
// residual of x * 2^e (e per row, so the largest element sits just inside f16 range), which
// keeps ~22 bits of every activation.  The nibbles are never converted: masked in place they
// ARE f16 subnormals (q * 2^-24, or 16 q * 2^-24 for the high nibble) and the matrix core
// multiplies subnormal inputs exactly.  What is left for the vector ALU is 5 integer ops per
// 8 weights to mask, one multiply-add per output and sub-block for the 6-bit scale, and the
// min term (sum of the sub-block's activations times its 6-bit min).
//
// Lane l owns weight row (l & 31) of the tile and half g2 = l >> 5 of every 32-byte chunk:
// five 16-byte loads per super-block (header + 4 half-chunks), each serving two nibble
// MFMAs of 16 k (k-slots: its bytes 0..7, then 8..15).  D comes back with x-column rows for
// that same weight row, so the scale and min of "its" row are already in its registers: no
// cross-lane traffic in the inner loop.  Rows are cut into K slices of BPW blocks, one wave
// each, so even a 4096-row matrix yields thousands of wave tasks; every wave issues all of
// its weight loads first, the workgroup then stages the activation fragments in LDS while
// those loads are in flight, and the K-slice partial sums meet in LDS at the end.
// ---------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) _Float16 half8_t;
typedef __attribute__((ext_vector_type(16))) float float16_t;

struct MfmaArgs {
  const float* A;        // [M][K]
  const uint8_t* W;      // Q4_K rows
  const uint8_t* W2;     // second matrix (DUAL) or null
  void* C;               // [M][N] f32 or f16
  const float* residual; // [M][N] or null
  int M, N, K, nb;
  float alpha;
  int c_f16, activation;
  float clamp_max;
};

struct WBlock {
  uint4 hdr;
  uint4 q[4];            // bytes [16*g2, 16*g2+16) of chunk c
};

__device__ __forceinline__ half8_t nib_frag(uint32_t w0, uint32_t w1, uint32_t mask) {
  typedef __attribute__((ext_vector_type(4))) uint32_t u4;
  const u4 v = {w0 & mask, (w0 >> 8) & mask, w1 & mask, (w1 >> 8) & mask};
  return __builtin_bit_cast(half8_t, v);
}

// Number of D entries a lane has to keep: x-column r lives in lane half (r >> 2) & 1, entry
// 4 * (r >> 3) + (r & 3).
template <int MT> struct MfmaShape { static constexpr int NI = MT == 1 ? 2 : (MT <= 4 ? 4 : 8); };

// One super-block of one 32-row tile.  acc[k]: activation row mrow(k) = (k&1) + 2*g2 + 4*(k>>1).
// sxi[sb][m] = (sum of the sub-block's 32 activations, 2^24 / activation scale of the sub-block).
template <int MT>
__device__ __forceinline__ void mfma_block(const WBlock& w, const _Float16* __restrict__ xfl, int xf_stride,
                                           const float2* __restrict__ sxi, int sb0, int g2,
                                           float (&acc)[MfmaShape<MT>::NI / 2]) {
  constexpr int NI = MfmaShape<MT>::NI, NO = NI / 2;
  // all eight 6-bit scales / mins of this lane's weight row, one byte each
  const uint32_t sc_lo4 = w.hdr.y & 0x3F3F3F3Fu;
  const uint32_t mn_lo4 = w.hdr.z & 0x3F3F3F3Fu;
  const uint32_t sc_hi4 = (w.hdr.w & 0x0F0F0F0Fu) | ((w.hdr.y >> 2) & 0x30303030u);
  const uint32_t mn_hi4 = ((w.hdr.w >> 4) & 0x0F0F0F0Fu) | ((w.hdr.z >> 2) & 0x30303030u);
  const float d = f16lo(w.hdr.x);
  const float dmin = f16hi(w.hdr.x);
  float blk[NO], blk_min[NO];
#pragma unroll
  for (int k = 0; k < NO; k++) blk[k] = blk_min[k] = 0.f;
  const float16_t zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int c = 0; c < 4; c++) {
    const uint32_t qw[4] = {w.q[c].x, w.q[c].y, w.q[c].z, w.q[c].w};
#pragma unroll
    for (int p = 0; p < 2; p++) {
      const int sb = 2 * c + p;
      // this lane's fragment of x-column (lane & 31) for k-slots [16*g2, 16*g2+16) of the
      // sub-block; lanes beyond the last x-column read a zero row (stride 0)
      const _Float16* xp = xfl + (sb0 + sb) * xf_stride;
      const half8_t xa0 = *reinterpret_cast<const half8_t*>(xp);
      const half8_t xa1 = *reinterpret_cast<const half8_t*>(xp + 8);
      const uint32_t mask = p ? 0x00F000F0u : 0x000F000Fu;
      float16_t dd = __builtin_amdgcn_mfma_f32_32x32x16_f16(xa0, nib_frag(qw[0], qw[1], mask), zero, 0, 0, 0);
      dd = __builtin_amdgcn_mfma_f32_32x32x16_f16(xa1, nib_frag(qw[2], qw[3], mask), dd, 0, 0, 0);
      const uint32_t sc4 = sb < 4 ? sc_lo4 : sc_hi4, mn4 = sb < 4 ? mn_lo4 : mn_hi4;
      // high nibbles carry an extra factor 16
      const float scf = (float)((sc4 >> (8 * (sb & 3))) & 0xFFu) * (p ? 0.0625f : 1.0f);
      const float mnf = (float)((mn4 >> (8 * (sb & 3))) & 0xFFu);
#pragma unroll
      for (int k = 0; k < NO; k++) {
        const int m = min((k & 1) + 2 * g2 + 4 * (k >> 1), MT - 1);
        const float2 si = sxi[(sb0 + sb) * MT + m];
        blk[k] = fmaf(scf * si.y, dd[2 * k] + dd[2 * k + 1], blk[k]);   // high + residual part
        blk_min[k] = fmaf(mnf, si.x, blk_min[k]);
      }
    }
  }
#pragma unroll
  for (int k = 0; k < NO; k++) acc[k] += d * blk[k] - dmin * blk_min[k];
}

// Loads this thread's 16-byte chunks of one tile slab (32 rows x SB super-blocks) into registers.
template <int SB, int NL, int NTHR>
__device__ __forceinline__ void gemv_slab_load(const uint8_t* __restrict__ base, int64_t tile, int s, int tid,
                                               int N, int nb, int64_t row_bytes, uint4 (&wreg)[NL]) {
  constexpr int SEG = SB * kBlockBytes, CH = SEG / 16, TOT = 32 * CH;
#pragma unroll
  for (int t = 0; t < NL; t++) {
    const int q = t * NTHR + tid;
    const int r = q / CH, within = (q - r * CH) * 16;
    if (q < TOT && s * SB + within / kBlockBytes < nb) {
      const int64_t row = min(tile * 32 + r, (int64_t)N - 1);
      wreg[t] = *reinterpret_cast<const uint4*>(base + row * row_bytes + (int64_t)s * SEG + within);
    }
  }
}

// MT activation rows (a.M <= MT); a workgroup of WAVES waves walks 32-row tiles in slabs of SB
// super-blocks.  Weights travel HBM -> registers -> LDS with fully contiguous 16-byte loads
// (each row contributes SB*144 consecutive bytes per slab, lanes take consecutive chunks), the
// next slab's loads are issued before the current slab is consumed, and every wave then reads
// its own super-blocks back from LDS in the MFMA operand layout.
template <int MT, int SB, bool DUAL, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void q4k_gemv_mfma_kernel(const MfmaArgs a) {
  constexpr int NTHR = 64 * WAVES;
  constexpr int XC = 2 * MT, NO = MfmaShape<MT>::NI / 2, NMAT = DUAL ? 2 : 1;
  constexpr int SEG = SB * kBlockBytes;          // bytes of one row in one slab
  constexpr int RS = SEG + 16;                   // LDS row stride: skews rows across banks
  constexpr int CH = SEG / 16;                   // 16-byte chunks per row segment
  constexpr int TOT = 32 * CH;                   // chunks per tile slab
  constexpr int NL = (TOT + NTHR - 1) / NTHR;    // chunks per thread
  constexpr int BPWAVE = (SB + WAVES - 1) / WAVES;   // super-blocks per wave per slab
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int nsub = a.nb * 8;
  _Float16* xf = reinterpret_cast<_Float16*>(smem_raw);                 // [nsub][XC][32]
  _Float16* xzero = xf + (size_t)nsub * XC * 32;                        // 32 zero halves
  float2* sxi = reinterpret_cast<float2*>(xzero + 32);                  // [nsub][MT]
  unsigned char* wl = reinterpret_cast<unsigned char*>(sxi + (size_t)nsub * MT);   // [32][RS]
  float* red = reinterpret_cast<float*>(wl + 32 * RS);                  // [WAVES][NMAT][NO][64]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wr = lane & 31, g2 = lane >> 5, xcol = lane & 31;
  const int64_t row_bytes = (int64_t)a.nb * kBlockBytes;
  const int nslab = (a.nb + SB - 1) / SB;
  const int64_t ntiles = ((int64_t)a.N + 31) / 32;

  // ---- this thread's share of the activations first (cache hits, short latency) ...
  // Work item = (activation row m, sub-block sb): 32 contiguous floats as eight 16-byte loads.
  const int items = MT * nsub;
  float xv[32];
  auto load32 = [&](int idx, float (&v)[32]) {
    const int sb = idx / MT, m = idx - sb * MT;
    const float* src = a.A + (int64_t)m * a.K + sb * 32;
    const int left = a.K - sb * 32;
#pragma unroll
    for (int q4 = 0; q4 < 8; q4++) {
      float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
      if (m < a.M) {
        if (4 * q4 + 3 < left) {
          t = *reinterpret_cast<const float4*>(src + 4 * q4);
        } else {
          if (4 * q4 < left) t.x = src[4 * q4];
          if (4 * q4 + 1 < left) t.y = src[4 * q4 + 1];
          if (4 * q4 + 2 < left) t.z = src[4 * q4 + 2];
        }
      }
      v[4 * q4] = t.x; v[4 * q4 + 1] = t.y; v[4 * q4 + 2] = t.z; v[4 * q4 + 3] = t.w;
    }
  };
  if (tid < items) load32(tid, xv);

  // ---- ... then the first slab of weights, in flight while the activations are converted
  uint4 wreg[NL];
#pragma unroll
  for (int t = 0; t < NL; t++) wreg[t] = make_uint4(0, 0, 0, 0);
#define DH_GLOAD(tile_, mat_, s_) \
  gemv_slab_load<SB, NL, NTHR>(((DUAL && (mat_)) ? a.W2 : a.W), (tile_), (s_), tid, a.N, a.nb, row_bytes, wreg)
  if ((int64_t)blockIdx.x < ntiles) DH_GLOAD(blockIdx.x, 0, 0);

  // ---- stage the activations in LDS.  Each sub-block gets its own power-of-two scale
  // (largest element just inside f16 range), so no reduction across threads is needed:
  // f16 high part, f16 residual, the plain sum (min term) and 2^24 / scale per (sb, m).
  auto stage = [&](int idx, const float (&v)[32]) {
    const int sb = idx / MT, m = idx - sb * MT;
    float s = 0.f, mx = 0.f;
#pragma unroll
    for (int j = 0; j < 32; j++) { s += v[j]; mx = fmaxf(mx, fabsf(v[j])); }
    int e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 127;
    e = max(-100, min(100, e));
    if (mx == 0.f) e = 14;
    const float sf = __uint_as_float((uint32_t)(127 + 14 - e) << 23);          // 2^(14-e)
    sxi[idx] = make_float2(s, __uint_as_float((uint32_t)(127 + 24 - 14 + e) << 23));   // 2^24 / sf
#pragma unroll
    for (int grp = 0; grp < 4; grp++) {
      half8_t hi, lo;
#pragma unroll
      for (int slot = 0; slot < 8; slot++) {
        // slot order inside a k-group follows the masked dwords: (b0,b2) (b1,b3) (b4,b6) (b5,b7)
        const int o = (slot & 4) | ((slot & 1) << 1) | ((slot >> 1) & 1);
        const float xs = v[grp * 8 + o] * sf;
        const _Float16 h = (_Float16)xs;
        hi[slot] = h;
        lo[slot] = (_Float16)(xs - (float)h);
      }
      *reinterpret_cast<half8_t*>(xf + (sb * XC + 2 * m) * 32 + grp * 8) = hi;
      *reinterpret_cast<half8_t*>(xf + (sb * XC + 2 * m + 1) * 32 + grp * 8) = lo;
    }
  };
  if (tid < items) stage(tid, xv);
  for (int idx = tid + NTHR; idx < items; idx += NTHR) {
    float v[32];
    load32(idx, v);
    stage(idx, v);
  }
  if (tid < 16) reinterpret_cast<uint32_t*>(xzero)[tid] = 0u;

  const _Float16* xfl = xcol < XC ? xf + xcol * 32 + g2 * 16 : xzero;
  const int xf_stride = xcol < XC ? XC * 32 : 0;

  for (int64_t tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
    float acc[NMAT][NO];
#pragma unroll
    for (int mt = 0; mt < NMAT; mt++)
#pragma unroll
      for (int k = 0; k < NO; k++) acc[mt][k] = 0.f;
#pragma unroll
    for (int mat = 0; mat < NMAT; mat++) {
      for (int s = 0; s < nslab; s++) {
        __syncthreads();   // everyone is done reading the previous slab (and, first time, staging x)
#pragma unroll
        for (int t = 0; t < NL; t++) {
          const int q = t * NTHR + tid;
          const int r = q / CH, within = (q - r * CH) * 16;
          if (q < TOT) *reinterpret_cast<uint4*>(wl + r * RS + within) = wreg[t];
        }
        __syncthreads();
        // next slab (next matrix, next tile) goes in flight before this one is consumed
        if (s + 1 < nslab) DH_GLOAD(tile, mat, s + 1);
        else if (mat + 1 < NMAT) DH_GLOAD(tile, mat + 1, 0);
        else if (tile + gridDim.x < ntiles) DH_GLOAD(tile + gridDim.x, 0, 0);
#pragma unroll
        for (int bb = 0; bb < BPWAVE; bb++) {
          const int bl = wave * BPWAVE + bb;           // super-block within the slab
          const int blk = s * SB + bl;
          if (bl < SB && blk < a.nb) {
            const unsigned char* p = wl + wr * RS + bl * kBlockBytes;
            WBlock w;
            w.hdr = *reinterpret_cast<const uint4*>(p);
#pragma unroll
            for (int c = 0; c < 4; c++) w.q[c] = *reinterpret_cast<const uint4*>(p + 16 + 32 * c + 16 * g2);
            mfma_block<MT>(w, xfl, xf_stride, sxi, blk * 8, g2, acc[mat]);
          }
        }
      }
    }
    // ---- the four waves' partial sums meet in LDS
#pragma unroll
    for (int mt = 0; mt < NMAT; mt++)
#pragma unroll
      for (int k = 0; k < NO; k++) red[((wave * NMAT + mt) * NO + k) * 64 + lane] = acc[mt][k];
    __syncthreads();
    for (int o = tid; o < NO * 64; o += NTHR) {
      const int ln = o & 63, k = o >> 6;
      const int m = (k & 1) + 2 * (ln >> 5) + 4 * (k >> 1);
      const int64_t row = tile * 32 + (ln & 31);
      if (m >= a.M || row >= a.N) continue;
      float sg = 0.f, su = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; w++) {
        sg += red[((w * NMAT) * NO + k) * 64 + ln];
        if (DUAL) su += red[((w * NMAT + 1) * NO + k) * 64 + ln];
      }
      float v;
      if (DUAL) {
        const float act = a.activation == DH_ACT_SILU ? act_silu(sg) : act_gelu(sg);
        v = act * su * a.alpha;
        if (a.activation == DH_ACT_SILU && a.clamp_max > 0.f) v = fminf(fmaxf(v, -a.clamp_max), a.clamp_max);
      } else {
        v = sg * a.alpha;
        if (a.residual) v += a.residual[(int64_t)m * a.N + row];
      }
      if (a.c_f16)
        reinterpret_cast<__half*>(a.C)[(int64_t)m * a.N + row] = __float2half(v);
      else
        reinterpret_cast<float*>(a.C)[(int64_t)m * a.N + row] = v;
    }
    // `red` is rewritten only after the next tile's slab barriers: no extra barrier needed
  }
#undef DH_GLOAD
}

size_t mfma_lds_bytes(int mt, int nb, int sb, bool dual, int waves) {
  const size_t nsub = (size_t)nb * 8;
  const int no = (mt == 1 ? 2 : (mt <= 4 ? 4 : 8)) / 2;
  return nsub * 2 * mt * 32 * 2 + 64 + nsub * mt * 8 + (size_t)32 * (sb * kBlockBytes + 16) +
         (size_t)waves * (dual ? 2 : 1) * no * 64 * 4;
}

constexpr size_t kMfmaMaxLds = 160 * 1024;

template <int MT, int SB, bool DUAL, int WAVES>
int launch_mfma_cfg(MfmaArgs a, const char* op) {
  const size_t lds = mfma_lds_bytes(MT, a.nb, SB, DUAL, WAVES);
  auto kern = q4k_gemv_mfma_kernel<MT, SB, DUAL, WAVES>;
  static bool attr_set = false;   // once per instantiation: the call costs microseconds
  if (!attr_set) {
    DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMfmaMaxLds));
    attr_set = true;
  }
  static int env_grid = -1;
  if (env_grid < 0) {
    const char* e = getenv("DH_GEMV_GRID");
    env_grid = e ? atoi(e) : 0;
  }
  // one tile per workgroup until the chip is covered ~4x, then workgroups walk several tiles
  const int64_t ntiles = dh::ceil_div(a.N, 32);
  const int grid = (int)std::min<int64_t>(ntiles, env_grid > 0 ? env_grid : 1024);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WAVES), lds, dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  return 0;
}

// Slab size: 4 super-blocks keep the workgroup's LDS small (several workgroups per CU overlap
// their phases); long rows use 16 so that few workgroups still keep enough bytes in flight.
template <int MT, bool DUAL>
int launch_mfma(const MfmaArgs& a, const char* op) {
  static int env_sb = -1;
  if (env_sb < 0) {
    const char* e = getenv("DH_GEMV_SB");
    env_sb = e ? atoi(e) : 0;
  }
  static int env_waves = -1;
  if (env_waves < 0) {
    const char* e = getenv("DH_GEMV_WAVES");
    env_waves = e ? atoi(e) : 0;
  }
  const int waves = env_waves > 0 ? env_waves : 8;
  int sb = env_sb > 0 ? env_sb : 16;
  while (sb > 4 && mfma_lds_bytes(MT, a.nb, sb, DUAL, waves) > kMfmaMaxLds) sb /= 2;
  if (mfma_lds_bytes(MT, a.nb, sb, DUAL, waves) > kMfmaMaxLds) return -1;
#define DH_CFG(S_, W_) if (sb == S_ && waves == W_) return launch_mfma_cfg<MT, S_, DUAL, W_>(a, op)
  DH_CFG(4, 4); DH_CFG(8, 4); DH_CFG(16, 4); DH_CFG(8, 8); DH_CFG(16, 8); DH_CFG(16, 16);
#undef DH_CFG
  return -1;
}

// Returns -1 when the shape is not served (activations too large for LDS).
template <bool DUAL>
int dispatch_mfma(const MfmaArgs& a, const char* op) {
  if (a.M > 8) return -1;
  const int mt = a.M <= 1 ? 1 : a.M <= 2 ? 2 : a.M <= 4 ? 4 : 8;
  switch (mt) {
    case 1: return launch_mfma<1, DUAL>(a, op);
    case 2: return launch_mfma<2, DUAL>(a, op);
    case 4: return launch_mfma<4, DUAL>(a, op);
    default: return launch_mfma<8, DUAL>(a, op);
  }
}

constexpr size_t kMaxLds = 128 * 1024;

size_t lds_bytes(int mt, int nb, bool dual) {
  return sizeof(float) * ((size_t)mt * nb * (kQK + 16) + (size_t)mt * nb * 8 +
                          (size_t)4 * 64 * mt * (dual ? 2 : 1));
}

template <int MT, bool DUAL>
int launch_lds(const GemvArgs& a, const char* op) {
  const size_t lds = lds_bytes(MT, a.nb, DUAL);
  auto kern = q4k_gemv_lds_kernel<MT, DUAL>;
  static bool attr_set = false;   // once per instantiation: the call costs microseconds
  if (!attr_set) {
    DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
    attr_set = true;
  }
  const int lanes_per_row = a.nb >= 16 ? 64 : a.nb * 4;
  const int rps = 64 / lanes_per_row;
  // enough rows per wave to amortise the activation staging, few enough to fill the chip
  int steps = (int)std::min<int64_t>(8, std::max<int64_t>(1, a.N / ((int64_t)4 * rps * 1024)));
  GemvArgs b = a;
  b.rows_per_wave = rps * steps;
  const int64_t rows_per_wg = (int64_t)4 * b.rows_per_wave;
  const int grid = (int)dh::ceil_div(a.N, rows_per_wg);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, dh::stream(), b);
  DH_CHECK_LAUNCH(op);
  return 0;
}

template <bool DUAL>
int dispatch_lds(GemvArgs a, const char* op) {
  // largest activation tile that fits in LDS; more rows of A than that re-read the weights
  int mt = a.M;
  while (mt > 1 && lds_bytes(mt, a.nb, DUAL) > kMaxLds) mt--;
  if (lds_bytes(mt, a.nb, DUAL) > kMaxLds)
    return dh::fail(1, "[%s] K=%d too large for the LDS-staged GEMV (max %zu bytes of LDS)", op, a.K,
                    kMaxLds);
  const int total_m = a.M;
  const size_t c_elem = a.c_f16 ? 2 : 4;
  for (int m0 = 0; m0 < total_m; m0 += mt) {
    GemvArgs b = a;
    const int cur = std::min(mt, total_m - m0);
    b.M = cur;
    b.A = a.A + (int64_t)m0 * a.K;
    b.C = static_cast<char*>(a.C) + (int64_t)m0 * a.N * c_elem;
    b.residual = a.residual ? a.residual + (int64_t)m0 * a.N : nullptr;
    int rc = 0;
    switch (cur) {
      case 1: rc = launch_lds<1, DUAL>(b, op); break;
      case 2: rc = launch_lds<2, DUAL>(b, op); break;
      case 3: rc = launch_lds<3, DUAL>(b, op); break;
      case 4: rc = launch_lds<4, DUAL>(b, op); break;
      case 5: rc = launch_lds<5, DUAL>(b, op); break;
      case 6: rc = launch_lds<6, DUAL>(b, op); break;
      case 7: rc = launch_lds<7, DUAL>(b, op); break;
      default: rc = launch_lds<8, DUAL>(b, op); break;
    }
    if (rc) return rc;
  }
  return 0;
}

// Kernel family used for M <= 8: 0 = matrix-core GEMV (default), 1 = register-resident
// dot2 GEMV for M == 1, 2 = LDS-staged vector GEMV.  DH_GEMV_PATH overrides (for measurements).
int gemv_path() {
  static int path = -1;
  if (path < 0) {
    const char* e = getenv("DH_GEMV_PATH");
    path = e ? atoi(e) : 0;
  }
  return path;
}

}  // namespace

extern "C" {

int dh_q4k_dequant(const void* d_W, int64_t num_blocks, float* d_out) {
  DH_REQUIRE_INIT("dh_q4k_dequant");
  if (num_blocks == 0) return 0;
  if (!d_W || !d_out) return dh::fail(1, "[dh_q4k_dequant] null pointer");
  if (num_blocks < 0 || num_blocks > (int64_t)1 << 31)
    return dh::fail(1, "[dh_q4k_dequant] invalid block count %lld", (long long)num_blocks);
  if (reinterpret_cast<uintptr_t>(d_W) & 15)
    return dh::fail(1, "[dh_q4k_dequant] weight pointer must be 16-byte aligned");
  const int64_t threads = num_blocks * 128;
  hipLaunchKernelGGL(q4k_dequant_kernel, dim3((unsigned)dh::ceil_div(threads, 256)), dim3(256), 0,
                     dh::stream(), static_cast<const uint8_t*>(d_W), num_blocks, d_out);
  DH_CHECK_LAUNCH("dh_q4k_dequant");
  return 0;
}

int dh_q4k_matmul(const void* d_A, int a_dtype, const void* d_W, void* d_C, int c_dtype, int M,
                  int N, int K, float alpha, const void* d_residual) {
  const char* op = "dh_q4k_matmul";
  DH_REQUIRE_INIT(op);
  if (M <= 0 || N <= 0 || K <= 0)
    return dh::fail(1, "[%s] Dimensions must be positive: M=%d, N=%d, K=%d", op, M, N, K);
  if (!d_A || !d_W || !d_C) return dh::fail(1, "[%s] null pointer", op);
  if (a_dtype != DH_F32) return dh::fail(1, "[%s] activations must be f32 (a_dtype=%d)", op, a_dtype);
  if (c_dtype != DH_F32 && c_dtype != DH_F16)
    return dh::fail(1, "[%s] output dtype must be f32 or f16 (c_dtype=%d)", op, c_dtype);
  if (reinterpret_cast<uintptr_t>(d_W) & 15)
    return dh::fail(1, "[%s] weight pointer must be 16-byte aligned", op);
  GemvArgs a{};
  a.A = static_cast<const float*>(d_A);
  a.W = static_cast<const uint8_t*>(d_W);
  a.W2 = nullptr;
  a.C = d_C;
  a.residual = static_cast<const float*>(d_residual);
  a.M = M; a.N = N; a.K = K;
  a.nb = (K + kQK - 1) / kQK;
  a.alpha = alpha;
  a.c_f16 = c_dtype == DH_F16;
  const int path = gemv_path();
  if (path == 0 && M <= 8) {
    MfmaArgs g{};
    g.A = a.A; g.W = a.W; g.W2 = nullptr; g.C = d_C; g.residual = a.residual;
    g.M = M; g.N = N; g.K = K; g.nb = a.nb; g.alpha = alpha; g.c_f16 = a.c_f16;
    const int rc = dispatch_mfma<false>(g, op);
    if (rc >= 0) return rc;
  }
  if (path <= 1 && M == 1 && (reinterpret_cast<uintptr_t>(d_A) & 15) == 0) {
    GemvM1Args g{};
    g.x = a.A; g.W = a.W; g.W2 = nullptr; g.C = d_C; g.residual = a.residual;
    g.N = N; g.K = K; g.nb = a.nb; g.alpha = alpha; g.c_f16 = a.c_f16;
    const int rc = dispatch_m1<false>(g, op);
    if (rc >= 0) return rc;
  }
  // tiles of up to 8 activation rows per pass over the weights
  const size_t c_elem = a.c_f16 ? 2 : 4;
  for (int m0 = 0; m0 < M; m0 += 8) {
    GemvArgs b = a;
    b.M = std::min(8, M - m0);
    b.A = a.A + (int64_t)m0 * K;
    b.C = static_cast<char*>(d_C) + (int64_t)m0 * N * c_elem;
    b.residual = a.residual ? a.residual + (int64_t)m0 * N : nullptr;
    const int rc = dispatch_lds<false>(b, op);
    if (rc) return rc;
  }
  return 0;
}

int dh_q4k_ffn_gate_up(const float* d_x, const void* d_Wgate, const void* d_Wup, float* d_out, int M,
                       int hidden, int inter, int activation, float alpha, float swiglu_limit) {
  const char* op = "dh_q4k_ffn_gate_up";
  DH_REQUIRE_INIT(op);
  if (M <= 0 || hidden <= 0 || inter <= 0)
    return dh::fail(1, "[%s] Dimensions must be positive: M=%d, hidden=%d, inter=%d", op, M, hidden, inter);
  if (!d_x || !d_Wgate || !d_Wup || !d_out) return dh::fail(1, "[%s] null pointer", op);
  if (activation != DH_ACT_SILU && activation != DH_ACT_GELU)
    return dh::fail(1, "[%s] unknown activation %d", op, activation);
  if ((reinterpret_cast<uintptr_t>(d_Wgate) | reinterpret_cast<uintptr_t>(d_Wup)) & 15)
    return dh::fail(1, "[%s] weight pointers must be 16-byte aligned", op);
  GemvArgs a{};
  a.A = d_x;
  a.W = static_cast<const uint8_t*>(d_Wgate);
  a.W2 = static_cast<const uint8_t*>(d_Wup);
  a.C = d_out;
  a.residual = nullptr;
  a.N = inter; a.K = hidden;
  a.nb = (hidden + kQK - 1) / kQK;
  a.alpha = alpha;
  a.c_f16 = 0;
  a.activation = activation;
  a.clamp_max = swiglu_limit;
  const int path = gemv_path();
  if (path == 0 && M <= 8) {
    MfmaArgs g{};
    g.A = d_x; g.W = a.W; g.W2 = a.W2; g.C = d_out; g.residual = nullptr;
    g.M = M; g.N = inter; g.K = hidden; g.nb = a.nb; g.alpha = alpha; g.c_f16 = 0;
    g.activation = activation; g.clamp_max = swiglu_limit;
    const int rc = dispatch_mfma<true>(g, op);
    if (rc >= 0) return rc;
  }
  if (path <= 1 && M == 1 && (reinterpret_cast<uintptr_t>(d_x) & 15) == 0) {
    GemvM1Args g{};
    g.x = d_x; g.W = a.W; g.W2 = a.W2; g.C = d_out; g.residual = nullptr;
    g.N = inter; g.K = hidden; g.nb = a.nb; g.alpha = alpha; g.c_f16 = 0;
    g.activation = activation; g.clamp_max = swiglu_limit;
    const int rc = dispatch_m1<true>(g, op);
    if (rc >= 0) return rc;
  }
  // any batch: tiles of up to 8 activation rows per pass
  for (int m0 = 0; m0 < M; m0 += 8) {
    GemvArgs b = a;
    b.M = std::min(8, M - m0);
    b.A = d_x + (int64_t)m0 * hidden;
    b.C = d_out + (int64_t)m0 * inter;
    const int rc = dispatch_lds<true>(b, op);
    if (rc) return rc;
  }
  return 0;
}

}  // extern "C"
