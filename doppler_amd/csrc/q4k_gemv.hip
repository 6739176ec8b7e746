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
#include "q4k_device.h"

namespace {

using dh::kBlockBytes;
using dh::kQK;

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
// GEMV on the matrix cores, M = 1..8 activation rows in one pass over the weights.
//
// v_mfma_f32_32x32x16_f16 computes D[32][32] += A[32][16] . B[16][32].  Here B is a tile of 32
// weight rows x 16 weights of one sub-block, A holds the activations for the same 16 k as up
// to 32 "x-columns": each activation row m contributes two, a high f16 part and the f16
// residual of x * 2^e (e per sub-block, so its largest element sits just inside f16 range),
// which keeps ~22 bits of every activation.  The nibbles are never converted: masked in
// place they ARE f16 subnormals (q * 2^-24, or 16 q * 2^-24 for the high nibble) and the
// matrix core multiplies subnormal inputs exactly.  What is left for the vector ALU is 5
// integer ops per 8 weights to mask, one multiply-add per output and sub-block for the 6-bit
// scale, and the min term (sum of the sub-block's activations times its 6-bit min).
//
// A kernel this short-lived (microseconds) pays for every instruction byte it touches: all
// compute units fetch the same code at the same moment.  The body is therefore kept small:
// loops stay rolled except the 8 sub-blocks of a super-block, edge handling lives in one
// shared slow path, and one kernel instance serves every tile.
//
// Data path: a workgroup of 8 waves owns 32-row tiles.  A tile slab (32 rows x SB
// super-blocks) travels HBM -> registers -> LDS as contiguous 16-byte chunks (a row
// contributes SB*144 consecutive bytes, consecutive lanes take consecutive chunks); the next
// slab's loads are issued before the current one is consumed.  Each wave then reads its own
// super-blocks back from LDS in the MFMA operand layout: lane l owns weight row (l & 31) and
// half g2 = l >> 5 of every 32-byte chunk (header + 4 x 16 bytes per super-block), each
// 16-byte piece serving two nibble MFMAs.  D comes back with the x-column results of that
// same weight row, so the scale and min of "its" row are already in the lane's registers.
// With ksplit > 1 the K range is cut into ksplit pieces handled by different workgroups;
// partial sums go to a workspace and the workgroup that arrives last adds them in fixed
// order, so results do not depend on scheduling.
// ---------------------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(8))) _Float16 half8_t;
typedef __attribute__((ext_vector_type(16))) float float16_t;

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

int env_int(const char* name, int dflt) { return dh::tuning_int(name, dflt); }

constexpr int kMaxDepth = 4;
constexpr int kRedSlots = 4;       // tiles a fast wave may run ahead of the slowest one

// LDS shape of the partial sums in the streaming kernel: slots (tiles in flight) and lanes kept.
template <int MT> struct RingShape {
  static constexpr int RS = MT >= 4 ? 2 : kRedSlots;
  static constexpr int LW = MT > 2 ? 64 : 32;
};

struct RingArgs {
  const float* A;        // [M][K]
  const uint8_t* W;      // Q4_K rows
  const uint8_t* W2;     // second matrix (DUAL) or null
  void* C;               // [M][N] f32 or f16
  const float* residual; // [M][N] or null
  int M, N, K, nb;
  int rows_per_tile;     // 1..32
  int depth;             // ring stages per wave, 2..kMaxDepth
  float alpha;
  int c_f16, activation;
  float clamp_max;
  // RMSNorm prologue: A is normalised per row before the product (norm_weight null = off)
  const float* norm_weight;   // [K]
  float norm_eps;
  int norm_weight_offset;     // 1: scale by (1 + w)
};

typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
#define DH_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

// s_waitcnt with only the vector-memory counter set (6 bits, split 4 + 2 in the encoding).
#define DH_WAIT_VM(k) __builtin_amdgcn_s_waitcnt(((k) & 0xF) | (((k) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

// Waits until at most n of this wave's vector-memory loads are outstanding; loads complete in
// issue order, so everything issued before the last n has landed.
__device__ __forceinline__ void wait_vm_at_most(int n) {
  switch (n) {
    case 1: DH_WAIT_VM(1); break;
    case 2: DH_WAIT_VM(2); break;
    case 3: DH_WAIT_VM(3); break;
    case 4: DH_WAIT_VM(4); break;
    case 5: DH_WAIT_VM(5); break;
    case 6: DH_WAIT_VM(6); break;
    case 8: DH_WAIT_VM(8); break;
    case 9: DH_WAIT_VM(9); break;
    case 10: DH_WAIT_VM(10); break;
    case 12: DH_WAIT_VM(12); break;
    case 15: DH_WAIT_VM(15); break;
    default: DH_WAIT_VM(0); break;      // other counts: wait for everything (always safe)
  }
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() would also wait for every
// load in flight (the direct-to-LDS loads count as LDS writers) and drain the ring.
#define DH_LDS_BARRIER() asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory")

// Activation staging.  Work item = (sub-block sb, activation row m) = 32 floats, shared by four
// consecutive lanes: lane grp = idx & 3 of the quad owns elements [8*grp, 8*grp+8), i.e. one
// k-group of the matrix-core fragment.  Zeros past K or M.
template <int MT>
__device__ __forceinline__ void stage_x_load(const float* __restrict__ A, int M, int K, int idx, float (&v)[8]) {
  const int item = idx >> 2, grp = idx & 3;
  const int sb = item / MT, m = item - sb * MT;
  const int k0 = sb * 32 + grp * 8, left = K - k0;
  const float* src = A + (int64_t)m * K + k0;
  if (m < M && left >= 8 && (reinterpret_cast<uintptr_t>(src) & 15) == 0) {
    const float4 t0 = reinterpret_cast<const float4*>(src)[0], t1 = reinterpret_cast<const float4*>(src)[1];
    v[0] = t0.x; v[1] = t0.y; v[2] = t0.z; v[3] = t0.w;
    v[4] = t1.x; v[5] = t1.y; v[6] = t1.z; v[7] = t1.w;
  } else if (m < M && left > 0) {
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float t = src[min(j, left - 1)];
      v[j] = j < left ? t : 0.f;
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; j++) v[j] = 0.f;
  }
}

// RMSNorm weights for the eight k of quarter item idx (1 + w when `offset`); 0 past K.
template <int MT>
__device__ __forceinline__ void stage_norm_weight_load(const float* __restrict__ w, int K, int offset, int idx,
                                                       float (&wn)[8]) {
  const int item = idx >> 2, grp = idx & 3;
  const int k0 = (item / MT) * 32 + grp * 8, left = K - k0;
  const float* src = w + k0;
  if (left >= 8 && (reinterpret_cast<uintptr_t>(src) & 15) == 0) {
    const float4 t0 = reinterpret_cast<const float4*>(src)[0], t1 = reinterpret_cast<const float4*>(src)[1];
    wn[0] = t0.x; wn[1] = t0.y; wn[2] = t0.z; wn[3] = t0.w;
    wn[4] = t1.x; wn[5] = t1.y; wn[6] = t1.z; wn[7] = t1.w;
  } else {
#pragma unroll
    for (int j = 0; j < 8; j++) wn[j] = j < left ? src[j] : 0.f;
  }
  if (offset) {
#pragma unroll
    for (int j = 0; j < 8; j++) wn[j] = j < left ? 1.0f + wn[j] : 0.f;
  }
}

// Sum / max across the four lanes of a quad (DPP quad_perm, no LDS traffic).
__device__ __forceinline__ float quad_xor_f32(float x, int pattern /* 1 or 2 */) {
  const int b = __float_as_int(x);
  const int r = pattern == 1 ? __builtin_amdgcn_update_dpp(b, b, 0xB1, 0xF, 0xF, false)    // [1,0,3,2]
                             : __builtin_amdgcn_update_dpp(b, b, 0x4E, 0xF, 0xF, false);   // [2,3,0,1]
  return __int_as_float(r);
}

// Converts one quarter work item to matrix-core fragments.  Each sub-block gets its own
// power-of-two scale (largest element just inside f16 range): f16 high part, f16 residual,
// the plain sum (min term) and 2^24 / scale per (sb, m).  All four lanes of the quad must call.
template <int MT>
__device__ __forceinline__ void stage_x_store(int idx, const float (&v)[8], _Float16* xf, float2* sxi) {
  constexpr int XC = 2 * MT;
  const int item = idx >> 2, grp = idx & 3;
  const int sb = item / MT, m = item - sb * MT;
  float s = 0.f, mx = 0.f;
#pragma unroll
  for (int j = 0; j < 8; j++) { s += v[j]; mx = fmaxf(mx, fabsf(v[j])); }
  s += quad_xor_f32(s, 1);
  mx = fmaxf(mx, quad_xor_f32(mx, 1));
  s += quad_xor_f32(s, 2);
  mx = fmaxf(mx, quad_xor_f32(mx, 2));
  int e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 127;
  e = max(-100, min(100, e));
  if (mx == 0.f) e = 14;
  const float sf = __uint_as_float((uint32_t)(127 + 14 - e) << 23);          // 2^(14-e)
  if (grp == 0) sxi[item] = make_float2(s, __uint_as_float((uint32_t)(127 + 24 - 14 + e) << 23));   // 2^24 / sf
  half8_t hi, lo;
#pragma unroll
  for (int slot = 0; slot < 8; slot++) {
    // slot order inside a k-group follows the masked dwords: (b0,b2) (b1,b3) (b4,b6) (b5,b7)
    const int o = (slot & 4) | ((slot & 1) << 1) | ((slot >> 1) & 1);
    const float xsc = v[o] * sf;
    const _Float16 h = (_Float16)xsc;
    hi[slot] = h;
    lo[slot] = (_Float16)(xsc - (float)h);
  }
  *reinterpret_cast<half8_t*>(xf + (sb * XC + 2 * m) * 32 + grp * 8) = hi;
  *reinterpret_cast<half8_t*>(xf + (sb * XC + 2 * m + 1) * 32 + grp * 8) = lo;
}

// Where a wave is in its list of work units (tile, matrix, super-block).
struct UnitCursor {
  int tl, mat, i;        // tile ordinal of this workgroup, matrix, block ordinal of this wave
};

// GEMV on the matrix cores with the weights streamed HBM -> LDS by the load unit itself
// (global_load_lds_dwordx4: no vector registers, no vector-ALU work on the way).
//
// A workgroup of WAVES (8 or 16) waves owns tiles of R <= 32 consecutive weight rows (R chosen by the host
// so that the tile count is a multiple of the number of compute units).  Inside a tile, wave
// w takes super-blocks w, w+WAVES, ...: one work unit = R rows x 1 super-block = R*144 bytes,
// fetched by up to five 16-byte-per-lane load instructions (9 lanes per row) into one stage of
// the wave's private ring in LDS, rows 144 bytes apart exactly as in memory.  Each wave keeps
// `depth` units in flight and synchronises with nobody while it streams: it waits on its own
// load counter, reads the stage back in the MFMA operand layout, re-issues the stage for the
// unit `depth` ahead and only then does the arithmetic.  Waves meet once per tile, to add
// their K slices.  The activation fragments live in a separate, statically declared LDS
// array: the compiler then knows that reading them cannot touch the bytes the load unit is
// writing and does not wait for the loads in flight.
template <int MT, bool DUAL, int XBYTES, int WAVES>
__global__ __launch_bounds__(64 * WAVES, WAVES / 4) void q4k_gemv_ring_kernel(const RingArgs a) {
  constexpr int NTHR = 64 * WAVES;
  constexpr int XC = 2 * MT, NO = MfmaShape<MT>::NI / 2, NMAT = DUAL ? 2 : 1;
  constexpr int RS = RingShape<MT>::RS, LW = RingShape<MT>::LW;
  __shared__ __align__(16) unsigned char xs[XBYTES];        // x fragments | zero row | (sum, 1/scale)
  // K-slice partial sums per tile slot: entry k of lane l belongs to activation row
  // (k & 1) + 2 * (l >> 5) + 4 * (k >> 1); up to two rows live in lanes 0..31 alone
  __shared__ float red[RS][WAVES][NMAT][NO][LW];
  __shared__ unsigned done[RS];                              // waves that delivered their partials
  __shared__ float norm_ss[WAVES][MT];
  extern __shared__ __align__(16) unsigned char ring[];     // [WAVES][depth][R*144]

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);     // provably wave-uniform
  const int g2 = lane >> 5, xcol = lane & 31;
  const int R = a.rows_per_tile, D = a.depth;
  const int nsub = a.nb * 8;
  _Float16* xf = reinterpret_cast<_Float16*>(xs);                       // [nsub][XC][32]
  _Float16* xzero = xf + (size_t)nsub * XC * 32;                        // 32 zero halves
  float2* sxi = reinterpret_cast<float2*>(xzero + 32);                  // [nsub][MT]
  const int64_t row_bytes = (int64_t)a.nb * kBlockBytes;
  const int ntiles = (a.N + R - 1) / R;
  const int ntl = (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;   // my tiles
  const int bpw = (a.nb - wave + WAVES - 1) / WAVES;                    // my blocks per tile
  const int stage_bytes = R * kBlockBytes;
  const int nlw = (9 * R + 63) >> 6;                                    // load instructions per unit
  unsigned char* my_ring = ring + (size_t)wave * D * stage_bytes;

  // chunk q = t*64 + lane of a unit: row q/9, 16-byte piece q%9 of the row's super-block
  uint32_t goff[5];
#pragma unroll
  for (int t = 0; t < 5; t++) {
    const int q = t * 64 + lane, r = q / 9;
    goff[t] = q < 9 * R ? (uint32_t)(r * row_bytes + (q - r * 9) * 16) : 0xFFFFFFFFu;
  }

  UnitCursor ic = {0, 0, 0};
  int issue_stage = 0, issued = 0;
  // Puts the loads of the next unit in flight (if there is one) into ring stage issue_stage.
#define DH_ISSUE_NEXT()                                                                           \
  do {                                                                                            \
    if (ic.tl < ntl && bpw > 0) {                                                                 \
      const int tile_ = blockIdx.x + ic.tl * gridDim.x;                                           \
      const uint8_t* base_ = ((DUAL && ic.mat) ? a.W2 : a.W) + (int64_t)tile_ * R * row_bytes +   \
                             (int64_t)(wave + WAVES * ic.i) * kBlockBytes;                        \
      unsigned char* st_ = my_ring + issue_stage * stage_bytes;                                   \
      const int rows_left_ = a.N - tile_ * R;                                                     \
      if (rows_left_ >= R) {                                                                      \
        _Pragma("unroll") for (int t = 0; t < 5; t++) {                                           \
          if (goff[t] != 0xFFFFFFFFu)                                                             \
            __builtin_amdgcn_global_load_lds(base_ + goff[t], DH_LDS_PTR(st_ + t * 1024), 16, 0, 0); \
        }                                                                                         \
      } else {                                                                                    \
        _Pragma("unroll") for (int t = 0; t < 5; t++) {                                           \
          const int q_ = t * 64 + lane, r_ = q_ / 9;                                              \
          const int64_t o_ = (int64_t)min(r_, rows_left_ - 1) * row_bytes + (q_ - r_ * 9) * 16;   \
          if (goff[t] != 0xFFFFFFFFu)                                                             \
            __builtin_amdgcn_global_load_lds(base_ + o_, DH_LDS_PTR(st_ + t * 1024), 16, 0, 0);   \
        }                                                                                         \
      }                                                                                           \
      issued++;                                                                                   \
      issue_stage = issue_stage + 1 == D ? 0 : issue_stage + 1;                                   \
      if (++ic.i == bpw) {                                                                        \
        ic.i = 0;                                                                                 \
        if (++ic.mat == NMAT) { ic.mat = 0; ic.tl++; }                                            \
      }                                                                                           \
    }                                                                                             \
  } while (0)

  // ---- stage the activations in LDS.  Work item = (sub-block sb, activation row m): 32 floats.
  // The first item's loads go out before the ring loads (loads complete in order), its
  // conversion runs while the ring fills.
  bool early_ring;
  {
    // Everything this thread needs from memory for its first quarter item is loaded before the
    // ring starts: loads complete in order, so a wait for a later load would also wait for the
    // ring loads in front of it.
    const int total = 4 * MT * nsub;
    const bool norm = a.norm_weight != nullptr;
    early_ring = wave * 64 >= total || total >= NTHR;
    float v0[8], wn0[8];
    if (tid < total) stage_x_load<MT>(a.A, a.M, a.K, tid, v0);
    float ss = 0.f;
    if (norm) {
      if (tid < total) stage_norm_weight_load<MT>(a.norm_weight, a.K, a.norm_weight_offset, tid, wn0);
#pragma unroll 1
      for (int idx = tid + NTHR; idx < total; idx += NTHR) {   // rows longer than one pass
        float t[8];
        stage_x_load<MT>(a.A, a.M, a.K, idx, t);
#pragma unroll
        for (int j = 0; j < 8; j++) ss = fmaf(t[j], t[j], ss);
      }
    }
    // Waves without staging work start their ring at once.  Waves that stage do so too when
    // every wave stages; otherwise they convert first and start their ring after the barrier,
    // so the others can begin computing as early as possible.  (Putting every wave's whole ring
    // in flight right behind the activation loads was measured slower, 9.3 vs 7.7 us on the
    // 6144 x 4096 product: the activation loads of the staging waves then queue behind the
    // other waves' weight loads in the memory system, and nothing can be consumed before the
    // activations are staged.  Starting the staging waves' rings after their activations have
    // arrived but before they convert them gains nothing either: 8.7 vs 7.4 us there, 20.7 vs
    // 20.6 us on the fused gate/up product.  Nor does handing units to whichever wave frees a
    // ring stage first (a counter in LDS, per-unit partial sums added in super-block order by
    // the wave that completes a tile): waves of a workgroup end up to 5 us apart under fixed
    // ownership, but the workgroup as a whole is limited by what the memory system delivers,
    // 17.2 vs 17.7 us for gate/up and 13.8 vs 13.0 us for the down projection, no change per step.
    // Nor letting the staging waves only stage and the other half own the whole weight stream:
    // 8.4 vs 7.5 us on the 6144 x 4096 product.)
    DH_WAIT_VM(0);
    if (norm && tid < total) {
#pragma unroll
      for (int j = 0; j < 8; j++) ss = fmaf(v0[j], v0[j], ss);
    }
    // RMSNorm prologue: the row's 1/rms is one factor per activation row, so it is applied to
    // the outputs at the tile end instead of to the activations here; the conversion below
    // does not have to wait for the sum of squares, only the tile ends do.  Per wave: sum of
    // squares of activation row m = (tid >> 2) % MT (lanes of a quad share a row, the lane
    // bits above select among MT rows).
    if (norm) {
      ss += quad_xor_f32(ss, 1);
      ss += quad_xor_f32(ss, 2);
      if (MT <= 1) ss += __shfl_xor(ss, 4);
      if (MT <= 2) ss += __shfl_xor(ss, 8);
      if (MT <= 4) ss += __shfl_xor(ss, 16);
      ss += __shfl_xor(ss, 32);
      if ((lane & 3) == 0 && (lane >> 2) < MT) norm_ss[wave][lane >> 2] = ss;
    }
    // Two places where ring stages are put in flight (a loop, so that the code exists once):
    // early waves before the conversion, late waves after it.
#pragma unroll 1
    for (int phase = 0; phase < 2; phase++) {
    const int nstart = early_ring == (phase == 0) ? D : 0;
    for (int d = 0; d < nstart; d++) DH_ISSUE_NEXT();
    if (phase != 0) continue;
#pragma unroll 1
    for (int idx = tid; idx < total; idx += NTHR) {
      float t[8], wn[8];
      if (idx == tid) {
#pragma unroll
        for (int j = 0; j < 8; j++) { t[j] = v0[j]; wn[j] = wn0[j]; }
      } else {
        stage_x_load<MT>(a.A, a.M, a.K, idx, t);
        if (norm) stage_norm_weight_load<MT>(a.norm_weight, a.K, a.norm_weight_offset, idx, wn);
      }
      if (norm) {
#pragma unroll
        for (int j = 0; j < 8; j++) t[j] = t[j] * wn[j];
      }
      stage_x_store<MT>(idx, t, xf, sxi);
    }
    if (tid < 16) reinterpret_cast<uint32_t*>(xzero)[tid] = 0u;
    if (tid < RS) done[tid] = 0u;
    DH_LDS_BARRIER();
    }
  }

  const _Float16* xfl = xcol < XC ? xf + xcol * 32 + g2 * 16 : xzero;
  const int xf_stride = xcol < XC ? XC * 32 : 0;
  // LDS byte address of this lane's header inside stage 0: rows past R re-read the last row
  const uint32_t lane_lds =
      (uint32_t)(uintptr_t)DH_LDS_PTR(my_ring) + (uint32_t)min(lane & 31, R - 1) * kBlockBytes;

  int consumed = 0, cstage = 0;
#pragma unroll 1
  for (int tl = 0; tl < ntl; tl++) {
    const int tile = blockIdx.x + tl * gridDim.x;
    const int slot = tl % RS;
#pragma unroll 1
    for (int mat = 0; mat < NMAT; mat++) {
      float acc[NO];
#pragma unroll
      for (int k = 0; k < NO; k++) acc[k] = 0.f;
#pragma unroll 1
      for (int i = 0; i < bpw; i++) {
        // units issued after this one: each put nlw load instructions behind ours
        wait_vm_at_most((issued - consumed - 1) * nlw);
            const uint32_t hp = lane_lds + cstage * stage_bytes, qp = hp + 16 + 16 * g2;
        u32x4 h, q0, q1, q2, q3;
        asm volatile(
            "ds_read_b128 %0, %5\n\t"
            "ds_read_b128 %1, %6\n\t"
            "ds_read_b128 %2, %6 offset:32\n\t"
            "ds_read_b128 %3, %6 offset:64\n\t"
            "ds_read_b128 %4, %6 offset:96\n\t"
            "s_waitcnt lgkmcnt(0)"
            : "=&v"(h), "=&v"(q0), "=&v"(q1), "=&v"(q2), "=&v"(q3)
            : "v"(hp), "v"(qp)
            : "memory");
        consumed++;
        cstage = cstage + 1 == D ? 0 : cstage + 1;
            DH_ISSUE_NEXT();            // the stage just read is free again
            WBlock w;
        w.hdr = make_uint4(h.x, h.y, h.z, h.w);
        w.q[0] = make_uint4(q0.x, q0.y, q0.z, q0.w);
        w.q[1] = make_uint4(q1.x, q1.y, q1.z, q1.w);
        w.q[2] = make_uint4(q2.x, q2.y, q2.z, q2.w);
        w.q[3] = make_uint4(q3.x, q3.y, q3.z, q3.w);
        mfma_block<MT>(w, xfl, xf_stride, sxi, (wave + WAVES * i) * 8, g2, acc);
          }
      if (lane < LW) {
#pragma unroll
        for (int k = 0; k < NO; k++) red[slot][wave][mat][k][lane] = acc[k];
      }
    }
    // ---- tile end.  Nobody waits: each wave reports its partial sums and moves on; the wave
    // that arrives last adds the K slices in wave order and writes the outputs.  LDS executes a
    // wave's operations in order, so every earlier arrival's partials are in place by then.
    // (The counter is bumped with a hand-written LDS atomic: the compiler would put a wait for
    // all loads in flight in front of its own, because the ring loads write LDS too.)
    unsigned arrived = 0;
    if (lane == 0) {
      const uint32_t cnt_addr = (uint32_t)(uintptr_t)DH_LDS_PTR(&done[slot]);
      asm volatile("ds_add_rtn_u32 %0, %1, %2\n\ts_waitcnt lgkmcnt(0)"
                   : "=&v"(arrived) : "v"(cnt_addr), "v"(1u) : "memory");
    }
    arrived = __builtin_amdgcn_readfirstlane(arrived);
    asm volatile("" ::: "memory");
    if (arrived == WAVES - 1) {
      const int r = lane & 31;
      const int64_t row = (int64_t)tile * R + r;
#pragma unroll 1
      for (int m = lane >> 5; m < MT; m += 2) {
      if (m < a.M && r < R && row < a.N) {
        // activation row m sits in entry (m & 1) + 2 * (m >> 2) of lane half (m >> 1) & 1
        const int k = (m & 1) + 2 * (m >> 2), col = (MT > 2 ? 32 * ((m >> 1) & 1) : 0) + r;
        float sg = 0.f, su = 0.f;
#pragma unroll
        for (int w = 0; w < WAVES; w++) {
          sg += red[slot][w][0][k][col];
          if (DUAL) su += red[slot][w][NMAT - 1][k][col];
        }
        if (a.norm_weight) {
          float tot = 0.f;
#pragma unroll
          for (int w = 0; w < WAVES; w++) tot += norm_ss[w][m];
          const float inv = 1.0f / sqrtf(tot / (float)a.K + a.norm_eps);
          sg *= inv;
          su *= inv;
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
      }
      if (lane == 0) done[slot] = 0u;
    }
    // more tiles than slots: keep the waves within one tile of each other instead
    if (ntl > RS) DH_LDS_BARRIER();
  }
#undef DH_ISSUE_NEXT
}

constexpr size_t kRingMaxLds = 160 * 1024;

size_t ring_x_bytes(int mt, int nb) { return (size_t)nb * 8 * mt * (2 * 32 * 2 + 8) + 64; }

template <int MT, bool DUAL, int XBYTES, int WAVES>
int launch_ring_cfg(RingArgs a, const char* op, bool may_shorten_tiles) {
  constexpr int NO = MfmaShape<MT>::NI / 2, NMAT = DUAL ? 2 : 1;
  const size_t fixed = XBYTES + sizeof(float) * RingShape<MT>::RS * WAVES * NMAT * NO * RingShape<MT>::LW + 512;
  auto kern = q4k_gemv_ring_kernel<MT, DUAL, XBYTES, WAVES>;
  static const int env_rows = env_int("DH_GEMV_ROWS", 0), env_depth = env_int("DH_GEMV_DEPTH", 0);
  // rows per tile: the smallest count that covers N with a whole number of tiles per compute unit
  const int ncu = dh::num_cus();
  const int per_cu = (int)dh::ceil_div(a.N, (int64_t)ncu * 32);
  int rows = (int)dh::ceil_div(a.N, (int64_t)ncu * per_cu);
  rows = std::max(4, std::min(32, rows));
  if (env_rows > 0) rows = std::min(32, env_rows);
  // a two-stage ring must fit beside the activations; shorter tiles (uneven tile counts per
  // compute unit) only when nothing else is left
  while (may_shorten_tiles && rows > 8 && fixed + (size_t)WAVES * 2 * rows * kBlockBytes > kRingMaxLds) rows -= 4;
  int depth = kMaxDepth;
  while (depth > 2 && fixed + (size_t)WAVES * depth * rows * kBlockBytes > kRingMaxLds) depth--;
  if (env_depth > 0) depth = std::max(2, std::min(kMaxDepth, env_depth));
  const size_t dyn = (size_t)WAVES * depth * rows * kBlockBytes;
  if (fixed + dyn > kRingMaxLds) return -1;
  a.rows_per_tile = rows;
  a.depth = depth;
  const int64_t ntiles = dh::ceil_div(a.N, rows);
  const int grid = (int)std::min<int64_t>(ntiles, ncu);
  if (dh::plan_note(DH_PLAN_GEMV_RING)) return 0;
  static bool attr_set = false;   // once per instantiation: the call costs microseconds
  if (!attr_set) {
    DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize,
                                         (int)(kRingMaxLds - fixed)));
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(grid), dim3(64 * WAVES), dyn, dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  return 0;
}

// Returns -1 when the activations of MT rows do not fit any of the kernel's static LDS arrays.
// MT <= 2 run with 16 waves per workgroup where the ring still fits (more loads in flight);
// four and eight activation rows need the LDS for their fragments and run with 8.
template <int MT, bool DUAL>
int launch_ring(const RingArgs& a, const char* op) {
  const size_t xb = ring_x_bytes(MT, a.nb);
  static const int env_waves = env_int("DH_GEMV_WAVES", 16);
  if constexpr (MT <= 2) {
    if (env_waves == 16) {
      int rc = -1;
      if (xb <= 20 * 1024) rc = launch_ring_cfg<MT, DUAL, 20 * 1024, 16>(a, op, false);
      else if (xb <= 40 * 1024) rc = launch_ring_cfg<MT, DUAL, 40 * 1024, 16>(a, op, false);
      else if (xb <= 56 * 1024) rc = launch_ring_cfg<MT, DUAL, 56 * 1024, 16>(a, op, false);
      if (rc >= 0) return rc;
    }
    if (xb <= 20 * 1024) return launch_ring_cfg<MT, DUAL, 20 * 1024, 8>(a, op, true);
    if (xb <= 40 * 1024) return launch_ring_cfg<MT, DUAL, 40 * 1024, 8>(a, op, true);
    if (xb <= 56 * 1024) return launch_ring_cfg<MT, DUAL, 56 * 1024, 8>(a, op, true);
    if constexpr (MT == 2) {
      if (xb <= 104 * 1024) return launch_ring_cfg<MT, DUAL, 104 * 1024, 8>(a, op, true);
    }
  } else {
    if (xb <= 40 * 1024) return launch_ring_cfg<MT, DUAL, 40 * 1024, 8>(a, op, true);
    if (xb <= 72 * 1024) return launch_ring_cfg<MT, DUAL, 72 * 1024, 8>(a, op, true);
    if (xb <= 104 * 1024) return launch_ring_cfg<MT, DUAL, 104 * 1024, 8>(a, op, true);
  }
  return -1;
}

template <bool DUAL>
int launch_ring_mt(int mt, const RingArgs& a, const char* op) {
  switch (mt) {
    case 8: return launch_ring<8, DUAL>(a, op);
    case 4: return launch_ring<4, DUAL>(a, op);
    case 2: return launch_ring<2, DUAL>(a, op);
    default: return launch_ring<1, DUAL>(a, op);
  }
}

// M <= 8 activation rows in as few passes over the weights as the LDS allows: 8, 4, 2 or 1 rows
// per pass (a pass with fewer rows than its kernel holds zero-fills the rest).
template <bool DUAL>
int dispatch_ring(const RingArgs& a, const char* op) {
  static const int env_mt = env_int("DH_GEMV_MT", 8);
  const size_t c_elem = a.c_f16 ? 2 : 4;
  // candidates in order of passes needed, smaller kernels first among equals
  int order[4] = {1, 2, 4, 8}, n = 0;
  for (int mt : {1, 2, 4, 8}) n += mt <= env_mt;
  std::stable_sort(order, order + n, [&](int x, int y) { return (a.M + x - 1) / x < (a.M + y - 1) / y; });
  for (int c = 0; c < n; c++) {
    const int mt = order[c];
    int rc = 0;
    for (int m0 = 0; m0 < a.M; m0 += mt) {
      RingArgs b = a;
      b.M = std::min(mt, a.M - m0);
      b.A = a.A + (int64_t)m0 * a.K;
      b.C = static_cast<char*>(a.C) + (int64_t)m0 * a.N * c_elem;
      b.residual = a.residual ? a.residual + (int64_t)m0 * a.N : nullptr;
      rc = launch_ring_mt<DUAL>(mt, b, op);
      if (rc) break;                 // -1 on the first pass: this row count does not fit
    }
    if (rc >= 0) return rc;
  }
  return -1;
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
  if (dh::plan_note(DH_PLAN_GEMV_LDS)) return 0;
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

// Kernel family used for M <= 8: 0 = matrix-core GEMV (default), 2 = LDS-staged vector GEMV.
// DH_GEMV_PATH overrides (for measurements).
int gemv_path() {
  static const int path = env_int("DH_GEMV_PATH", 0);
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

// Shared body of dh_q4k_matmul and dh_q4k_matmul_rmsnorm.
static int q4k_matmul_impl(const char* op, const void* d_A, int a_dtype, const float* d_norm_weight,
                           float eps, int weight_offset, bool normed, const void* d_W, void* d_C,
                           int c_dtype, int M, int N, int K, float alpha, const void* d_residual) {
  DH_REQUIRE_INIT(op);
  if (M <= 0 || N <= 0 || K <= 0)
    return dh::fail(1, "[%s] Dimensions must be positive: M=%d, N=%d, K=%d", op, M, N, K);
  if (!d_A || !d_W || !d_C) return dh::fail(1, "[%s] null pointer", op);
  if (a_dtype != DH_F32) return dh::fail(1, "[%s] activations must be f32 or f16 (a_dtype=%d)", op, a_dtype);
  if (c_dtype != DH_F32 && c_dtype != DH_F16)
    return dh::fail(1, "[%s] output dtype must be f32 or f16 (c_dtype=%d)", op, c_dtype);
  if (reinterpret_cast<uintptr_t>(d_W) & 15)
    return dh::fail(1, "[%s] weight pointer must be 16-byte aligned", op);
  if (normed && !d_norm_weight) return dh::fail(1, "[%s] norm weight pointer is null", op);
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
  if ((path == 0 || normed) && M <= 2) {
    const int rc = dh::q4k_gemv_i8(op, a.A, a.W, nullptr, d_C, a.c_f16, a.residual, M, N, K, alpha, 0, 0.f,
                                   normed ? d_norm_weight : nullptr, eps, weight_offset);
    if (rc >= 0) return rc;
  }
  if ((path == 0 || normed) && M < 16) {
    // below the GEMM's batch size: passes of up to 8 rows, each one sweep over the weights
    int rc = 0;
    for (int m0 = 0; m0 < M && rc == 0; m0 += 8) {
      rc = dh::q4k_gemv_rows(op, a.A + (int64_t)m0 * K, a.W, nullptr, static_cast<char*>(d_C) + (int64_t)m0 * N * (a.c_f16 ? 2 : 4),
                             a.c_f16, a.residual ? a.residual + (int64_t)m0 * N : nullptr, std::min(8, M - m0), N, K, alpha, 0,
                             0.f, normed ? d_norm_weight : nullptr, eps, weight_offset);
      if (rc < 0 && m0 > 0) return dh::fail(2, "[%s] internal: GEMV pass %d did not launch after pass 0 did", op, m0 / 8);
    }
    if (rc >= 0) return rc;
  }
  if ((path == 0 || normed) && M < 16) {
    // below the GEMM's batch size: passes of up to 8 rows through the streaming GEMV
    int rc = 0;
    for (int m0 = 0; m0 < M && rc == 0; m0 += 8) {
      RingArgs g{};
      g.A = a.A + (int64_t)m0 * K; g.W = a.W; g.W2 = nullptr;
      g.C = static_cast<char*>(d_C) + (int64_t)m0 * N * (a.c_f16 ? 2 : 4);
      g.residual = a.residual ? a.residual + (int64_t)m0 * N : nullptr;
      g.M = std::min(8, M - m0); g.N = N; g.K = K; g.nb = a.nb; g.alpha = alpha; g.c_f16 = a.c_f16;
      g.norm_weight = normed ? d_norm_weight : nullptr;
      g.norm_eps = eps; g.norm_weight_offset = weight_offset;
      rc = dispatch_ring<false>(g, op);
      if (rc < 0 && m0 > 0) return dh::fail(2, "[%s] internal: GEMV pass %d did not fit after pass 0 did", op, m0 / 8);
    }
    if (rc >= 0) return rc;
  }
  if (path != 2 && dh::q4k_gemm_serves(M, K, d_A))
    return dh::q4k_gemm(op, a.A, a.W, d_C, a.c_f16, M, N, K, alpha, a.residual, normed ? d_norm_weight : nullptr, eps,
                        weight_offset);
  if (normed)
    return dh::fail(1, "[%s] the RMSNorm prologue serves any K up to 15 rows (K <= 14336 for matrices of more than "
                    "61440 rows) and K <= 16384 from 16 rows on (M=%d, K=%d); run dh_rmsnorm and dh_q4k_matmul instead", op,
                    M, K);
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

int dh_q4k_matmul(const void* d_A, int a_dtype, const void* d_W, void* d_C, int c_dtype, int M,
                  int N, int K, float alpha, const void* d_residual) {
  if (a_dtype == DH_F16) {
    // f16 activations: widened (exactly) into the library's f32 staging rows, as many rows per
    // pass as the staging holds; the product accumulates in f32 like the f32-activation path
    const char* op = "dh_q4k_matmul";
    DH_REQUIRE_INIT(op);
    if (M <= 0 || N <= 0 || K <= 0)
      return dh::fail(1, "[%s] Dimensions must be positive: M=%d, N=%d, K=%d", op, M, N, K);
    if (!d_A || !d_W || !d_C) return dh::fail(1, "[%s] null pointer", op);
    if (c_dtype != DH_F32 && c_dtype != DH_F16)
      return dh::fail(1, "[%s] output dtype must be f32 or f16 (c_dtype=%d)", op, c_dtype);
    if (M < 16 && gemv_path() == 0) {
      // below the GEMM's batch size the GEMV kernels load the f16 rows themselves (K a multiple of 4 and
      // 8-byte aligned rows; otherwise they decline and the rows are widened first)
      if (reinterpret_cast<uintptr_t>(d_W) & 15)
        return dh::fail(1, "[%s] weight pointer must be 16-byte aligned", op);
      const uint16_t* A16 = static_cast<const uint16_t*>(d_A);
      const float* res = static_cast<const float*>(d_residual);
      const int c_f16 = c_dtype == DH_F16;
      int rc = -1;
      if (M <= 2)
        rc = dh::q4k_gemv_i8(op, reinterpret_cast<const float*>(A16), static_cast<const uint8_t*>(d_W), nullptr, d_C, c_f16,
                             res, M, N, K, alpha, 0, 0.f, nullptr, 0.f, 0, 1);
      if (rc < 0) {
        rc = 0;
        for (int m0 = 0; m0 < M && rc == 0; m0 += 8) {
          rc = dh::q4k_gemv_rows(op, reinterpret_cast<const float*>(A16 + (int64_t)m0 * K), static_cast<const uint8_t*>(d_W),
                                 nullptr, static_cast<char*>(d_C) + (int64_t)m0 * N * (c_f16 ? 2 : 4), c_f16,
                                 res ? res + (int64_t)m0 * N : nullptr, std::min(8, M - m0), N, K, alpha, 0, 0.f, nullptr, 0.f,
                                 0, 1);
          if (rc < 0 && m0 > 0) return dh::fail(2, "[%s] internal: GEMV pass %d did not launch after pass 0 did", op, m0 / 8);
        }
      }
      if (rc >= 0) return rc;
    }
    size_t bytes = 0;
    float* wide = dh::widened_activations(&bytes);
    int64_t rows_per_pass = (int64_t)(bytes / sizeof(float)) / K;
    if (rows_per_pass >= 16) rows_per_pass &= ~(int64_t)15;
    if (rows_per_pass < 1)
      return dh::fail(1, "[%s] K=%d is too long for f16 activations (at most %zu)", op, K, bytes / sizeof(float));
    const size_t c_elem = c_dtype == DH_F16 ? 2 : 4;
    for (int64_t m0 = 0; m0 < M; m0 += rows_per_pass) {
      const int rows = (int)std::min<int64_t>(rows_per_pass, M - m0);
      int rc = dh_cast_f16_to_f32(static_cast<const uint16_t*>(d_A) + m0 * K, wide, (int64_t)rows * K);
      if (rc) return rc;
      rc = q4k_matmul_impl(op, wide, DH_F32, nullptr, 0.f, 0, false, d_W, static_cast<char*>(d_C) + m0 * N * c_elem,
                           c_dtype, rows, N, K, alpha,
                           d_residual ? static_cast<const float*>(d_residual) + m0 * N : nullptr);
      if (rc) return rc;
    }
    return 0;
  }
  return q4k_matmul_impl("dh_q4k_matmul", d_A, a_dtype, nullptr, 0.f, 0, false, d_W, d_C, c_dtype, M, N, K,
                         alpha, d_residual);
}

int dh_q4k_matmul_rmsnorm(const float* d_A, const float* d_norm_weight, float eps, int weight_offset,
                          const void* d_W, void* d_C, int c_dtype, int M, int N, int K, float alpha,
                          const void* d_residual) {
  return q4k_matmul_impl("dh_q4k_matmul_rmsnorm", d_A, DH_F32, d_norm_weight, eps, weight_offset, true, d_W,
                         d_C, c_dtype, M, N, K, alpha, d_residual);
}

// Shared body of dh_q4k_ffn_gate_up and dh_q4k_ffn_gate_up_rmsnorm.
static int q4k_ffn_impl(const char* op, const float* d_x, const float* d_norm_weight, float eps,
                        int weight_offset, bool normed, const void* d_Wgate, const void* d_Wup,
                        float* d_out, int M, int hidden, int inter, int activation, float alpha,
                        float swiglu_limit) {
  DH_REQUIRE_INIT(op);
  if (M <= 0 || hidden <= 0 || inter <= 0)
    return dh::fail(1, "[%s] Dimensions must be positive: M=%d, hidden=%d, inter=%d", op, M, hidden, inter);
  if (!d_x || !d_Wgate || !d_Wup || !d_out) return dh::fail(1, "[%s] null pointer", op);
  if (activation != DH_ACT_SILU && activation != DH_ACT_GELU)
    return dh::fail(1, "[%s] unknown activation %d", op, activation);
  if ((reinterpret_cast<uintptr_t>(d_Wgate) | reinterpret_cast<uintptr_t>(d_Wup)) & 15)
    return dh::fail(1, "[%s] weight pointers must be 16-byte aligned", op);
  if (normed && !d_norm_weight) return dh::fail(1, "[%s] norm weight pointer is null", op);
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
  if ((path == 0 || normed) && M <= 2) {
    const int rc = dh::q4k_gemv_i8(op, d_x, a.W, a.W2, d_out, 0, nullptr, M, inter, hidden, alpha, activation,
                                   swiglu_limit, normed ? d_norm_weight : nullptr, eps, weight_offset);
    if (rc >= 0) return rc;
  }
  if ((path == 0 || normed) && M < 16) {
    int rc = 0;
    for (int m0 = 0; m0 < M && rc == 0; m0 += 8) {
      rc = dh::q4k_gemv_rows(op, d_x + (int64_t)m0 * hidden, a.W, a.W2, d_out + (int64_t)m0 * inter, 0, nullptr,
                             std::min(8, M - m0), inter, hidden, alpha, activation, swiglu_limit,
                             normed ? d_norm_weight : nullptr, eps, weight_offset);
      if (rc < 0 && m0 > 0) return dh::fail(2, "[%s] internal: GEMV pass %d did not launch after pass 0 did", op, m0 / 8);
    }
    if (rc >= 0) return rc;
  }
  if ((path == 0 || normed) && M < 16) {
    int rc = 0;
    for (int m0 = 0; m0 < M && rc == 0; m0 += 8) {
      RingArgs g{};
      g.A = d_x + (int64_t)m0 * hidden; g.W = a.W; g.W2 = a.W2; g.C = d_out + (int64_t)m0 * inter; g.residual = nullptr;
      g.M = std::min(8, M - m0); g.N = inter; g.K = hidden; g.nb = a.nb; g.alpha = alpha; g.c_f16 = 0;
      g.activation = activation; g.clamp_max = swiglu_limit;
      g.norm_weight = normed ? d_norm_weight : nullptr;
      g.norm_eps = eps; g.norm_weight_offset = weight_offset;
      rc = dispatch_ring<true>(g, op);
      if (rc < 0 && m0 > 0) return dh::fail(2, "[%s] internal: GEMV pass %d did not fit after pass 0 did", op, m0 / 8);
    }
    if (rc >= 0) return rc;
  }
  if (path != 2 && dh::q4k_gemm_serves(M, hidden, d_x))
    return dh::q4k_gemm_gate_up(op, d_x, a.W, a.W2, d_out, M, hidden, inter, activation, alpha, swiglu_limit,
                                normed ? d_norm_weight : nullptr, eps, weight_offset);
  if (normed)
    return dh::fail(1, "[%s] the RMSNorm prologue serves any hidden size up to 15 rows (hidden <= 14336 for more than "
                    "30720 intermediate rows) and hidden <= 16384 from 16 rows on (M=%d, hidden=%d); run dh_rmsnorm and "
                    "dh_q4k_ffn_gate_up instead", op, M, hidden);
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

int dh_q4k_matmul_plan(int M, int N, int K, int normed, int dual, int num_cus) {
  const char* op = "dh_q4k_matmul_plan";
  if (num_cus <= 0) num_cus = dh::ready() ? dh::num_cus() : 256;
  dh::plan_begin(num_cus);
  // the dispatchers look at shapes, alignment and null-ness only: stand-in addresses, never touched
  const float* x = reinterpret_cast<const float*>(uintptr_t{1} << 20);
  const void* w = reinterpret_cast<const void*>(uintptr_t{2} << 20);
  float* c = reinterpret_cast<float*>(uintptr_t{3} << 20);
  int rc;
  if (dual)
    rc = q4k_ffn_impl(op, x, normed ? x : nullptr, 1e-6f, 0, normed != 0, w, w, c, M, K, N, DH_ACT_SILU, 1.0f, 0.0f);
  else
    rc = q4k_matmul_impl(op, x, DH_F32, normed ? x : nullptr, 1e-6f, 0, normed != 0, w, c, DH_F32, M, N, K, 1.0f, nullptr);
  const int family = dh::plan_end();
  return rc == 0 ? family : 0;
}

int dh_q4k_gemv_layout(int M, int N, int K, int normed, int dual, int num_cus, int64_t* out12) {
  if (!out12) return 0;
  const int family = dh_q4k_matmul_plan(M, N, K, normed, dual, num_cus);
  const int64_t* rec = dh::plan_layout_record();
  for (int i = 0; i < 12; i++) out12[i] = rec[i];
  return family;
}

int dh_q4k_ffn_gate_up(const float* d_x, const void* d_Wgate, const void* d_Wup, float* d_out, int M,
                       int hidden, int inter, int activation, float alpha, float swiglu_limit) {
  return q4k_ffn_impl("dh_q4k_ffn_gate_up", d_x, nullptr, 0.f, 0, false, d_Wgate, d_Wup, d_out, M, hidden,
                      inter, activation, alpha, swiglu_limit);
}

int dh_q4k_ffn_gate_up_rmsnorm(const float* d_x, const float* d_norm_weight, float eps, int weight_offset,
                               const void* d_Wgate, const void* d_Wup, float* d_out, int M, int hidden,
                               int inter, int activation, float alpha, float swiglu_limit) {
  return q4k_ffn_impl("dh_q4k_ffn_gate_up_rmsnorm", d_x, d_norm_weight, eps, weight_offset, true, d_Wgate,
                      d_Wup, d_out, M, hidden, inter, activation, alpha, swiglu_limit);
}

}  // extern "C"
