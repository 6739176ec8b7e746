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

constexpr size_t kMaxLds = 128 * 1024;

size_t lds_bytes(int mt, int nb, bool dual) {
  return sizeof(float) * ((size_t)mt * nb * (kQK + 16) + (size_t)mt * nb * 8 +
                          (size_t)4 * 64 * mt * (dual ? 2 : 1));
}

template <int MT, bool DUAL>
int launch_lds(const GemvArgs& a, const char* op) {
  const size_t lds = lds_bytes(MT, a.nb, DUAL);
  auto kern = q4k_gemv_lds_kernel<MT, DUAL>;
  DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxLds));
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
