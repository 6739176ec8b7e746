// Q4_K prefill GEMM for gfx950: C[M,N] = alpha * A[M,K] . dequant(W)[N,K]^T for M >= 16, and
// the fused gate/up projection with gated activation, on the matrix cores.
//
// Tiles: a wave computes a 64 x 64 (or 32 x 32) quadrant with v_mfma_f32_32x32x16_f16 (f32
// accumulators), four waves a 128 x 128 (64 x 64) tile, and a workgroup is one or two such groups
// stacked along M against the same weight tile: 256 x 128 with eight waves for large problems.
// K advances 64 at a time: one 32-byte nibble chunk of a super-block (low nibbles = sub-block
// 2c, high = 2c+1) per weight row.
//   weights  a thread loads 8 or 16 nibble bytes of a row + the block header and rebuilds the
//            weights as f16: (w & 0x000F000F) | 0x64006400 is the pair (1024 + q) in f16, one
//            packed subtract and one packed fma with (d*sc, -dmin*mn) finish them: about 2
//            vector ops per weight, paid once per workgroup tile (hence the tall tiles).
//   A        packed once per product by a pre-pass (pack_a_row_kernel / pack_a_kernel): each
//            row scaled by the power of two that puts its largest element at 2^14, rounded to
//            f16, k-permuted, rows zero-padded to a multiple of 64.  The GEMM tiles then copy
//            16-byte pieces into LDS, no conversion in the K loop, and the epilogue divides the
//            row factor out again, exactly: activations beyond the f16 range (65504) neither
//            overflow nor lose small rows to subnormals.
// Both tiles sit in LDS as [row][64 k] with a 16-byte pad (conflict-free 16-byte fragment
// reads) and are double-buffered, one barrier per K step.
// The K loop is bound by instruction issue, not by memory (with every load served from the
// first-level cache it runs 3 % faster) and not by the matrix cores alone (they are busy for
// half of the loop's cycles at the 1.84 GHz the part holds under this load).  Measured on this
// part: a wave issues an independent vector instruction every 5 cycles and a dependent one every
// 8, a matrix-core instruction occupies its pipe for 32, and a wave may issue 4 vector
// instructions behind a matrix-core instruction at no cost.  Hence:
//   * every wave both multiplies and produces, and the producer's work of a step (LDS stores of
//     the A tile, scale unpack, nibble dwords, the loads two tiles ahead) is dealt out in pieces
//     behind the matrix-core instructions of the same step, in program order pinned with
//     scheduling barriers;
//   * fragments are double-buffered in registers, so LDS latency runs under the previous slice;
//   * all global loads are unconditional: one conditional load makes the compiler wait for every
//     outstanding load before a tile is used, which halves the lookahead.
// Tried and measured slower: producer / multiplier wave specialisation (four waves each: the
// producers' 250 vector instructions per step at one wave per SIMD took longer than the
// multipliers' step, 1.3 us per K step against 1.0 us for eight symmetric waves on the same
// 256 x 128 x 2 problem), two A sub-tiles per wave (one wave per SIMD), 256 x 64 blocks.
// k order inside every group of 4 is (0, 2, 1, 3) in BOTH tiles: that is the order the masked
// nibble pairs come out in, and a contraction index may be permuted freely when both operands
// agree.
#include <algorithm>
#include <cstdlib>

#include "dh_common.h"
#include "q4k_device.h"

namespace {

using dh::kBlockBytes;
using dh::kQK;

typedef __attribute__((ext_vector_type(8))) _Float16 half8_t;
typedef __attribute__((ext_vector_type(2))) _Float16 half2_t;
typedef __attribute__((ext_vector_type(16))) float float16_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

int env_ksplit() { return dh::tuning_int("DH_GEMM_KSPLIT", 0); }

constexpr int BK = 64;
constexpr int LDS_ROW = BK + 8;                    // halves per LDS row (144 bytes)

struct GemmArgs {
  const float* A;        // [M][K]
  const _Float16* Apk;   // [M][kpad] packed activations (see pack_a_kernel)
  int kpad;              // K rounded up to a multiple of 64
  const uint8_t* W;      // Q4_K rows [N][nb*144]
  const uint8_t* W2;     // second matrix (DUAL) or null
  void* C;               // [M][N] f32 or f16
  const float* residual; // [M][N] or null
  int M, N, K, nb;
  float alpha;
  int c_f16, activation;
  float clamp_max;
  // split-K: blockIdx.z takes K steps [z * kt_per_split, ...) and writes its raw partial product to
  // partial[z][M][N]; splitk_reduce_kernel adds the pieces in order
  int ksplit, kt_per_split;
  float* partial;
  const float2* row_scale;   // [M] (multiplier applied before the f16 rounding, its inverse)
  // RMSNorm prologue (norm_weight null = off): rows are normalised while they are packed
  const float* norm_weight;  // [K]
  float norm_eps;
  int norm_weight_offset;    // 1: scale by (1 + w)
};

// Packs the activations for the matrix cores, one wave per row (four rows per workgroup):
// finds the row's largest magnitude, scales by the power of two that puts it at 2^14 ((1, 1) for
// an all-zero row), rounds to f16 and writes the row with its k in (0, 2, 1, 3) order inside
// every group of four (the order the masked nibble pairs of the weights come out in), zero-padded
// to kpad.  out_scale[m] = (factor, 1 / factor).
__global__ __launch_bounds__(256) void pack_a_kernel(const float* __restrict__ A, int M, int K, int kpad,
                                                     _Float16* __restrict__ Apk, float2* __restrict__ out_scale) {
  const int lane = threadIdx.x & 63, m = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (m >= M) return;
  const float* row = A + (int64_t)m * K;
  const bool vec = (K & 3) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0;
  float mx = 0.f;
  if (vec) {
    for (int k = 4 * lane; k < K; k += 256) {
      const float4 v = *reinterpret_cast<const float4*>(row + k);
      mx = fmaxf(fmaxf(mx, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w)));
    }
  } else {
    for (int k = lane; k < K; k += 64) mx = fmaxf(mx, fabsf(row[k]));
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
  int e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 127;
  e = max(-100, min(100, e));
  if (!(mx > 0.f) || !(mx < INFINITY)) e = 14;
  const float mul = __uint_as_float((uint32_t)(127 + 14 - e) << 23);
  if (lane == 0) out_scale[m] = make_float2(mul, __uint_as_float((uint32_t)(127 - 14 + e) << 23));
  _Float16* dst = Apk + (int64_t)m * kpad;
  for (int k = 4 * lane; k < kpad; k += 256) {
    float v[4];
    if (vec && k + 3 < K) {
      const float4 t = *reinterpret_cast<const float4*>(row + k);      // second read: cache hit
      v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) v[j] = k + j < K ? row[k + j] : 0.f;
    }
    const half2_t p0 = {(_Float16)(v[0] * mul), (_Float16)(v[2] * mul)};
    const half2_t p1 = {(_Float16)(v[1] * mul), (_Float16)(v[3] * mul)};
    *reinterpret_cast<uint2*>(dst + k) = make_uint2(__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1));
  }
}

// The same packing with one workgroup per row and the row held in registers (NV float4 per
// thread, K <= 1024 NV): every load of a row is in flight at once and the row is read once.  One
// wave per row walks its row in dependent steps and is latency-bound (14.5 us for 512 x 6912).
template <int NV>
__global__ __launch_bounds__(256) void pack_a_row_kernel(const float* __restrict__ A, int M, int K, int kpad,
                                                         _Float16* __restrict__ Apk, float2* __restrict__ out_scale,
                                                         const float* __restrict__ norm_w, float norm_eps,
                                                         int norm_w_offset) {
  __shared__ float wave_max[4];
  __shared__ float wave_ss[4];
  const int tid = threadIdx.x, m = blockIdx.x;
  const float* row = A + (int64_t)m * K;
  const bool vec = (K & 3) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0;
  float v[NV][4];
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int k = 4 * tid + 1024 * i;
    if (vec && k + 3 < K) {
      const float4 t = *reinterpret_cast<const float4*>(row + k);
      v[i][0] = t.x; v[i][1] = t.y; v[i][2] = t.z; v[i][3] = t.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) v[i][j] = k + j < K ? row[k + j] : 0.f;
    }
  }
  if (norm_w) {
    // RMSNorm of the row, same arithmetic as the stand-alone kernel: x * rsqrt(mean x^2 + eps) * w
    float wn[NV][4];
    const bool wvec = (K & 3) == 0 && (reinterpret_cast<uintptr_t>(norm_w) & 15) == 0;
#pragma unroll
    for (int i = 0; i < NV; i++) {
      const int k = 4 * tid + 1024 * i;
      if (wvec && k + 3 < K) {
        const float4 t = *reinterpret_cast<const float4*>(norm_w + k);
        wn[i][0] = t.x; wn[i][1] = t.y; wn[i][2] = t.z; wn[i][3] = t.w;
      } else {
#pragma unroll
        for (int j = 0; j < 4; j++) wn[i][j] = k + j < K ? norm_w[k + j] : 0.f;
      }
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) ss = fmaf(v[i][j], v[i][j], ss);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
    if ((tid & 63) == 0) wave_ss[tid >> 6] = ss;
    __syncthreads();
    const float inv = 1.0f / sqrtf((wave_ss[0] + wave_ss[1] + wave_ss[2] + wave_ss[3]) / (float)K + norm_eps);
#pragma unroll
    for (int i = 0; i < NV; i++)
#pragma unroll
      for (int j = 0; j < 4; j++) v[i][j] = v[i][j] * inv * (norm_w_offset ? 1.0f + wn[i][j] : wn[i][j]);
  }
  float mx = 0.f;
#pragma unroll
  for (int i = 0; i < NV; i++)
#pragma unroll
    for (int j = 0; j < 4; j++) mx = fmaxf(mx, fabsf(v[i][j]));
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) mx = fmaxf(mx, __shfl_xor(mx, off, 64));
  if ((tid & 63) == 0) wave_max[tid >> 6] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(wave_max[0], wave_max[1]), fmaxf(wave_max[2], wave_max[3]));
  int e = (int)((__float_as_uint(mx) >> 23) & 0xFF) - 127;
  e = max(-100, min(100, e));
  if (!(mx > 0.f) || !(mx < INFINITY)) e = 14;
  const float mul = __uint_as_float((uint32_t)(127 + 14 - e) << 23);
  if (tid == 0) out_scale[m] = make_float2(mul, __uint_as_float((uint32_t)(127 - 14 + e) << 23));
  _Float16* dst = Apk + (int64_t)m * kpad;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int k = 4 * tid + 1024 * i;
    if (k < kpad) {
      const half2_t p0 = {(_Float16)(v[i][0] * mul), (_Float16)(v[i][2] * mul)};
      const half2_t p1 = {(_Float16)(v[i][1] * mul), (_Float16)(v[i][3] * mul)};
      *reinterpret_cast<uint2*>(dst + k) = make_uint2(__builtin_bit_cast(uint32_t, p0), __builtin_bit_cast(uint32_t, p1));
    }
  }
}

// Dequantisation in pieces, for the K loop that spreads it between the matrix-core
// instructions.  Scales of sub-blocks 2c, 2c+1 as broadcastable f16 pairs, without a branch on c:
struct PairScales {
  half2_t slo, mlo, shi, mhi;     // (scale, scale), (-min, -min) of the low- and high-nibble sub-block
};
__device__ __forceinline__ PairScales pair_scales_f16(const u32x4_t hdr, const int c) {
  const float d = f16lo(hdr[0]), dmin = f16hi(hdr[0]);
  const int sh = (c & 1) * 16;
  const uint32_t a1 = hdr[1] >> sh, a2 = hdr[2] >> sh, a3 = hdr[3] >> sh;
  const bool low = c < 2;
  const uint32_t scp = low ? (a1 & 0x3F3Fu) : ((a3 & 0x0F0Fu) | ((a1 >> 2) & 0x3030u));
  const uint32_t mnp = low ? (a2 & 0x3F3Fu) : (((a3 >> 4) & 0x0F0Fu) | ((a2 >> 2) & 0x3030u));
  const _Float16 sl = (_Float16)(d * (float)(scp & 0xFFu)), sh_ = (_Float16)(d * (float)((scp >> 8) & 0xFFu));
  const _Float16 ml = (_Float16)(-dmin * (float)(mnp & 0xFFu)), mh = (_Float16)(-dmin * (float)((mnp >> 8) & 0xFFu));
  PairScales r;
  r.slo = half2_t{sl, sl}; r.mlo = half2_t{ml, ml};
  r.shi = half2_t{sh_, sh_}; r.mhi = half2_t{mh, mh};
  return r;
}
// One dword of nibbles (8 weights) -> two low-nibble and two high-nibble f16 pairs.
// `magic` is 0x64006400 held in a vector register (see magic_1024): with the constant visible the
// compiler emits v_and + v_or, since one instruction may read only one literal or scalar.
__device__ __forceinline__ void dequant_dword(const uint32_t w, const PairScales& ps, const uint32_t magic, uint32_t& lo0,
                                              uint32_t& lo1, uint32_t& hi0, uint32_t& hi1) {
  const half2_t k1024 = {(_Float16)1024.f, (_Float16)1024.f};
  const half2_t v0 = __builtin_bit_cast(half2_t, (w & 0x000F000Fu) | magic) - k1024;
  const half2_t v1 = __builtin_bit_cast(half2_t, ((w >> 8) & 0x000F000Fu) | magic) - k1024;
  const half2_t v2 = __builtin_bit_cast(half2_t, ((w >> 4) & 0x000F000Fu) | magic) - k1024;
  const half2_t v3 = __builtin_bit_cast(half2_t, ((w >> 12) & 0x000F000Fu) | magic) - k1024;
  lo0 = __builtin_bit_cast(uint32_t, v0 * ps.slo + ps.mlo);
  lo1 = __builtin_bit_cast(uint32_t, v1 * ps.slo + ps.mlo);
  hi0 = __builtin_bit_cast(uint32_t, v2 * ps.shi + ps.mhi);
  hi1 = __builtin_bit_cast(uint32_t, v3 * ps.shi + ps.mhi);
}

__device__ __forceinline__ uint32_t magic_1024() {
  uint32_t m;
  asm("v_mov_b32 %0, 0x64006400" : "=v"(m));
  return m;
}

// tanh-form GELU with tanh(t) = 1 - 2 / (1 + e^{2t}): a handful of instructions, inlined once per
// accumulator element in the epilogue.
__device__ __forceinline__ float gelu_tanh_fast(float x) {
  const float t = fminf(fmaxf(0.7978845608f * (x + 0.044715f * x * x * x), -15.0f), 15.0f);
  return 0.5f * x * (2.0f - 2.0f / (1.0f + __expf(2.0f * t)));
}


// T = MFMA tiles per wave along each of M and N (T = 2: a 64 x 64 quadrant per wave, T = 1:
// 32 x 32 when larger tiles would leave most compute units idle).  Four waves cover a
// 64T x 64T tile; MG = groups of four waves stacked along M, all multiplying against the same
// weight tile.  Workgroup tile: 64T MG x 64T.  The weights of a tile are dequantised once per
// workgroup, so MG = 2 halves that work per matrix-core instruction.
template <bool DUAL, int T, int MG>
__global__ __launch_bounds__(256 * MG) void q4k_gemm_kernel(const GemmArgs a) {
  constexpr int NMAT = DUAL ? 2 : 1;
  constexpr int SUBM = 64 * T;                               // rows of one group's A tile
  constexpr int BM = SUBM * MG, BN = 64 * T;
  constexpr int A_HALVES = BM * LDS_ROW, B_HALVES = BN * LDS_ROW;
  extern __shared__ __align__(16) _Float16 lds[];            // [2 buffers][A | B | (B2)]
  constexpr int BUF_HALVES = A_HALVES + NMAT * B_HALVES;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  constexpr int PT = 256 * MG;                               // threads of the workgroup
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int wm = (wave >> 2) * SUBM + ((wave >> 1) & 1) * 32 * T, wn = (wave & 1) * 32 * T;
  const int fr = lane & 31, fg = lane >> 5;                  // fragment row / k half
  const int64_t row_bytes = (int64_t)a.nb * kBlockBytes;
  const int kt0 = a.ksplit > 1 ? (int)blockIdx.z * a.kt_per_split : 0;
  const int nkt = a.ksplit > 1 ? min((a.K + BK - 1) / BK, kt0 + a.kt_per_split) : (a.K + BK - 1) / BK;

  // ---- global -> register staging
  // A: 16-byte pieces of the packed rows, idx = tid + PT i: row idx >> 3, halves 8 * (idx & 7)
  // W: item (matrix, row, half) = 16 nibble bytes of one row + its block header; SPLIT threads
  //    share an item (QD dwords each) when there are more threads than items
  constexpr int NA = BM * 8 / PT;                            // 16-byte loads of A per thread
  constexpr int ITEMS = 2 * BN * NMAT;
  constexpr int SPLIT = PT > ITEMS ? (PT / ITEMS > 2 ? 2 : PT / ITEMS) : 1;
  constexpr int QD = 4 / SPLIT;                              // dwords of nibbles per thread and item
  constexpr int UNITS = ITEMS * SPLIT;
  constexpr int NW = UNITS > PT ? UNITS / PT : 1;            // units per thread
  constexpr bool ALL_ACTIVE = UNITS >= PT;                   // every producer thread has its units
  static_assert(BM * 8 % PT == 0 && (UNITS % PT == 0 || UNITS < PT), "producer threads must tile the work");
  // per-thread byte offsets of the loads (the host checks that both operands stay below 2 GB)
  uint32_t w_off[NW], a_off[NA];
  bool w_second[NW];
  int w_lds[NW], w_qoff[NW];
  bool w_active[NW];
#pragma unroll
  for (int j = 0; j < NW; j++) {
    const int u = tid + PT * j, it = u / SPLIT, sub = u % SPLIT;
    const int mt = it / (2 * BN), rem = it % (2 * BN), row = rem >> 1, half = rem & 1;
    w_active[j] = u < UNITS;
    w_qoff[j] = 16 + 16 * half + 8 * sub;
    // rows past the tile or the matrix re-read row N - 1: the loads stay unconditional
    // a matrix's units are a multiple of 64 threads: uniform per wave, so the base stays scalar
    w_second[j] = NMAT > 1 && __builtin_amdgcn_readfirstlane(mt & 1) != 0;
    w_off[j] = (uint32_t)((int64_t)min(n0 + row, a.N - 1) * row_bytes);
    w_lds[j] = A_HALVES + (mt % NMAT) * B_HALVES + row * LDS_ROW + 16 * half + 8 * sub;
  }
  // Two register sets: while tile kt is multiplied, tile kt+1 waits in one set and the loads of
  // tile kt+2 are in flight into the other, so a load has two K steps to arrive.
  struct Staged {
    u32x4_t a[NA];
    u32x4_t q[NW], h[NW];
  };
  Staged st0, st1;
  // row factors of this tile's activation rows: one global read each, then LDS
  __shared__ float2 rs_lds[BM];
  for (int r = threadIdx.x; r < BM; r += blockDim.x) rs_lds[r] = a.row_scale[min(m0 + r, a.M - 1)];

  // Every load is unconditional (past the end of K the last tile is loaded again and never used,
  // rows past the matrix re-read its last row): loads complete in order, so with exactly one
  // tile's loads issued per step the wait in front of the older tile leaves the younger tile's
  // loads in flight.  A load under a condition turns that wait into "all loads", and a load then
  // has one K step to arrive instead of two.
#pragma unroll
  for (int i = 0; i < NA; i++) {
    const int idx = tid + PT * i, r = idx >> 3;
    a_off[i] = (uint32_t)(((int64_t)min(m0 + r, a.M - 1) * a.kpad + 8 * (idx & 7)) * 2);
  }
  // Buffer loads: address = descriptor base + per-thread 32-bit offset + per-step scalar offset,
  // so the loop holds no vector address arithmetic (and a read past a tensor would return 0).
  const __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<_Float16*>(a.Apk), 0, (int)min((int64_t)a.M * a.kpad * 2, (int64_t)0x7fffffff), 0x00020000);
  const int w_bytes = (int)min((int64_t)a.N * row_bytes, (int64_t)0x7fffffff);
  const __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(a.W), 0, w_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t w2_rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t*>(NMAT > 1 ? a.W2 : a.W), 0, w_bytes, 0x00020000);
  auto load_tile = [&](int kt, Staged& st) {
#pragma unroll
    for (int i = 0; i < NA; i++)
      st.a[i] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(a_rsrc, a_off[i], kt * (BK * 2), 0));
    const int blk = kt >> 2, c = kt & 3;
#pragma unroll
    for (int j = 0; j < NW; j++) {
      const __amdgpu_buffer_rsrc_t r = w_second[j] ? w2_rsrc : w_rsrc;
      st.h[j] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(r, w_off[j], blk * kBlockBytes, 0));
      if constexpr (QD == 4) {
        st.q[j] = __builtin_bit_cast(u32x4_t, __builtin_amdgcn_raw_buffer_load_b128(r, w_off[j] + w_qoff[j],
                                                                                  blk * kBlockBytes + 32 * c, 0));
      } else {
        const auto v = __builtin_amdgcn_raw_buffer_load_b64(r, w_off[j] + w_qoff[j], blk * kBlockBytes + 32 * c, 0);
        st.q[j][0] = v[0];
        st.q[j][1] = v[1];
      }
    }
  };

  float16_t acc[NMAT][T][T];
#pragma unroll
  for (int mt = 0; mt < NMAT; mt++)
#pragma unroll
    for (int i = 0; i < T; i++)
#pragma unroll
      for (int j = 0; j < T; j++)
#pragma unroll
        for (int e = 0; e < 16; e++) acc[mt][i][j][e] = 0.f;

  // Multiplies the tile in LDS buffer kt & 1.  Fragments are double-buffered in registers: the
  // reads of k slice ks+1 are issued before the matrix-core instructions of slice ks, so the LDS
  // latency runs under them.  after(slot) is called behind every matrix-core instruction
  // (slot = its index within the K step).
  constexpr int NMFMA = (BK / 16) * NMAT * T * T;
  constexpr int FD = 2;                                      // fragment sets in flight (3 and 4 measured: no gain)
  auto multiply_step = [&](int kt, auto&& after) {
    const _Float16* At = lds + (kt & 1) * BUF_HALVES;
    half8_t af[FD][T], bf[FD][NMAT][T];
    auto read_frags = [&](int ks, half8_t (&fa)[T], half8_t (&fb)[NMAT][T]) {
#pragma unroll
      for (int i = 0; i < T; i++)
        fa[i] = *reinterpret_cast<const half8_t*>(At + (wm + 32 * i + fr) * LDS_ROW + 16 * ks + 8 * fg);
#pragma unroll
      for (int mt = 0; mt < NMAT; mt++)
#pragma unroll
        for (int j = 0; j < T; j++)
          fb[mt][j] = *reinterpret_cast<const half8_t*>(At + A_HALVES + mt * B_HALVES + (wn + 32 * j + fr) * LDS_ROW +
                                                        16 * ks + 8 * fg);
    };
#pragma unroll
    for (int ks = 0; ks < FD - 1; ks++) read_frags(ks, af[ks], bf[ks]);
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      if (ks + FD - 1 < BK / 16) read_frags(ks + FD - 1, af[(ks + FD - 1) % FD], bf[(ks + FD - 1) % FD]);
#pragma unroll
      for (int mt = 0; mt < NMAT; mt++)
#pragma unroll
        for (int i = 0; i < T; i++)
#pragma unroll
          for (int j = 0; j < T; j++) {
            // accumulators pinned to the accumulation registers: left to itself the compiler keeps
            // them in vector registers and copies all of them aside and back every K step
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0"
                         : "+a"(acc[mt][i][j])
                         : "v"(af[ks % FD][i]), "v"(bf[ks % FD][mt][j]));
            after(((ks * NMAT + mt) * T + i) * T + j);
          }
    }
  };
  auto no_hook = [](int) {};

  // The producer's work of one K step in NPARTS pieces, so that it can be dealt out between the
  // matrix-core instructions of the same wave (each runs for 32 cycles while the wave is free to
  // issue vector instructions): piece 0 stores the A tile, then per weight unit the scales and
  // its dwords of nibbles, and the last piece issues the loads two tiles ahead.
  constexpr int NPARTS = 2 + (1 + QD) * NW;
  PairScales ps[NW];
  const uint32_t magic = magic_1024();
  uint32_t lo_w[NW][2 * QD], hi_w[NW][2 * QD];
  auto produce_part = [&](int part, int kt, Staged& nxt) {      // moves tile kt + 1
    _Float16* At = lds + ((kt & 1) ^ 1) * BUF_HALVES;
    if (part == 0) {
#pragma unroll
      for (int i = 0; i < NA; i++) {
        const int idx = tid + PT * i, r = idx >> 3;
        *reinterpret_cast<u32x4_t*>(At + r * LDS_ROW + 8 * (idx & 7)) = nxt.a[i];
      }
    } else if (part == NPARTS - 1) {
      load_tile(min(kt + 3, nkt - 1), nxt);
    } else {
      const int j = (part - 1) / (1 + QD), d = (part - 1) % (1 + QD) - 1;
      if (ALL_ACTIVE || w_active[j]) {
        if (d < 0) {
          ps[j] = pair_scales_f16(nxt.h[j], (kt + 1) & 3);
        } else {
          dequant_dword(nxt.q[j][d], ps[j], magic, lo_w[j][2 * d], lo_w[j][2 * d + 1], hi_w[j][2 * d], hi_w[j][2 * d + 1]);
          if (d & 1) {
            _Float16* Bt = At + w_lds[j] + 4 * (d - 1);
            *reinterpret_cast<uint4*>(Bt) = make_uint4(lo_w[j][2 * d - 2], lo_w[j][2 * d - 1], lo_w[j][2 * d], lo_w[j][2 * d + 1]);
            *reinterpret_cast<uint4*>(Bt + 32) = make_uint4(hi_w[j][2 * d - 2], hi_w[j][2 * d - 1], hi_w[j][2 * d], hi_w[j][2 * d + 1]);
          }
        }
      }
    }
  };
  auto produce_first = [&]() {
    load_tile(kt0, st0);
#pragma unroll
    for (int part = 0; part < NPARTS - 1; part++) produce_part(part, kt0 - 1, st0);   // tile kt0 into its buffer
    load_tile(min(kt0 + 1, nkt - 1), st0);
    load_tile(min(kt0 + 2, nkt - 1), st1);
  };
  // Multiplies tile kt and, between its matrix-core instructions, moves tile kt+1 out of `nxt`
  // into the other LDS buffer and reloads `nxt` with tile kt+3.
  auto fused_step = [&](int kt, Staged& nxt) {
    multiply_step(kt, [&](int slot) {
#pragma unroll
      for (int part = 0; part < NPARTS; part++)
        if (part * NMFMA / NPARTS == slot) produce_part(part, kt, nxt);
      __builtin_amdgcn_sched_barrier(0);
    });
  };

  produce_first();
  __syncthreads();
  int kt = kt0;
  for (; kt + 2 < nkt; kt += 2) {        // st0 holds the tiles at odd distance from kt0, st1 the even ones
    fused_step(kt, st0);
    __syncthreads();
    fused_step(kt + 1, st1);
    __syncthreads();
  }
  if (kt + 1 < nkt) {
    fused_step(kt, st0);
    __syncthreads();
    kt++;
  }
  multiply_step(kt, no_hook);

  // the matrix-core instructions above are inline asm, invisible to the compiler's hazard
  // checks: give the last one time to retire before its accumulators are read
  asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
  // ---- epilogue: lane holds column n = lane & 31 of rows 8 (e / 4) + 4 fg + (e % 4)
#pragma unroll
  for (int i = 0; i < T; i++)
#pragma unroll
    for (int j = 0; j < T; j++) {
      const int n = n0 + wn + 32 * j + fr;
#pragma unroll
      for (int e = 0; e < 16; e++) {
        const int rl = wm + 32 * i + 8 * (e >> 2) + 4 * fg + (e & 3);
        const int m = m0 + rl;
        if (m < a.M && n < a.N) {
          float v;
          const float unscale = rs_lds[rl].y;
          if (!DUAL && a.ksplit > 1) {
            a.partial[((int64_t)blockIdx.z * a.M + m) * a.N + n] = acc[0][i][j][e] * unscale;
            continue;
          }
          if (DUAL) {
            const float g = acc[0][i][j][e] * unscale, u = acc[NMAT - 1][i][j][e] * unscale;
            v = (a.activation == DH_ACT_SILU ? act_silu(g) : gelu_tanh_fast(g)) * u * a.alpha;
            if (a.activation == DH_ACT_SILU && a.clamp_max > 0.f) v = fminf(fmaxf(v, -a.clamp_max), a.clamp_max);
          } else {
            v = acc[0][i][j][e] * unscale * a.alpha;
            if (a.residual) v += a.residual[(int64_t)m * a.N + n];
          }
          if (a.c_f16)
            reinterpret_cast<__half*>(a.C)[(int64_t)m * a.N + n] = __float2half(v);
          else
            reinterpret_cast<float*>(a.C)[(int64_t)m * a.N + n] = v;
        }
      }
    }
}

// C = alpha * (sum of the split-K pieces, in split order) + residual.  Four consecutive outputs per
// thread when the row length allows 16-byte accesses, every piece's load in flight before the sums.
constexpr int kMaxSplit = 8;
template <bool VEC>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const GemmArgs a) {
  const int64_t total = (int64_t)a.M * a.N;
  constexpr int W = VEC ? 4 : 1;
  const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * W;
  if (i >= total) return;
  float p[kMaxSplit][W];
#pragma unroll
  for (int z = 0; z < kMaxSplit; z++) {
    if (z < a.ksplit) {
      if constexpr (VEC) {
        const float4 t = *reinterpret_cast<const float4*>(a.partial + (int64_t)z * total + i);
        p[z][0] = t.x; p[z][1] = t.y; p[z][2] = t.z; p[z][3] = t.w;
      } else {
        p[z][0] = a.partial[(int64_t)z * total + i];
      }
    }
  }
  float r[W];
#pragma unroll
  for (int e = 0; e < W; e++) r[e] = 0.f;
  if (a.residual) {
    if constexpr (VEC) {
      const float4 t = *reinterpret_cast<const float4*>(a.residual + i);
      r[0] = t.x; r[1] = t.y; r[2] = t.z; r[3] = t.w;
    } else {
      r[0] = a.residual[i];
    }
  }
#pragma unroll
  for (int e = 0; e < W; e++) {
    float s = 0.f;
#pragma unroll
    for (int z = 0; z < kMaxSplit; z++)
      if (z < a.ksplit) s += p[z][e];
    r[e] = s * a.alpha + r[e];
  }
  if (a.c_f16) {
    __half* c = reinterpret_cast<__half*>(a.C) + i;
#pragma unroll
    for (int e = 0; e < W; e++) c[e] = __float2half(r[e]);
  } else if constexpr (VEC) {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(a.C) + i) = make_float4(r[0], r[1], r[2], r[3]);
  } else {
    reinterpret_cast<float*>(a.C)[i] = r[0];
  }
}

template <bool DUAL, int T, int MG>
int launch_gemm_cfg(const GemmArgs& a, const char* op) {
  constexpr int BM = 64 * T * MG, BN = 64 * T;
  const size_t lds = (size_t)2 * (BM + (DUAL ? 2 : 1) * BN) * LDS_ROW * sizeof(_Float16);
  auto kern = q4k_gemm_kernel<DUAL, T, MG>;
  static bool attr_set = false;   // once per instantiation: the call costs microseconds
  if (!attr_set) {
    DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  const dim3 grid((unsigned)dh::ceil_div(a.N, BN), (unsigned)dh::ceil_div(a.M, BM), (unsigned)std::max(1, a.ksplit));
  hipLaunchKernelGGL(kern, grid, dim3(256 * MG), lds, dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  if (a.ksplit > 1) {
    const int64_t total = (int64_t)a.M * a.N;
    if (a.ksplit > kMaxSplit) return dh::fail(2, "[%s] internal: K cut into %d pieces, the reduction takes %d", op, a.ksplit, kMaxSplit);
    const bool vec = total % 4 == 0 && (reinterpret_cast<uintptr_t>(a.C) | reinterpret_cast<uintptr_t>(a.residual)) % 16 == 0;
    if (vec)
      hipLaunchKernelGGL(splitk_reduce_kernel<true>, dim3((unsigned)dh::ceil_div(total / 4, 256)), dim3(256), 0, dh::stream(), a);
    else
      hipLaunchKernelGGL(splitk_reduce_kernel<false>, dim3((unsigned)dh::ceil_div(total, 256)), dim3(256), 0, dh::stream(), a);
    DH_CHECK_LAUNCH(op);
  }
  return 0;
}

// 128 x 128 tiles when they occupy at least half of the compute units (their higher matrix-core
// share wins from there on), else 64 x 64.
template <bool DUAL>
int launch_gemm(GemmArgs a, const char* op) {
  // rows beyond the capacity of the packed-activation scratch go in further passes
  a.kpad = (a.K + BK - 1) / BK * BK;
  if (a.norm_weight && a.K > 16384)
    return dh::fail(1, "[%s] the RMSNorm prologue serves K <= 16384 at M >= 16 (K=%d)", op, a.K);
  // the kernel addresses a weight row as a 32-bit byte offset into a buffer descriptor
  if ((int64_t)a.N * a.nb * kBlockBytes >= ((int64_t)1 << 31))
    return dh::fail(1, "[%s] a weight tensor of %d x %d (2 GB or more) is beyond the prefill GEMM; split it by rows", op,
                    a.N, a.K);
  if (dh::plan_note(DH_PLAN_GEMM)) return 0;
  size_t pk_bytes = 0;
  _Float16* packed = reinterpret_cast<_Float16*>(dh::gemm_packed_a(&pk_bytes));
  float2* scales = reinterpret_cast<float2*>(dh::gemm_row_scale());
  if (!packed || !scales) return dh::fail(2, "[%s] the library's scratch buffers are missing (dh_init)", op);
  const int cap = (int)std::min<size_t>((size_t)dh::gemm_row_scale_capacity(), pk_bytes / ((size_t)a.kpad * 2));
  if (cap < 16) return dh::fail(1, "[%s] K=%d is too long for the prefill GEMM's activation scratch", op, a.K);
  if (a.M > cap) {
    const size_t c_elem = a.c_f16 ? 2 : 4;
    for (int m0 = 0; m0 < a.M; m0 += cap) {
      GemmArgs b = a;
      b.M = std::min(cap, a.M - m0);
      b.A = a.A + (int64_t)m0 * a.K;
      b.C = static_cast<char*>(a.C) + (int64_t)m0 * a.N * c_elem;
      b.residual = a.residual ? a.residual + (int64_t)m0 * a.N : nullptr;
      const int rc = launch_gemm<DUAL>(b, op);
      if (rc) return rc;
    }
    return 0;
  }
#define DH_PACK_ROWS(NV_)                                                                          \
  hipLaunchKernelGGL(pack_a_row_kernel<NV_>, dim3((unsigned)a.M), dim3(256), 0, dh::stream(), a.A, a.M, a.K, \
                     a.kpad, packed, scales, a.norm_weight, a.norm_eps, a.norm_weight_offset)
  if (a.K <= 2048) DH_PACK_ROWS(2);
  else if (a.K <= 4096) DH_PACK_ROWS(4);
  else if (a.K <= 8192) DH_PACK_ROWS(8);
  else if (a.K <= 16384) DH_PACK_ROWS(16);
  else if (a.norm_weight)
    return dh::fail(1, "[%s] the RMSNorm prologue serves K <= 16384 at M >= 16 (K=%d)", op, a.K);
  else
    hipLaunchKernelGGL(pack_a_kernel, dim3((unsigned)dh::ceil_div(a.M, 4)), dim3(256), 0, dh::stream(), a.A, a.M, a.K,
                       a.kpad, packed, scales);
#undef DH_PACK_ROWS
  DH_CHECK_LAUNCH(op);
  a.row_scale = scales;
  a.Apk = packed;
  // Tile choice, largest first: 256 x 128 (eight waves) when such tiles fill the compute units,
  // for the fused gate/up pair 128 x 64 (eight waves) next, then 128 x 128 (four waves, two
  // workgroups per compute unit) when those occupy at least half of them, else 64 x 64.
  const int64_t big_tiles = dh::ceil_div(a.M, 128) * dh::ceil_div(a.N, 128);
  const int64_t tall_tiles = dh::ceil_div(a.M, 256) * dh::ceil_div(a.N, 128);
  a.ksplit = 1;
  if (tall_tiles >= dh::num_cus()) return launch_gemm_cfg<DUAL, 2, 2>(a, op);
  if (2 * big_tiles >= dh::num_cus()) {
    if constexpr (DUAL) {
      return launch_gemm_cfg<true, 1, 2>(a, op);
    } else {
      return launch_gemm_cfg<false, 2, 1>(a, op);
    }
  }
  // Few tiles and a long K: every workgroup would walk K alone at one memory round trip per
  // step.  Cut K so that about three workgroups share a compute unit and overlap each other's
  // waits; the pieces meet in the library's scratch buffer.
  if (!DUAL) {
    static const int env_split = env_ksplit();
    static const int env_big = dh::tuning_int("DH_GEMM_BIGSPLIT", 1);
    // 128 x 128 tiles with K cut into pieces when that fills the compute units: their matrix-core
    // share is higher than that of 64 x 64 tiles
    if (env_big) {
      const int nkt = (a.K + BK - 1) / BK;
      size_t ws_bytes = 0;
      float* ws = dh::splitk_workspace(&ws_bytes);
      int split = (int)std::min<int64_t>(8, dh::num_cus() / std::max<int64_t>(1, big_tiles));
      split = std::min(split, nkt / 8);
      while (split > 1 && (size_t)split * a.M * a.N * sizeof(float) > ws_bytes) split--;
      if (split > 1 && ws && big_tiles * split * 2 >= dh::num_cus()) {
        a.kt_per_split = (int)dh::ceil_div(nkt, split);
        a.ksplit = (int)dh::ceil_div(nkt, a.kt_per_split);
        a.partial = ws;
        return launch_gemm_cfg<false, 2, 1>(a, op);
      }
    }
    const int64_t tiles = dh::ceil_div(a.M, 64) * dh::ceil_div(a.N, 64);
    const int nkt = (a.K + BK - 1) / BK;
    size_t ws_bytes = 0;
    float* ws = dh::splitk_workspace(&ws_bytes);
    int split = (int)std::min<int64_t>(8, dh::ceil_div(3 * (int64_t)dh::num_cus(), tiles));
    split = std::min(split, nkt / 8);
    if (env_split > 0) split = env_split;
    while (split > 1 && (size_t)split * a.M * a.N * sizeof(float) > ws_bytes) split--;
    if (split > 1 && ws) {
      a.kt_per_split = (int)dh::ceil_div(nkt, split);
      a.ksplit = (int)dh::ceil_div(nkt, a.kt_per_split);
      a.partial = ws;
    }
  }
  return launch_gemm_cfg<DUAL, 1, 1>(a, op);
}

}  // namespace


namespace dh {

bool q4k_gemm_serves(int M, int K, const void* A) {
  (void)K; (void)A;          // any K and alignment: the packing pre-pass has a scalar path
  return M >= 16;
}

int q4k_gemm(const char* op, const float* A, const uint8_t* W, void* C, int c_f16, int M, int N, int K,
             float alpha, const float* residual, const float* norm_weight, float norm_eps, int norm_weight_offset) {
  GemmArgs a{};
  a.A = A; a.W = W; a.W2 = nullptr; a.C = C; a.residual = residual;
  a.M = M; a.N = N; a.K = K; a.nb = (K + kQK - 1) / kQK;
  a.alpha = alpha; a.c_f16 = c_f16;
  a.norm_weight = norm_weight; a.norm_eps = norm_eps; a.norm_weight_offset = norm_weight_offset;
  return launch_gemm<false>(a, op);
}

int q4k_gemm_gate_up(const char* op, const float* A, const uint8_t* Wg, const uint8_t* Wu, float* C, int M,
                     int hidden, int inter, int activation, float alpha, float clamp_max,
                     const float* norm_weight, float norm_eps, int norm_weight_offset) {
  GemmArgs a{};
  a.A = A; a.W = Wg; a.W2 = Wu; a.C = C; a.residual = nullptr;
  a.M = M; a.N = inter; a.K = hidden; a.nb = (hidden + kQK - 1) / kQK;
  a.alpha = alpha; a.c_f16 = 0; a.activation = activation; a.clamp_max = clamp_max;
  a.norm_weight = norm_weight; a.norm_eps = norm_eps; a.norm_weight_offset = norm_weight_offset;
  return launch_gemm<true>(a, op);
}

}  // namespace dh
