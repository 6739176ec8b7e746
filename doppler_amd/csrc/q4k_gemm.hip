// Q4_K prefill GEMM for gfx950: C[M,N] = alpha * A[M,K] . dequant(W)[N,K]^T for M >= 16, and
// the fused gate/up projection with gated activation, on the matrix cores.
//
// Tile: 128 (M) x 128 (N) per workgroup of 4 waves, each wave a 64 x 64 quadrant computed with
// v_mfma_f32_32x32x16_f16 (2 x 2 MFMA tiles, f32 accumulators).  K advances 64 at a time: one
// 32-byte nibble chunk of a super-block (low nibbles = sub-block 2c, high = 2c+1) per weight row.
//   weights  thread (row, half) loads 16 nibble bytes + the block header, rebuilds 32 weights
//            as f16: (w & 0x000F000F) | 0x64006400 is the pair (1024 + q) in f16, one packed
//            subtract and one packed fma with (d*sc, -dmin*mn) finish them: about 2 vector ops
//            per weight, paid once per 128 rows of A.
//   A        packed once per product by a pre-pass (pack_a_row_kernel / pack_a_kernel): each row scaled by the power
//            of two that puts its largest element at 2^14, rounded to f16, k-permuted, rows
//            zero-padded to a multiple of 64.  The GEMM tiles then copy 16-byte pieces into
//            LDS, no conversion in the K loop (every column tile used to redo it), and the
//            epilogue divides the row factor out again, exactly: activations beyond the f16
//            range (65504) neither overflow nor lose small rows to subnormals.
// Both tiles sit in LDS as [row][64 k] with a 16-byte pad (conflict-free 16-byte fragment
// reads) and are double-buffered, one barrier per K step.
// SPEC (used where only one workgroup fits a compute unit, the fused gate/up tile): the
// workgroup has eight waves, waves 0..3 only multiply (fragment reads + matrix-core
// instructions), waves 4..7 only produce (global loads two tiles ahead, dequantise, write the
// next LDS buffer).  Each SIMD then holds one wave of either kind, so the vector ALU work of the
// dequantisation runs under the matrix-core work instead of in front of it; with all waves doing
// both in turn (one barrier per step keeps them in phase) the two never overlap.  Where two or
// more four-wave workgroups share a compute unit they overlap each other and that is faster.
// A 256 (M) x 128 (N) tile with the same split (two A tiles against one weight tile, half the
// dequantisation per output) was measured too: 368 against 326 us at M = 2048, N = 12288,
// K = 4096; one workgroup of it per compute unit loses to two 128 x 128 workgroups.
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

int env_ksplit() {
  const char* e = getenv("DH_GEMM_KSPLIT");
  return e ? atoi(e) : 0;
}

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

// 16 nibble bytes -> 16 low-nibble and 16 high-nibble weights as f16, k order (0,2,1,3) per dword.
__device__ __forceinline__ void dequant16(const uint4 q, float sc_lo, float mn_lo, float sc_hi, float mn_hi,
                                          uint4 (&lo)[2], uint4 (&hi)[2]) {
  const uint32_t w[4] = {q.x, q.y, q.z, q.w};
  const half2_t k1024 = {(_Float16)1024.f, (_Float16)1024.f};
  const half2_t slo = {(_Float16)sc_lo, (_Float16)sc_lo}, mlo = {(_Float16)-mn_lo, (_Float16)-mn_lo};
  const half2_t shi = {(_Float16)sc_hi, (_Float16)sc_hi}, mhi = {(_Float16)-mn_hi, (_Float16)-mn_hi};
  uint32_t lo_w[8], hi_w[8];
#pragma unroll
  for (int d = 0; d < 4; d++) {
    const uint32_t p[4] = {(w[d] & 0x000F000Fu) | 0x64006400u, ((w[d] >> 8) & 0x000F000Fu) | 0x64006400u,
                           ((w[d] >> 4) & 0x000F000Fu) | 0x64006400u, ((w[d] >> 12) & 0x000F000Fu) | 0x64006400u};
    half2_t v[4];
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = __builtin_bit_cast(half2_t, p[i]) - k1024;     // exact: q
    lo_w[2 * d] = __builtin_bit_cast(uint32_t, v[0] * slo + mlo);
    lo_w[2 * d + 1] = __builtin_bit_cast(uint32_t, v[1] * slo + mlo);
    hi_w[2 * d] = __builtin_bit_cast(uint32_t, v[2] * shi + mhi);
    hi_w[2 * d + 1] = __builtin_bit_cast(uint32_t, v[3] * shi + mhi);
  }
  lo[0] = make_uint4(lo_w[0], lo_w[1], lo_w[2], lo_w[3]);
  lo[1] = make_uint4(lo_w[4], lo_w[5], lo_w[6], lo_w[7]);
  hi[0] = make_uint4(hi_w[0], hi_w[1], hi_w[2], hi_w[3]);
  hi[1] = make_uint4(hi_w[4], hi_w[5], hi_w[6], hi_w[7]);
}

// tanh-form GELU with tanh(t) = 1 - 2 / (1 + e^{2t}): a handful of instructions, inlined once per
// accumulator element in the epilogue.
__device__ __forceinline__ float gelu_tanh_fast(float x) {
  const float t = fminf(fmaxf(0.7978845608f * (x + 0.044715f * x * x * x), -15.0f), 15.0f);
  return 0.5f * x * (2.0f - 2.0f / (1.0f + __expf(2.0f * t)));
}

#ifdef DH_GEMM_TRACE
__device__ unsigned long long dh_gemm_trace_buf[8 * 128];
#define DH_GTS() do { if (lane == 0 && blockIdx.x == 1 && blockIdx.y == 1 && blockIdx.z == 0 && tsn < 127) \
                        dh_gemm_trace_buf[wave * 128 + tsn++] = wall_clock64(); } while (0)
#else
#define DH_GTS() do {} while (0)
#endif

// T = MFMA tiles per wave along each of M and N: workgroup tile 64T x 64T (T = 2: 128 x 128 for
// large problems, T = 1: 64 x 64 when a 128-tiling would leave most compute units idle).
template <bool DUAL, int T, bool SPEC>
__global__ __launch_bounds__(SPEC ? 512 : 256) void q4k_gemm_kernel(const GemmArgs a) {
  constexpr int NMAT = DUAL ? 2 : 1;
  constexpr int BM = 64 * T, BN = 64 * T;
  constexpr int A_HALVES = BM * LDS_ROW, B_HALVES = BN * LDS_ROW;
  extern __shared__ __align__(16) _Float16 lds[];            // [2 buffers][A | B | (B2)]
  constexpr int BUF_HALVES = A_HALVES + NMAT * B_HALVES;

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const bool producer = !SPEC || wave >= 4, multiplier = !SPEC || wave < 4;
  const int tid = threadIdx.x & 255;            // index inside the role's 256 threads
#ifdef DH_GEMM_TRACE
  int tsn = 0;
#endif
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int wm = (wave >> 1) * 32 * T, wn = (wave & 1) * 32 * T;     // the wave's quadrant
  const int fr = lane & 31, fg = lane >> 5;                  // fragment row / k half
  const int64_t row_bytes = (int64_t)a.nb * kBlockBytes;
  const int kt0 = a.ksplit > 1 ? (int)blockIdx.z * a.kt_per_split : 0;
  const int nkt = a.ksplit > 1 ? min((a.K + BK - 1) / BK, kt0 + a.kt_per_split) : (a.K + BK - 1) / BK;

  // ---- global -> register staging roles
  // A: 16-byte pieces of the packed rows, idx = tid + 256 i: row idx >> 3, halves 8 * (idx & 7)
  // W: thread (row tid >> 1, half tid & 1): 16 nibble bytes + header
  const int w_row = tid >> 1, w_half = tid & 1;
  const int64_t w_off = (int64_t)min(n0 + w_row, a.N - 1) * row_bytes;
  constexpr int NA = BM * 8 / 256;                           // 16-byte loads of A per thread
  const bool w_active = w_row < BN;
  // Two register sets: while tile kt is multiplied, tile kt+1 waits in one set and the loads of
  // tile kt+2 are in flight into the other, so a load has two K steps to arrive.
  struct Staged {
    u32x4_t a[NA];
    u32x4_t q[NMAT], h[NMAT];
  };
  Staged st0, st1;
  // row factors of this tile's activation rows: one global read each, then LDS
  __shared__ float2 rs_lds[BM];
  if (threadIdx.x < BM) rs_lds[threadIdx.x] = a.row_scale[min(m0 + (int)threadIdx.x, a.M - 1)];

  auto load_tile = [&](int kt, Staged& st) {
#pragma unroll
    for (int i = 0; i < NA; i++) {
      const int idx = tid + 256 * i, r = idx >> 3;
      const int m = min(m0 + r, a.M - 1);
      st.a[i] = *reinterpret_cast<const u32x4_t*>(a.Apk + (int64_t)m * a.kpad + kt * BK + 8 * (idx & 7));
    }
    const int blk = kt >> 2, c = kt & 3;
#pragma unroll
    for (int mt = 0; mt < NMAT; mt++) {
      if (w_active) {
        const uint8_t* bp = (mt ? a.W2 : a.W) + w_off + (int64_t)blk * kBlockBytes;
        st.h[mt] = *reinterpret_cast<const u32x4_t*>(bp);
        st.q[mt] = *reinterpret_cast<const u32x4_t*>(bp + 16 + 32 * c + 16 * w_half);
      }
    }
  };
  auto store_tile = [&](int kt, int buf, const Staged& st) {
    _Float16* At = lds + buf * BUF_HALVES;
#pragma unroll
    for (int i = 0; i < NA; i++) {
      const int idx = tid + 256 * i, r = idx >> 3;
      *reinterpret_cast<u32x4_t*>(At + r * LDS_ROW + 8 * (idx & 7)) = st.a[i];
    }
    const int c = kt & 3;
#pragma unroll
    for (int mt = 0; mt < NMAT; mt++) {
      if (!w_active) break;
      float sc_lo, sc_hi, mn_lo, mn_hi;
      const uint4 hdr = make_uint4(st.h[mt][0], st.h[mt][1], st.h[mt][2], st.h[mt][3]);
      const uint4 qv = make_uint4(st.q[mt][0], st.q[mt][1], st.q[mt][2], st.q[mt][3]);
      q4k_pair_scales(hdr, c, sc_lo, sc_hi, mn_lo, mn_hi);
      uint4 lo[2], hi[2];
      dequant16(qv, sc_lo, mn_lo, sc_hi, mn_hi, lo, hi);
      _Float16* Bt = lds + buf * BUF_HALVES + A_HALVES + mt * B_HALVES + w_row * LDS_ROW;
      *reinterpret_cast<uint4*>(Bt + 16 * w_half) = lo[0];
      *reinterpret_cast<uint4*>(Bt + 16 * w_half + 8) = lo[1];
      *reinterpret_cast<uint4*>(Bt + 32 + 16 * w_half) = hi[0];
      *reinterpret_cast<uint4*>(Bt + 32 + 16 * w_half + 8) = hi[1];
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

  // One K step.  Multipliers: the tile in LDS buffer kt & 1.  Producers: move tile kt+1 from `nxt`
  // into the other buffer and start the loads of tile kt+3 into `nxt`.
  auto k_step = [&](int kt, Staged& nxt) {
    DH_GTS();
    const int buf = kt & 1;
    const _Float16* At = lds + buf * BUF_HALVES;
    if (multiplier) {
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      half8_t af[T], bf[NMAT][T];
#pragma unroll
      for (int i = 0; i < T; i++)
        af[i] = *reinterpret_cast<const half8_t*>(At + (wm + 32 * i + fr) * LDS_ROW + 16 * ks + 8 * fg);
#pragma unroll
      for (int mt = 0; mt < NMAT; mt++)
#pragma unroll
        for (int j = 0; j < T; j++)
          bf[mt][j] = *reinterpret_cast<const half8_t*>(At + A_HALVES + mt * B_HALVES + (wn + 32 * j + fr) * LDS_ROW +
                                                        16 * ks + 8 * fg);
#pragma unroll
      for (int mt = 0; mt < NMAT; mt++)
#pragma unroll
        for (int i = 0; i < T; i++)
#pragma unroll
          for (int j = 0; j < T; j++)
            // accumulators pinned to the accumulation registers: left to itself the compiler keeps
            // them in vector registers and copies all of them aside and back every K step
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[mt][i][j]) : "v"(af[i]), "v"(bf[mt][j]));
    }
    }
    DH_GTS();
    if (producer) {
      if (kt + 1 < nkt) store_tile(kt + 1, buf ^ 1, nxt);
      if (kt + 3 < nkt) load_tile(kt + 3, nxt);
    }
    __syncthreads();
  };

  if (producer) {
    load_tile(kt0, st0);
    store_tile(kt0, kt0 & 1, st0);
    if (kt0 + 1 < nkt) load_tile(kt0 + 1, st0);
    if (kt0 + 2 < nkt) load_tile(kt0 + 2, st1);
  }
  __syncthreads();
  for (int kt = kt0; kt < nkt; kt += 2) {
    k_step(kt, st0);
    if (kt + 1 < nkt) k_step(kt + 1, st1);
  }

  DH_GTS();
#ifdef DH_GEMM_TRACE
  if (lane == 0 && blockIdx.x == 1 && blockIdx.y == 1 && blockIdx.z == 0) dh_gemm_trace_buf[wave * 128 + 127] = tsn;
#endif
  if (!multiplier) return;
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
        const int m = m0 + wm + 32 * i + 8 * (e >> 2) + 4 * fg + (e & 3);
        if (m < a.M && n < a.N) {
          float v;
          const float unscale = rs_lds[wm + 32 * i + 8 * (e >> 2) + 4 * fg + (e & 3)].y;
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

// C = alpha * (sum of the split-K pieces, in split order) + residual.
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const GemmArgs a) {
  const int64_t total = (int64_t)a.M * a.N;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  float s = 0.f;
  for (int z = 0; z < a.ksplit; z++) s += a.partial[(int64_t)z * total + i];
  float v = s * a.alpha;
  if (a.residual) v += a.residual[i];
  if (a.c_f16)
    reinterpret_cast<__half*>(a.C)[i] = __float2half(v);
  else
    reinterpret_cast<float*>(a.C)[i] = v;
}

template <bool DUAL, int T>
int launch_gemm_cfg(const GemmArgs& a, const char* op) {
  constexpr bool SPEC = DUAL && T == 2;      // 110 KB of LDS: one workgroup per compute unit
  constexpr int BM = 64 * T, BN = 64 * T;
  const size_t lds = (size_t)2 * (DUAL ? 3 : 2) * BM * LDS_ROW * sizeof(_Float16);
  auto kern = q4k_gemm_kernel<DUAL, T, SPEC>;
  static bool attr_set = false;   // once per instantiation: the call costs microseconds
  if (!attr_set) {
    DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
    attr_set = true;
  }
  const dim3 grid((unsigned)dh::ceil_div(a.N, BN), (unsigned)dh::ceil_div(a.M, BM), (unsigned)std::max(1, a.ksplit));
  hipLaunchKernelGGL(kern, grid, dim3(SPEC ? 512 : 256), lds, dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  if (a.ksplit > 1) {
    const int64_t total = (int64_t)a.M * a.N;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned)dh::ceil_div(total, 256)), dim3(256), 0, dh::stream(), a);
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
  const int64_t big_tiles = dh::ceil_div(a.M, 128) * dh::ceil_div(a.N, 128);
  a.ksplit = 1;
  if (2 * big_tiles >= dh::num_cus()) return launch_gemm_cfg<DUAL, 2>(a, op);
  // Few tiles and a long K: every workgroup would walk K alone at one memory round trip per
  // step.  Cut K so that about three workgroups share a compute unit and overlap each other's
  // waits; the pieces meet in the library's scratch buffer.
  if (!DUAL) {
    static const int env_split = env_ksplit();
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
  return launch_gemm_cfg<DUAL, 1>(a, op);
}

}  // namespace

#ifdef DH_GEMM_TRACE
extern "C" int dh_debug_gemm_trace(void* host_dst) {
  return (int)hipMemcpyFromSymbol(host_dst, HIP_SYMBOL(dh_gemm_trace_buf), sizeof(dh_gemm_trace_buf));
}
#endif

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
