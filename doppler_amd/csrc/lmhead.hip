// Dense f16-weight GEMV (the tied LM head), optionally fused with greedy argmax, and the
// stand-alone two-phase argmax over f32 logits.
//
// The LM head reads vocab*hidden*2 bytes per token (1.24 GB at 151936 x 4096): pure HBM
// streaming.  One wave per output row, 16 bytes (8 halves) per lane per step so a wave
// consumes 1 KB of the row per load instruction; activations sit in LDS as f32 and are
// read with conflict-free 16-byte accesses.  Argmax candidates (value, index) are reduced
// per wave, per workgroup, then across workgroups by a one-workgroup kernel; ties always go
// to the lower index, the rule of the reference's candidate_beats().
#include <algorithm>
#include <cfloat>

#include "dh_common.h"

namespace {

constexpr int kMaxParts = 2048;

struct Cand {
  float v;
  uint32_t i;
};

__device__ __forceinline__ bool beats(float cv, uint32_t ci, float bv, uint32_t bi) {
  if (cv > bv) return true;
  if (cv < bv) return false;
  return ci < bi;
}

__device__ __forceinline__ Cand wave_best(Cand c) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(c.v, off, 64);
    const uint32_t oi = __shfl_xor(c.i, off, 64);
    if (beats(ov, oi, c.v, c.i)) { c.v = ov; c.i = oi; }
  }
  return c;
}

// Workgroup-wide best of 256 threads; valid in thread 0.
__device__ __forceinline__ Cand block_best_256(Cand c, float* sv, uint32_t* si) {
  c = wave_best(c);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) { sv[wave] = c.v; si[wave] = c.i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; w++)
      if (beats(sv[w], si[w], c.v, c.i)) { c.v = sv[w]; c.i = si[w]; }
  }
  return c;
}

__device__ __forceinline__ float softcap_f(float x, float cap) {
  return cap > 0.f ? cap * tanhf(x / cap) : x;
}

struct F16GemvArgs {
  const float* A;      // [M][K]
  const __half* W;     // [N][K]
  float* C;            // [M][N] or null
  int N, K;
  float alpha;
  int rows_per_wave;
  // argmax (M == 1 only)
  float softcap;
  int64_t pad_id;
  float* part_val;
  uint32_t* part_idx;
  // RMSNorm of the activation row in the prologue (register kernel only; null = off)
  const float* norm_weight;
  float norm_eps;
  int norm_weight_offset;
};

// 16 bytes of a weight row, marked non-temporal.  Every row is read once per call, by one wave, as whole
// cache lines (a wave's load covers 1 KB of consecutive bytes): with the streaming hint the [151936 x 4096]
// f16 head is read at 6.6 TB/s against 5.9 TB/s with ordinary loads.  (The same hint on loads whose cache
// lines are shared between waves, the Q4_K units' 144-byte row pieces and the decode attention's K/V rows,
// made those kernels slower.)
__device__ __forceinline__ uint4 stream_load_16(const uint4* p) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(t[0], t[1], t[2], t[3]);
}

// M = 1, K <= 4096: every lane meets the same 64 activations in every row (its eight 16-byte
// chunks sit at fixed k), so they live in registers for the whole kernel; LDS only hands the row to
// the lanes once, at the start.
template <bool ARGMAX>
__global__ __launch_bounds__(256) void f16w_gemv_xreg_kernel(const F16GemvArgs a) {
  __shared__ float sv[4];
  __shared__ uint32_t si[4];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int kvec = a.K >> 3;
  // The activation row reaches the lanes through LDS: the workgroup loads it once (thread t takes the
  // 16-byte pieces t, t + 256, ..), and with a norm weight normalises it on the way, the same arithmetic
  // in the same order as the stand-alone RMSNorm launch (per-thread sums of squares over its pieces, wave
  // sums, the four waves added in order; (x * inv_rms) * w), so the fused call gives the bits of norm
  // launch + plain call.  Four waves loading the row each cost four times the traffic through the L2.
  __shared__ __align__(16) float xs[4096];
  __shared__ float red[4];
  // the wave's first weight row is requested before any of that, so that it travels meanwhile
  uint4 raw[8];
  {
    const int64_t row = (int64_t)blockIdx.x * 4 + wave;
    const uint4* wrow = reinterpret_cast<const uint4*>(a.W + min(row, (int64_t)a.N - 1) * a.K);
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const int v = lane + 64 * u;
      raw[u] = v < kvec ? stream_load_16(wrow + v) : make_uint4(0, 0, 0, 0);
    }
  }
  {
    const int nvec = a.K >> 2;
    float4 xv[4], wv[4];
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int iv = tid + 256 * j;
      xv[j] = make_float4(0.f, 0.f, 0.f, 0.f);
      wv[j] = make_float4(1.f, 1.f, 1.f, 1.f);
      if (iv < nvec) {
        xv[j] = reinterpret_cast<const float4*>(a.A)[iv];
        if (a.norm_weight != nullptr) wv[j] = reinterpret_cast<const float4*>(a.norm_weight)[iv];
      }
    }
    if (a.norm_weight != nullptr) {
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        ss = fmaf(xv[j].x, xv[j].x, ss); ss = fmaf(xv[j].y, xv[j].y, ss);
        ss = fmaf(xv[j].z, xv[j].z, ss); ss = fmaf(xv[j].w, xv[j].w, ss);
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      if (lane == 0) red[wave] = ss;
      __syncthreads();
      const float total = red[0] + red[1] + red[2] + red[3];
      const float inv = 1.0f / sqrtf(total / (float)a.K + a.norm_eps);
      const bool off = a.norm_weight_offset != 0;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        xv[j].x = xv[j].x * inv * (off ? 1.0f + wv[j].x : wv[j].x); xv[j].y = xv[j].y * inv * (off ? 1.0f + wv[j].y : wv[j].y);
        xv[j].z = xv[j].z * inv * (off ? 1.0f + wv[j].z : wv[j].z); xv[j].w = xv[j].w * inv * (off ? 1.0f + wv[j].w : wv[j].w);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; j++) reinterpret_cast<float4*>(xs)[tid + 256 * j] = xv[j];
    __syncthreads();
  }
  float x[8][8];
#pragma unroll
  for (int u = 0; u < 8; u++) {
    const int v = lane + 64 * u;     // v < 512: inside xs (pieces past K hold zeros)
    const float4 xa = reinterpret_cast<const float4*>(xs)[2 * v], xb = reinterpret_cast<const float4*>(xs)[2 * v + 1];
    x[u][0] = xa.x; x[u][1] = xa.y; x[u][2] = xa.z; x[u][3] = xa.w;
    x[u][4] = xb.x; x[u][5] = xb.y; x[u][6] = xb.z; x[u][7] = xb.w;
  }
  Cand best{-3.402823e+38f, 0xFFFFFFFFu};   // only lane 0 ever updates its candidate
  for (int r = 0; r < a.rows_per_wave; r++) {
    const int64_t row = ((int64_t)r * gridDim.x + blockIdx.x) * 4 + wave;
    if (row >= a.N) break;   // wave-uniform
    const uint4* wrow = reinterpret_cast<const uint4*>(a.W + row * a.K);
    if (r > 0) {
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int v = lane + 64 * u;
        raw[u] = v < kvec ? stream_load_16(wrow + v) : make_uint4(0, 0, 0, 0);
      }
    }
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int u = 0; u < 8; u++) {
      const __half2* h2 = reinterpret_cast<const __half2*>(&raw[u]);
      const float2 w0 = __half22float2(h2[0]), w1 = __half22float2(h2[1]);
      const float2 w2 = __half22float2(h2[2]), w3 = __half22float2(h2[3]);
      s0 = fmaf(x[u][0], w0.x, s0); s1 = fmaf(x[u][1], w0.y, s1);
      s0 = fmaf(x[u][2], w1.x, s0); s1 = fmaf(x[u][3], w1.y, s1);
      s0 = fmaf(x[u][4], w2.x, s0); s1 = fmaf(x[u][5], w2.y, s1);
      s0 = fmaf(x[u][6], w3.x, s0); s1 = fmaf(x[u][7], w3.y, s1);
    }
    const float logit = dh::wave_sum_uniform(s0 + s1) * a.alpha;
    if (lane == 0) {
      if (a.C) a.C[row] = logit;
      if (ARGMAX && row != a.pad_id) {
        const float v = softcap_f(logit, a.softcap);
        if (beats(v, (uint32_t)row, best.v, best.i)) { best.v = v; best.i = (uint32_t)row; }
      }
    }
  }
  if (ARGMAX) {
    const Cand c = block_best_256(best, sv, si);
    if (tid == 0) { a.part_val[blockIdx.x] = c.v; a.part_idx[blockIdx.x] = c.i; }
  }
}

template <int MT, bool ARGMAX>
__global__ __launch_bounds__(256) void f16w_gemv_kernel(const F16GemvArgs a) {
  extern __shared__ float xs[];   // [MT][K]
  __shared__ float sv[4];
  __shared__ uint32_t si[4];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  for (int i = tid; i < MT * a.K; i += 256) xs[i] = a.A[i];
  __syncthreads();

  const int kvec = a.K >> 3;
  // rows are dealt round-robin over all waves of the grid: at any moment the whole chip reads
  // one contiguous band of the matrix, which keeps every HBM channel busy
  Cand best{-3.402823e+38f, 0xFFFFFFFFu};   // only lane 0 ever updates its candidate
  for (int r = 0; r < a.rows_per_wave; r++) {
    const int64_t row = ((int64_t)r * gridDim.x + blockIdx.x) * 4 + wave;
    if (row >= a.N) break;   // wave-uniform
    const uint4* wrow = reinterpret_cast<const uint4*>(a.W + row * a.K);
    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; m++) acc[m] = 0.f;
    // eight 16-byte loads per lane go out before any of them is used (4 KB of the row per wave)
    for (int v0 = lane; v0 < kvec; v0 += 8 * 64) {
      uint4 raw[8];
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int v = v0 + 64 * u;
        raw[u] = v < kvec ? stream_load_16(wrow + v) : make_uint4(0, 0, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < 8; u++) {
        const int v = min(v0 + 64 * u, kvec - 1);      // zero weights past the row: any x will do
        const __half2* h2 = reinterpret_cast<const __half2*>(&raw[u]);
        const float2 w0 = __half22float2(h2[0]), w1 = __half22float2(h2[1]);
        const float2 w2 = __half22float2(h2[2]), w3 = __half22float2(h2[3]);
#pragma unroll
        for (int m = 0; m < MT; m++) {
          const float4 xa = *reinterpret_cast<const float4*>(xs + m * a.K + v * 8);
          const float4 xb = *reinterpret_cast<const float4*>(xs + m * a.K + v * 8 + 4);
          float s = acc[m];
          s = fmaf(xa.x, w0.x, s); s = fmaf(xa.y, w0.y, s);
          s = fmaf(xa.z, w1.x, s); s = fmaf(xa.w, w1.y, s);
          s = fmaf(xb.x, w2.x, s); s = fmaf(xb.y, w2.y, s);
          s = fmaf(xb.z, w3.x, s); s = fmaf(xb.w, w3.y, s);
          acc[m] = s;
        }
      }
    }
#pragma unroll
    for (int m = 0; m < MT; m++) {
      acc[m] = dh::wave_sum_uniform(acc[m]) * a.alpha;
    }
    if (lane == 0) {
      if (a.C) {
#pragma unroll
        for (int m = 0; m < MT; m++) a.C[(int64_t)m * a.N + row] = acc[m];
      }
      if (ARGMAX && row != a.pad_id) {
        const float v = softcap_f(acc[0], a.softcap);
        if (beats(v, (uint32_t)row, best.v, best.i)) { best.v = v; best.i = (uint32_t)row; }
      }
    }
  }
  if (ARGMAX) {
    const Cand c = block_best_256(best, sv, si);
    if (tid == 0) { a.part_val[blockIdx.x] = c.v; a.part_idx[blockIdx.x] = c.i; }
  }
}

// Phase 1 of the stand-alone argmax: grid-stride scan of f32 logits.
__global__ __launch_bounds__(256) void argmax_scan_kernel(const float* __restrict__ logits, int vocab,
                                                          int64_t pad_id, float softcap,
                                                          float* __restrict__ part_val,
                                                          uint32_t* __restrict__ part_idx) {
  __shared__ float sv[4];
  __shared__ uint32_t si[4];
  Cand best{-3.402823e+38f, 0xFFFFFFFFu};
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < vocab; i += (int64_t)gridDim.x * 256) {
    if (i == pad_id) continue;
    const float v = softcap_f(logits[i], softcap);
    if (beats(v, (uint32_t)i, best.v, best.i)) { best.v = v; best.i = (uint32_t)i; }
  }
  const Cand c = block_best_256(best, sv, si);
  if (threadIdx.x == 0) { part_val[blockIdx.x] = c.v; part_idx[blockIdx.x] = c.i; }
}

// Phase 2: one workgroup folds the per-workgroup candidates and writes the token.
__global__ __launch_bounds__(256) void argmax_final_kernel(const float* __restrict__ part_val,
                                                           const uint32_t* __restrict__ part_idx, int parts,
                                                           uint32_t* __restrict__ token_out, int out_index) {
  __shared__ float sv[4];
  __shared__ uint32_t si[4];
  Cand best{-3.402823e+38f, 0xFFFFFFFFu};
  for (int i = threadIdx.x; i < parts; i += 256)
    if (beats(part_val[i], part_idx[i], best.v, best.i)) { best.v = part_val[i]; best.i = part_idx[i]; }
  const Cand c = block_best_256(best, sv, si);
  // nothing beat the neutral start (every logit <= -3.4e38, NaN, or masked): index 0, as the
  // reference kernel's (NEG_INF, 0) start does
  if (threadIdx.x == 0) token_out[out_index] = c.i == 0xFFFFFFFFu ? 0u : c.i;
}

template <int MT, bool ARGMAX>
int launch_gemv(F16GemvArgs a, int* parts_out, const char* op) {
  const size_t lds = (size_t)MT * a.K * sizeof(float);
  auto kern = f16w_gemv_kernel<MT, ARGMAX>;
  static bool attr_set = false;   // once per instantiation: the call costs microseconds
  if (!attr_set) {
    DH_CHECK_HIP(op, hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024));
    attr_set = true;
  }
  // ~1024 workgroups when N allows (4 per CU), never more than kMaxParts partial candidates
  int rpw = (int)std::max<int64_t>(1, dh::ceil_div(a.N, (int64_t)4 * 1024));
  int grid = (int)dh::ceil_div(a.N, (int64_t)4 * rpw);
  while (grid > kMaxParts) { rpw++; grid = (int)dh::ceil_div(a.N, (int64_t)4 * rpw); }
  a.rows_per_wave = rpw;
  if (MT == 1 && a.K <= 4096 && (reinterpret_cast<uintptr_t>(a.A) & 15) == 0)
    hipLaunchKernelGGL(f16w_gemv_xreg_kernel<ARGMAX>, dim3(grid), dim3(256), 0, dh::stream(), a);
  else
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  if (parts_out) *parts_out = grid;
  return 0;
}

int check_f16w_shape(const char* op, int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0) return dh::fail(1, "[%s] Dimensions must be positive: M=%d, N=%d, K=%d", op, M, N, K);
  if (K % 8) return dh::fail(1, "[%s] K=%d must be a multiple of 8 for f16 weights", op, K);
  if ((size_t)K * sizeof(float) > 128 * 1024) return dh::fail(1, "[%s] K=%d too large (max 32768)", op, K);
  return 0;
}

}  // namespace

extern "C" {

int dh_f16w_matmul(const float* d_A, const void* d_W, float* d_C, int M, int N, int K, float alpha) {
  const char* op = "dh_f16w_matmul";
  DH_REQUIRE_INIT(op);
  if (int rc = check_f16w_shape(op, M, N, K)) return rc;
  if (!d_A || !d_W || !d_C) return dh::fail(1, "[%s] null pointer", op);
  if (reinterpret_cast<uintptr_t>(d_W) & 15) return dh::fail(1, "[%s] weight pointer must be 16-byte aligned", op);
  int mt = std::min(M, 4);
  while (mt > 1 && (size_t)mt * K * sizeof(float) > 128 * 1024) mt--;
  for (int m0 = 0; m0 < M; m0 += mt) {
    F16GemvArgs a{};
    const int cur = std::min(mt, M - m0);
    a.A = d_A + (int64_t)m0 * K;
    a.W = static_cast<const __half*>(d_W);
    a.C = d_C + (int64_t)m0 * N;
    a.N = N; a.K = K; a.alpha = alpha;
    int rc;
    switch (cur) {
      case 1: rc = launch_gemv<1, false>(a, nullptr, op); break;
      case 2: rc = launch_gemv<2, false>(a, nullptr, op); break;
      case 3: rc = launch_gemv<3, false>(a, nullptr, op); break;
      default: rc = launch_gemv<4, false>(a, nullptr, op); break;
    }
    if (rc) return rc;
  }
  return 0;
}

size_t dh_lmhead_argmax_workspace_bytes(int vocab) {
  (void)vocab;
  return (size_t)kMaxParts * 8;
}

static int lmhead_argmax_impl(const char* op, const float* d_h, const float* d_norm_weight, float eps, int weight_offset,
                              const void* d_E, int vocab, int hidden, int64_t pad_token_id, float logit_softcap,
                              void* d_workspace, uint32_t* d_token_out, int output_index, float* d_logits_out) {
  DH_REQUIRE_INIT(op);
  if (int rc = check_f16w_shape(op, 1, vocab, hidden)) return rc;
  if (!d_h || !d_E || !d_workspace || !d_token_out) return dh::fail(1, "[%s] null pointer", op);
  if (output_index < 0) return dh::fail(1, "[%s] outputIndex must be non-negative", op);
  if (reinterpret_cast<uintptr_t>(d_E) & 15) return dh::fail(1, "[%s] weight pointer must be 16-byte aligned", op);
  if (d_norm_weight) {
    // the norm runs on the row in registers: only the kernel that keeps it there serves it
    if (hidden > 4096 || (reinterpret_cast<uintptr_t>(d_h) & 15) || (reinterpret_cast<uintptr_t>(d_norm_weight) & 15))
      return dh::fail(1, "[%s] the RMSNorm prologue is served for hidden <= 4096 and 16-byte aligned rows (hidden=%d): "
                         "run dh_rmsnorm in front of dh_lmhead_argmax_f16 instead", op, hidden);
    if (!(eps >= 0.f)) return dh::fail(1, "[%s] eps must be non-negative", op);
  }
  F16GemvArgs a{};
  a.A = d_h; a.W = static_cast<const __half*>(d_E); a.C = d_logits_out;
  a.N = vocab; a.K = hidden; a.alpha = 1.0f;
  a.softcap = logit_softcap; a.pad_id = pad_token_id;
  a.part_val = static_cast<float*>(d_workspace);
  a.part_idx = reinterpret_cast<uint32_t*>(static_cast<char*>(d_workspace) + (size_t)kMaxParts * 4);
  a.norm_weight = d_norm_weight; a.norm_eps = eps; a.norm_weight_offset = weight_offset;
  int parts = 0;
  if (int rc = launch_gemv<1, true>(a, &parts, op)) return rc;
  hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(256), 0, dh::stream(), a.part_val, a.part_idx, parts,
                     d_token_out, output_index);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_lmhead_argmax_f16(const float* d_h, const void* d_E, int vocab, int hidden, int64_t pad_token_id,
                         float logit_softcap, void* d_workspace, uint32_t* d_token_out, int output_index,
                         float* d_logits_out) {
  return lmhead_argmax_impl("dh_lmhead_argmax_f16", d_h, nullptr, 0.f, 0, d_E, vocab, hidden, pad_token_id, logit_softcap,
                            d_workspace, d_token_out, output_index, d_logits_out);
}

int dh_lmhead_argmax_f16_rmsnorm(const float* d_h, const float* d_norm_weight, float eps, int weight_offset,
                                 const void* d_E, int vocab, int hidden, int64_t pad_token_id, float logit_softcap,
                                 void* d_workspace, uint32_t* d_token_out, int output_index, float* d_logits_out) {
  const char* op = "dh_lmhead_argmax_f16_rmsnorm";
  if (!d_norm_weight) return dh::fail(1, "[%s] null norm weight", op);
  return lmhead_argmax_impl(op, d_h, d_norm_weight, eps, weight_offset, d_E, vocab, hidden, pad_token_id, logit_softcap,
                            d_workspace, d_token_out, output_index, d_logits_out);
}

size_t dh_argmax_workspace_bytes(void) { return (size_t)kMaxParts * 8; }

int dh_argmax(const float* d_logits, int vocab, int64_t pad_token_id, float logit_softcap, void* d_workspace,
              uint32_t* d_token_out, int output_index) {
  const char* op = "dh_argmax";
  DH_REQUIRE_INIT(op);
  if (vocab <= 0) return dh::fail(1, "[%s] vocabSize must be positive, got %d", op, vocab);
  if (!d_logits || !d_workspace || !d_token_out) return dh::fail(1, "[%s] null pointer", op);
  if (output_index < 0) return dh::fail(1, "[%s] outputIndex must be non-negative", op);
  float* pv = static_cast<float*>(d_workspace);
  uint32_t* pi = reinterpret_cast<uint32_t*>(static_cast<char*>(d_workspace) + (size_t)kMaxParts * 4);
  const int parts = (int)std::min<int64_t>(256, dh::ceil_div(vocab, 256));
  hipLaunchKernelGGL(argmax_scan_kernel, dim3(parts), dim3(256), 0, dh::stream(), d_logits, vocab, pad_token_id,
                     logit_softcap, pv, pi);
  DH_CHECK_LAUNCH(op);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(1), dim3(256), 0, dh::stream(), pv, pi, parts, d_token_out,
                     output_index);
  DH_CHECK_LAUNCH(op);
  return 0;
}

}  // extern "C"
