// Top-k temperature sampling over f32 logits: exact top-k (ties to the lower index), softmax of
// value / temperature over the k candidates in f64, inverse-CDF pick with a caller-supplied
// uniform number.  Follows the reference's sampler oracle, tests/kernels/reference/sample.js:62-92,
// with the kernel's extras (soft cap, pad id) of src/gpu/kernels/sample.wgsl:35-51.
//
// Selection is a tournament of 1024-element bitonic sorts (registers + lane shuffles, LDS only
// for the widest exchanges): round 0 sorts slices of the vocabulary and keeps the best k of
// each, later rounds sort 1024 surviving candidates at a time, until one workgroup holds them
// all; that workgroup also draws the token.  k <= 256, so a round shrinks the field at least
// four-fold.  A round costs ~16 us whatever its grid: the 55 dependent exchange steps of the
// network set its length (3 rounds at k = 40 over 151,936 logits, 5 at k = 256); as a rolled
// loop with run-time distances it cost 25.
#include <algorithm>
#include <cfloat>

#include "dh_common.h"

namespace {

constexpr int kSortN = 1024;
constexpr int kMaxTopK = 256;

struct SampleArgs {
  const float* logits;      // round 0 input (vocab entries), else null
  const float* in_val;      // later rounds: candidate values / ids
  const uint32_t* in_idx;
  int n_in;                 // entries of the input
  int top_k;
  float* out_val;           // [groups][top_k]
  uint32_t* out_idx;
  int64_t pad_id;
  float softcap;
  double temperature, random_value;
  uint32_t* token_out;      // written by the last round (one workgroup)
  int output_index;
};

// a ranks before b: larger value first, lower id among equals
__device__ __forceinline__ bool ranks_before(float av, uint32_t ai, float bv, uint32_t bi) {
  return av > bv || (av == bv && ai < bi);
}

// Value of lane (l ^ dist).  The network below is fully unrolled, so dist is a constant where this
// is called: partners inside a quad and 8 lanes apart come through the DPP path of the vector ALU
// (quad_perm, row_ror:8), the rest through the LDS crossbar.
__device__ __forceinline__ uint32_t lane_xor(uint32_t x, int dist) {
  if (dist == 1) return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0xB1, 0xF, 0xF, false);
  if (dist == 2) return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x4E, 0xF, 0xF, false);
  if (dist == 8) return (uint32_t)__builtin_amdgcn_update_dpp((int)x, (int)x, 0x128, 0xF, 0xF, false);
  return (uint32_t)__shfl_xor((int)x, dist, 64);
}

// Sorts 1024 (value, id) pairs best first, four per thread: element i = 4 * tid + r.  A bitonic
// network; exchanges at distance 1 and 2 stay inside a thread's registers, distances 4..128 are
// lane shuffles inside a wave, only the three steps at distance 256 and 512 go through LDS and
// a barrier.
__device__ __forceinline__ void sort1024(float (&v)[4], uint32_t (&id)[4], float* s_val, uint32_t* s_idx, int tid) {
#pragma unroll
  for (int k = 2; k <= kSortN; k <<= 1) {
#pragma unroll
    for (int j = k >> 1; j > 0; j >>= 1) {
      if (j >= 4) {
        float pv[4];
        uint32_t pi[4];
        if (j >= 256) {
          __syncthreads();
#pragma unroll
          for (int r = 0; r < 4; r++) { s_val[4 * tid + r] = v[r]; s_idx[4 * tid + r] = id[r]; }
          __syncthreads();
#pragma unroll
          for (int r = 0; r < 4; r++) { pv[r] = s_val[(4 * tid + r) ^ j]; pi[r] = s_idx[(4 * tid + r) ^ j]; }
        } else {
#pragma unroll
          for (int r = 0; r < 4; r++) {
            pv[r] = __uint_as_float(lane_xor(__float_as_uint(v[r]), j >> 2));
            pi[r] = lane_xor(id[r], j >> 2);
          }
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const int i = 4 * tid + r;
          const bool keep_better = ((i & j) == 0) == ((i & k) == 0);
          const bool partner_better = ranks_before(pv[r], pi[r], v[r], id[r]);
          if (partner_better == keep_better) { v[r] = pv[r]; id[r] = pi[r]; }
        }
      } else {
        // pairs (r, r + j) inside the thread: j = 2 -> (0,2) (1,3); j = 1 -> (0,1) (2,3)
#pragma unroll
        for (int p = 0; p < 2; p++) {
          const int lo = j == 2 ? p : 2 * p, hi = lo + j;
          const bool best_first = ((4 * tid + lo) & k) == 0;
          float av = v[0], bv = v[0];
          uint32_t ai = id[0], bi = id[0];
#pragma unroll
          for (int r = 0; r < 4; r++) {
            if (r == lo) { av = v[r]; ai = id[r]; }
            if (r == hi) { bv = v[r]; bi = id[r]; }
          }
          const bool swap = best_first ? ranks_before(bv, bi, av, ai) : ranks_before(av, ai, bv, bi);
#pragma unroll
          for (int r = 0; r < 4; r++) {
            if (swap && r == lo) { v[r] = bv; id[r] = bi; }
            if (swap && r == hi) { v[r] = av; id[r] = ai; }
          }
        }
      }
    }
  }
}

__global__ __launch_bounds__(256) void topk_round_kernel(const SampleArgs a) {
  __shared__ float val[kSortN];
  __shared__ uint32_t idx[kSortN];
  __shared__ double prob[kMaxTopK];
  const int tid = threadIdx.x;
  const int base = blockIdx.x * kSortN;
  float v[4];
  uint32_t id[4];
#pragma unroll
  for (int r = 0; r < 4; r++) {
    const int g = base + 4 * tid + r;
    v[r] = -INFINITY;                         // padding never ranks before a real entry
    id[r] = 0xFFFFFFFFu;
    if (g < a.n_in) {
      if (a.logits) {
        float x = a.logits[g];
        if (a.softcap > 0.f) x = a.softcap * tanhf(x / a.softcap);
        if ((int64_t)g != a.pad_id && x == x) { v[r] = x; id[r] = (uint32_t)g; }   // pad id, NaN: out
      } else {
        v[r] = a.in_val[g];
        id[r] = a.in_idx[g];
      }
    }
  }
  sort1024(v, id, val, idx, tid);
  if (gridDim.x > 1) {
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int i = 4 * tid + r;
      if (i < a.top_k) {
        a.out_val[blockIdx.x * a.top_k + i] = v[r];
        a.out_idx[blockIdx.x * a.top_k + i] = id[r];
      }
    }
    return;
  }
  // ---- the field is down to one workgroup: softmax over the candidates and the draw
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 4; r++) { val[4 * tid + r] = v[r]; idx[4 * tid + r] = id[r]; }
  __syncthreads();
  int n = min(a.top_k, a.n_in);
  while (n > 0 && idx[n - 1] == 0xFFFFFFFFu) n--;               // padding / excluded entries
  const double mx = n > 0 ? (double)val[0] / a.temperature : 0.0;
  for (int i = tid; i < n; i += 256) prob[i] = exp((double)val[i] / a.temperature - mx);
  __syncthreads();
  if (tid == 0) {
    double sum = 0.0;
    for (int i = 0; i < n; i++) sum += prob[i];
    uint32_t pick = n > 0 ? idx[n - 1] : 0u;
    double cum = 0.0;
    for (int i = 0; i < n; i++) {
      cum += prob[i] / sum;
      if (cum >= a.random_value) { pick = idx[i]; break; }
    }
    a.token_out[a.output_index] = pick;
  }
}

int groups_of(int n) { return (n + kSortN - 1) / kSortN; }

}  // namespace

extern "C" {

size_t dh_sample_topk_workspace_bytes(int vocab, int top_k) {
  if (vocab <= 0 || top_k <= 0) return 256;
  const size_t first = (size_t)groups_of(vocab) * (size_t)std::min(top_k, kMaxTopK);
  // two ping-pong candidate lists (values + ids); the second round's output is at most a quarter
  return std::max<size_t>(256, 2 * first * 8);
}

int dh_sample_topk(const float* d_logits, int vocab, double temperature, int top_k, double random_value,
                   int64_t pad_token_id, float logit_softcap, void* d_workspace, uint32_t* d_token_out,
                   int output_index) {
  const char* op = "dh_sample_topk";
  DH_REQUIRE_INIT(op);
  if (vocab <= 0) return dh::fail(1, "[%s] vocabSize must be positive, got %d", op, vocab);
  if (top_k < 1 || top_k > kMaxTopK) return dh::fail(1, "[%s] topK must be in 1..%d, got %d", op, kMaxTopK, top_k);
  if (!(temperature > 0.0)) return dh::fail(1, "[%s] temperature must be positive", op);
  if (!(random_value >= 0.0 && random_value <= 1.0)) return dh::fail(1, "[%s] randomValue must be in [0, 1]", op);
  if (output_index < 0) return dh::fail(1, "[%s] outputIndex must be non-negative", op);
  if (!d_logits || !d_workspace || !d_token_out) return dh::fail(1, "[%s] null pointer", op);
  SampleArgs a{};
  a.top_k = std::min(top_k, vocab);
  a.pad_id = pad_token_id; a.softcap = logit_softcap;
  a.temperature = temperature; a.random_value = random_value;
  a.token_out = d_token_out; a.output_index = output_index;
  const size_t half = (size_t)groups_of(vocab) * (size_t)a.top_k;
  float* val[2] = {static_cast<float*>(d_workspace), static_cast<float*>(d_workspace) + 2 * half};
  uint32_t* idx[2] = {reinterpret_cast<uint32_t*>(val[0] + half), reinterpret_cast<uint32_t*>(val[1] + half)};
  int n = vocab, round = 0;
  a.logits = d_logits;
  while (true) {
    const int groups = groups_of(n);
    a.n_in = n;
    a.out_val = val[round & 1];
    a.out_idx = idx[round & 1];
    hipLaunchKernelGGL(topk_round_kernel, dim3(groups), dim3(256), 0, dh::stream(), a);
    DH_CHECK_LAUNCH(op);
    if (groups == 1) break;
    a.logits = nullptr;
    a.in_val = a.out_val;
    a.in_idx = a.out_idx;
    n = groups * a.top_k;
    round++;
  }
  return 0;
}

}  // extern "C"
