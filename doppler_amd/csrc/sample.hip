// Top-k temperature sampling over f32 logits: exact top-k (ties to the lower index), softmax of
// value / temperature over the k candidates in f64, inverse-CDF pick with a caller-supplied
// uniform number.  Follows the reference's sampler oracle, tests/kernels/reference/sample.js:62-92,
// with the kernel's extras (soft cap, pad id) of src/gpu/kernels/sample.wgsl:35-51.
//
// Selection is a tournament of 1024-element bitonic sorts in LDS: round 0 sorts slices of the
// vocabulary and keeps the best k of each, later rounds sort 1024 surviving candidates at a time,
// until one workgroup holds them all; that workgroup also draws the token.  k <= 256, so a round
// shrinks the field at least four-fold.
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

__global__ __launch_bounds__(256) void topk_round_kernel(const SampleArgs a) {
  __shared__ float val[kSortN];
  __shared__ uint32_t idx[kSortN];
  __shared__ double prob[kMaxTopK];
  const int tid = threadIdx.x;
  const int base = blockIdx.x * kSortN;
  for (int i = tid; i < kSortN; i += 256) {
    const int g = base + i;
    float v = -INFINITY;                      // padding never ranks before a real entry
    uint32_t id = 0xFFFFFFFFu;
    if (g < a.n_in) {
      if (a.logits) {
        id = (uint32_t)g;
        v = a.logits[g];
        if (a.softcap > 0.f) v = a.softcap * tanhf(v / a.softcap);
        if ((int64_t)g == a.pad_id || !(v == v)) { v = -INFINITY; id = 0xFFFFFFFFu; }   // pad id, NaN: out
      } else {
        v = a.in_val[g];
        id = a.in_idx[g];
      }
    }
    val[i] = v;
    idx[i] = id;
  }
  __syncthreads();
  // bitonic sort, best first
  for (int k = 2; k <= kSortN; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int t = tid; t < kSortN / 2; t += 256) {
        const int lo = 2 * t - (t & (j - 1)), hi = lo + j;       // pair (lo, lo + j)
        const bool descending = (lo & k) == 0;
        const float av = val[lo], bv = val[hi];
        const uint32_t ai = idx[lo], bi = idx[hi];
        const bool swap = descending ? ranks_before(bv, bi, av, ai) : ranks_before(av, ai, bv, bi);
        if (swap) {
          val[lo] = bv; idx[lo] = bi;
          val[hi] = av; idx[hi] = ai;
        }
      }
      __syncthreads();
    }
  }
  if (gridDim.x > 1) {
    for (int i = tid; i < a.top_k; i += 256) {
      a.out_val[blockIdx.x * a.top_k + i] = val[i];
      a.out_idx[blockIdx.x * a.top_k + i] = idx[i];
    }
    return;
  }
  // ---- the field is down to one workgroup: softmax over the candidates and the draw
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
