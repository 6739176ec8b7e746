// Decode attention (one query token) over an f16 KV cache with grouped-query heads.
//
// Split-K over the context: grid = (kv head, split).  A workgroup walks its slice of keys in
// tiles of 64, stages the K and V tiles of ONE kv head in LDS and serves all G = H/Hkv query
// heads that share it from that single copy, so K/V are read from HBM once per kv head
// rather than once per query head.  Scores and softmax statistics are fp32; each split keeps
// an online-softmax state (m, l, o) per query head and a second tiny kernel merges the
// splits with the usual log-sum-exp rescale.
#include <algorithm>
#include <cfloat>

#include "dh_common.h"

namespace {

constexpr int kTileKeys = 64;
constexpr int kMaxG = 8;       // query heads per kv head
constexpr int kMaxPairs = 4;   // output element pairs per thread (G*D <= 2048)

struct AttnArgs {
  const float* Q;       // [H][D]
  const __half* K;      // [rows][Hkv][D]
  const __half* V;
  float* O;             // [H][D]
  float* ws;            // [H][nsplit][D + 2]  (o..., m, l)
  int H, Hkv, G, kbeg, kend, nsplit, tiles_per_split;
  float scale, softcap;
  int kv_start, ring_window;  // ring_window > 0: row = (kv_start + k) % ring_window
};

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

template <int D>
__global__ __launch_bounds__(256) void attn_decode_split_kernel(const AttnArgs a) {
  constexpr int RS = D + 8;             // LDS row stride in halves: 16-byte aligned, bank-skewed
  constexpr int PART = D / 4;           // halves of a K row handled by one lane
  __shared__ __align__(16) __half k_tile[kTileKeys * RS];
  __shared__ __align__(16) __half v_tile[kTileKeys * RS];
  __shared__ __align__(16) float q_s[kMaxG * D];
  __shared__ float p_s[kMaxG * kTileKeys];   // scores, then probabilities
  __shared__ float alpha_s[kMaxG];           // per-head rescale of the running output
  __shared__ float m_s[kMaxG], l_s[kMaxG];
  __shared__ float red_s[kMaxPairs * 2 * 256];  // cross key-subset reduction at the end

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int kvh = blockIdx.x, split = blockIdx.y;
  const int G = a.G;
  const int EP = G * D / 2;                       // output element pairs of this kv head
  const int KS = EP >= 256 ? 1 : 256 / EP;        // key subsets when threads outnumber pairs
  const int npairs = EP >= 256 ? (EP + 255) / 256 : 1;

  for (int i = tid; i < G * D; i += 256) q_s[i] = a.Q[(int64_t)(kvh * G) * D + i];
  if (tid < G) { m_s[tid] = -FLT_MAX; l_s[tid] = 0.f; }
  float2 o_acc[kMaxPairs];
#pragma unroll
  for (int i = 0; i < kMaxPairs; i++) o_acc[i] = make_float2(0.f, 0.f);
  __syncthreads();

  const int tile0 = split * a.tiles_per_split;
  const int key_lo = a.kbeg + tile0 * kTileKeys;
  const int key_hi = min(a.kend, key_lo + a.tiles_per_split * kTileKeys);

  for (int kt = key_lo; kt < key_hi; kt += kTileKeys) {
    const int nkeys = min(kTileKeys, key_hi - kt);
    // ---- stage K and V tiles: 16 bytes per thread per step, rows are D*2 contiguous bytes
    constexpr int VEC_PER_ROW = D / 8;
    for (int i = tid; i < kTileKeys * VEC_PER_ROW; i += 256) {
      const int r = i / VEC_PER_ROW, cvec = i - r * VEC_PER_ROW;
      uint4 kv = make_uint4(0, 0, 0, 0), vv = make_uint4(0, 0, 0, 0);
      if (r < nkeys) {
        int64_t row = (int64_t)a.kv_start + kt + r;
        if (a.ring_window > 0) row %= a.ring_window;
        const int64_t off = (row * a.Hkv + kvh) * D + cvec * 8;
        kv = *reinterpret_cast<const uint4*>(a.K + off);
        vv = *reinterpret_cast<const uint4*>(a.V + off);
      }
      *reinterpret_cast<uint4*>(k_tile + r * RS + cvec * 8) = kv;
      *reinterpret_cast<uint4*>(v_tile + r * RS + cvec * 8) = vv;
    }
    __syncthreads();

    // ---- scores: lane (key = tid>>2, part = tid&3) covers a quarter of the head dim
    {
      const int key = tid >> 2, part = tid & 3;
      float kf[PART];
#pragma unroll
      for (int v8 = 0; v8 < PART / 8; v8++) {
        const uint4 raw = *reinterpret_cast<const uint4*>(k_tile + key * RS + part * PART + v8 * 8);
        const __half2* h2 = reinterpret_cast<const __half2*>(&raw);
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const float2 f = __half22float2(h2[j]);
          kf[v8 * 8 + 2 * j] = f.x;
          kf[v8 * 8 + 2 * j + 1] = f.y;
        }
      }
      for (int g = 0; g < G; g++) {
        const float* qg = q_s + g * D + part * PART;
        float dot = 0.f;
#pragma unroll
        for (int j = 0; j < PART; j += 4) {
          const float4 qv = *reinterpret_cast<const float4*>(qg + j);
          dot = fmaf(qv.x, kf[j], dot);
          dot = fmaf(qv.y, kf[j + 1], dot);
          dot = fmaf(qv.z, kf[j + 2], dot);
          dot = fmaf(qv.w, kf[j + 3], dot);
        }
        dot += __shfl_xor(dot, 1, 64);
        dot += __shfl_xor(dot, 2, 64);
        if (part == 0) {
          float s = dot * a.scale;
          if (a.softcap > 0.f) s = tanhf(s / a.softcap) * a.softcap;
          p_s[g * kTileKeys + key] = key < nkeys ? s : -FLT_MAX;
        }
      }
    }
    __syncthreads();

    // ---- online softmax per query head: wave w takes heads w, w+4
    for (int g = wave; g < G; g += 4) {
      const float s = p_s[g * kTileKeys + lane];
      const float m_old = m_s[g];
      const float m_new = fmaxf(m_old, wave_max(s));
      const float p = lane < nkeys ? __expf(s - m_new) : 0.f;
      const float psum = wave_sum(p);
      p_s[g * kTileKeys + lane] = p;
      if (lane == 0) {
        const float alpha = __expf(m_old - m_new);
        alpha_s[g] = alpha;
        l_s[g] = l_s[g] * alpha + psum;
        m_s[g] = m_new;
      }
    }
    __syncthreads();

    // ---- o = o*alpha + P.V : each thread owns pairs of adjacent output dims
#pragma unroll
    for (int i = 0; i < kMaxPairs; i++) {
      if (i >= npairs) break;
      const int ep = (EP >= 256 ? tid + i * 256 : tid % EP);
      const int ks = EP >= 256 ? 0 : tid / EP;
      if (ep < EP && ks < KS) {
        const int g = ep / (D / 2), dp = ep - g * (D / 2);
        const float alpha = alpha_s[g];
        float2 acc = make_float2(o_acc[i].x * alpha, o_acc[i].y * alpha);
        const float* pg = p_s + g * kTileKeys;
        for (int k = ks; k < nkeys; k += KS) {
          const float2 vf = __half22float2(*reinterpret_cast<const __half2*>(v_tile + k * RS + dp * 2));
          const float p = pg[k];
          acc.x = fmaf(p, vf.x, acc.x);
          acc.y = fmaf(p, vf.y, acc.y);
        }
        o_acc[i] = acc;
      }
    }
    __syncthreads();
  }

  // ---- combine key subsets, then write the split's (o, m, l)
#pragma unroll
  for (int i = 0; i < kMaxPairs; i++) {
    red_s[(i * 2) * 256 + tid] = o_acc[i].x;
    red_s[(i * 2 + 1) * 256 + tid] = o_acc[i].y;
  }
  __syncthreads();
  for (int i = 0; i < npairs; i++) {
    const int ep = tid + i * 256;
    if (ep < EP && (EP >= 256 || tid < EP)) {
      float ox = 0.f, oy = 0.f;
      if (EP >= 256) {
        ox = red_s[(i * 2) * 256 + tid];
        oy = red_s[(i * 2 + 1) * 256 + tid];
      } else {
        for (int ks = 0; ks < KS; ks++) {
          ox += red_s[ks * EP + ep];
          oy += red_s[256 + ks * EP + ep];
        }
      }
      const int g = ep / (D / 2), dp = ep - g * (D / 2);
      const int h = kvh * G + g;
      if (a.nsplit == 1) {
        const float l = l_s[g];
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        a.O[(int64_t)h * D + 2 * dp] = ox * inv;
        a.O[(int64_t)h * D + 2 * dp + 1] = oy * inv;
      } else {
        float* w = a.ws + ((int64_t)h * a.nsplit + split) * (D + 2);
        w[2 * dp] = ox;
        w[2 * dp + 1] = oy;
      }
    }
  }
  if (a.nsplit > 1 && tid < G) {
    float* w = a.ws + ((int64_t)(kvh * G + tid) * a.nsplit + split) * (D + 2);
    w[D] = m_s[tid];
    w[D + 1] = l_s[tid];
  }
}

// One workgroup per query head: out[d] = sum_s e^{m_s - M} o_s[d] / sum_s e^{m_s - M} l_s.
// The per-split factors are computed once, in parallel over splits, and kept in LDS; the
// D threads then walk the splits with independent (prefetchable) loads.
template <int D>
__global__ __launch_bounds__(D) void attn_decode_merge_kernel(const float* __restrict__ ws,
                                                              float* __restrict__ O, int nsplit) {
  __shared__ float f_s[1024];
  __shared__ float red[4];
  const int h = blockIdx.x, d = threadIdx.x;
  const float* base = ws + (int64_t)h * nsplit * (D + 2);
  float M = -FLT_MAX;
  for (int s = d; s < nsplit; s += D) M = fmaxf(M, base[s * (D + 2) + D]);
  M = wave_max(M);
  if ((d & 63) == 0) red[d >> 6] = M;
  __syncthreads();
  M = red[0];
  for (int w = 1; w < D / 64; w++) M = fmaxf(M, red[w]);
  __syncthreads();
  float den = 0.f;
  for (int s = d; s < nsplit; s += D) {
    const float f = __expf(base[s * (D + 2) + D] - M);
    f_s[s] = f;
    den = fmaf(f, base[s * (D + 2) + D + 1], den);
  }
  den = wave_sum(den);
  if ((d & 63) == 0) red[d >> 6] = den;
  __syncthreads();
  den = 0.f;
  for (int w = 0; w < D / 64; w++) den += red[w];
  float num = 0.f;
#pragma unroll 8
  for (int s = 0; s < nsplit; s++) num = fmaf(f_s[s], base[s * (D + 2) + d], num);
  O[(int64_t)h * D + d] = den > 0.f ? num / den : 0.f;
}

__global__ void zero_f32_kernel(float* p, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

int max_splits_for(int kv_len) { return std::max(1, (kv_len + kTileKeys - 1) / kTileKeys); }

int choose_splits(int Hkv, int nkeys) {
  const int tiles = std::max(1, (nkeys + kTileKeys - 1) / kTileKeys);
  const int want = std::max(1, 1024 / std::max(1, Hkv));   // aim for ~4 workgroups per CU
  return std::min(tiles, want);
}

template <int D>
int launch(const AttnArgs& a, const char* op) {
  hipLaunchKernelGGL(attn_decode_split_kernel<D>, dim3(a.Hkv, a.nsplit), dim3(256), 0, dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  if (a.nsplit > 1) {
    hipLaunchKernelGGL(attn_decode_merge_kernel<D>, dim3(a.H), dim3(D), 0, dh::stream(), a.ws, a.O, a.nsplit);
    DH_CHECK_LAUNCH(op);
  }
  return 0;
}

}  // namespace

extern "C" {

size_t dh_attn_decode_workspace_bytes(int H, int D, int kv_len) {
  if (H <= 0 || D <= 0 || kv_len <= 0) return 256;
  const size_t splits = (size_t)std::min(max_splits_for(kv_len), 1024);
  return std::max<size_t>(256, (size_t)H * splits * (D + 2) * sizeof(float));
}

int dh_attn_decode(const float* d_Q, const void* d_K, const void* d_V, float* d_O, int H, int Hkv, int D,
                   int kv_len, float scale, int causal, int start_pos, float softcap, int sliding_window,
                   int kv_start, int kv_layout, void* d_workspace) {
  const char* op = "dh_attn_decode";
  DH_REQUIRE_INIT(op);
  if (H <= 0 || Hkv <= 0 || D <= 0) return dh::fail(1, "[%s] numHeads/numKVHeads/headDim must be positive", op);
  if (H % Hkv) return dh::fail(1, "[%s] numHeads=%d must be a multiple of numKVHeads=%d", op, H, Hkv);
  const int G = H / Hkv;
  if (G > kMaxG) return dh::fail(1, "[%s] %d query heads per kv head not supported (max %d)", op, G, kMaxG);
  if (D != 64 && D != 128) return dh::fail(1, "[%s] headDim %d not supported (64, 128)", op, D);
  if ((int64_t)G * D > 2048) return dh::fail(1, "[%s] G*headDim=%d exceeds 2048", op, G * D);
  if (kv_len < 0 || start_pos < 0 || sliding_window < 0 || kv_start < 0)
    return dh::fail(1, "[%s] kvLen, startPos, slidingWindow and kvStart must be non-negative", op);
  if (kv_layout != DH_KV_CONTIGUOUS && kv_layout != DH_KV_RING)
    return dh::fail(1, "[%s] kvLayout %d not supported (contiguous, ring)", op, kv_layout);
  if (kv_layout == DH_KV_RING && sliding_window <= 0)
    return dh::fail(1, "[%s] ring layout needs slidingWindow > 0", op);
  if (!d_Q || !d_O) return dh::fail(1, "[%s] null pointer", op);

  // visible key range [kbeg, kend) in cache-relative indices (abs_key = kv_start + k)
  int64_t kbeg = 0, kend = kv_len;
  if (causal) kend = std::min<int64_t>(kend, (int64_t)start_pos - kv_start + 1);
  if (sliding_window > 0 && start_pos >= sliding_window)
    kbeg = std::max<int64_t>(0, (int64_t)start_pos - sliding_window + 1 - kv_start);
  if (kend <= kbeg) {
    hipLaunchKernelGGL(zero_f32_kernel, dim3((H * D + 255) / 256), dim3(256), 0, dh::stream(), d_O, H * D);
    DH_CHECK_LAUNCH(op);
    return 0;
  }
  if (!d_K || !d_V) return dh::fail(1, "[%s] null pointer", op);
  if ((reinterpret_cast<uintptr_t>(d_K) | reinterpret_cast<uintptr_t>(d_V)) & 15)
    return dh::fail(1, "[%s] K/V pointers must be 16-byte aligned", op);

  AttnArgs a{};
  a.Q = d_Q; a.K = static_cast<const __half*>(d_K); a.V = static_cast<const __half*>(d_V);
  a.O = d_O; a.ws = static_cast<float*>(d_workspace);
  a.H = H; a.Hkv = Hkv; a.G = G;
  a.kbeg = (int)kbeg; a.kend = (int)kend;
  const int nkeys = (int)(kend - kbeg);
  int nsplit = choose_splits(Hkv, nkeys);
  const int tiles = (nkeys + kTileKeys - 1) / kTileKeys;
  a.tiles_per_split = (tiles + nsplit - 1) / nsplit;
  nsplit = (tiles + a.tiles_per_split - 1) / a.tiles_per_split;   // no empty splits
  a.nsplit = nsplit;
  if (nsplit > 1 && !d_workspace) return dh::fail(1, "[%s] workspace is required", op);
  a.scale = scale; a.softcap = softcap;
  a.kv_start = kv_start;
  a.ring_window = kv_layout == DH_KV_RING ? sliding_window : 0;
  return D == 64 ? launch<64>(a, op) : launch<128>(a, op);
}

}  // extern "C"
