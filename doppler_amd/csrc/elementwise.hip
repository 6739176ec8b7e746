// Normalisation, rotary embedding, KV-cache writes and the elementwise glue ops.
// All of these move a few KB per token: they are launch-bound, so each is one launch with
// 16-byte accesses where alignment allows and no intermediate buffers.
#include <algorithm>
#include <cmath>

#include "dh_common.h"

namespace {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// Sum over a 256-thread workgroup; every thread gets the result.  `red` is 4 floats of LDS.
__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) red[wave] = v;
  __syncthreads();
  const float total = red[0] + red[1] + red[2] + red[3];
  __syncthreads();
  return total;
}

__device__ __forceinline__ float load_norm_weight(const void* w, int is_f16, int i, int offset) {
  float v = 1.0f;
  if (w) v = is_f16 ? __half2float(static_cast<const __half*>(w)[i]) : static_cast<const float*>(w)[i];
  else return 1.0f;
  return offset ? 1.0f + v : v;
}

// ---------------------------------------------------------------------------------------
// RMSNorm: one workgroup per token.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const void* __restrict__ w,
                                                      int w_f16, float* __restrict__ out, int hidden,
                                                      float eps, int w_offset,
                                                      const float* __restrict__ pre,
                                                      const float* __restrict__ post,
                                                      float* __restrict__ prenorm, float out_scale) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * hidden;
  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += 256) {
    float v = x[base + i];
    if (pre) v += pre[base + i];
    ss = fmaf(v, v, ss);
  }
  const float total = block_sum_256(ss, red);
  const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
  for (int i = threadIdx.x; i < hidden; i += 256) {
    float v = x[base + i];
    if (pre) v += pre[base + i];
    if (prenorm) prenorm[base + i] = v;
    float y = v * inv * load_norm_weight(w, w_f16, i, w_offset);
    if (post) y += post[base + i];
    out[base + i] = y * out_scale;
  }
}

// Fast path: hidden a multiple of 4 and at most 256*4*VPT.  Each thread keeps its slice of
// the row in registers (all 16-byte loads are issued before the first use, so the row costs
// one memory round trip instead of one per element) and the second pass re-reads nothing.
template <int VPT>
__global__ __launch_bounds__(256) void rmsnorm_vec_kernel(const float* __restrict__ x, const void* __restrict__ w,
                                                          int w_f16, float* __restrict__ out, int hidden,
                                                          float eps, int w_offset,
                                                          const float* __restrict__ pre,
                                                          const float* __restrict__ post,
                                                          float* __restrict__ prenorm, float out_scale) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * hidden;
  const int nvec = hidden >> 2;
  float4 v[VPT];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; j++) {
    const int iv = threadIdx.x + j * 256;
    v[j] = make_float4(0.f, 0.f, 0.f, 0.f);
    if (iv < nvec) {
      v[j] = reinterpret_cast<const float4*>(x + base)[iv];
      if (pre) {
        const float4 p = reinterpret_cast<const float4*>(pre + base)[iv];
        v[j].x += p.x; v[j].y += p.y; v[j].z += p.z; v[j].w += p.w;
      }
    }
  }
#pragma unroll
  for (int j = 0; j < VPT; j++) {
    ss = fmaf(v[j].x, v[j].x, ss); ss = fmaf(v[j].y, v[j].y, ss);
    ss = fmaf(v[j].z, v[j].z, ss); ss = fmaf(v[j].w, v[j].w, ss);
  }
  const float total = block_sum_256(ss, red);
  const float inv = 1.0f / sqrtf(total / (float)hidden + eps);
#pragma unroll
  for (int j = 0; j < VPT; j++) {
    const int iv = threadIdx.x + j * 256;
    if (iv < nvec) {
      if (prenorm) reinterpret_cast<float4*>(prenorm + base)[iv] = v[j];
      float4 y;
      y.x = v[j].x * inv * load_norm_weight(w, w_f16, 4 * iv, w_offset);
      y.y = v[j].y * inv * load_norm_weight(w, w_f16, 4 * iv + 1, w_offset);
      y.z = v[j].z * inv * load_norm_weight(w, w_f16, 4 * iv + 2, w_offset);
      y.w = v[j].w * inv * load_norm_weight(w, w_f16, 4 * iv + 3, w_offset);
      if (post) {
        const float4 p = reinterpret_cast<const float4*>(post + base)[iv];
        y.x += p.x; y.y += p.y; y.z += p.z; y.w += p.w;
      }
      y.x *= out_scale; y.y *= out_scale; y.z *= out_scale; y.w *= out_scale;
      reinterpret_cast<float4*>(out + base)[iv] = y;
    }
  }
}

// Two chained normalisations of a token in one launch, one workgroup per token.
//   sandwich (mode 0):      post = rmsnorm(x, w_a) (+ residual);  second = rmsnorm(post, w_b)
//   residual-next (mode 1): post = (x + residual) * scale;        second = rmsnorm(post, w_a)
// Outputs: first_out = post, second_out = second.  A thread re-reads only what it wrote itself, and
// first_out may alias x or residual (each element is read before the same thread overwrites it).
__global__ __launch_bounds__(256) void rmsnorm_pair_kernel(const float* x, const float* residual,
                                                           const void* __restrict__ wa, int wa_f16,
                                                           const void* __restrict__ wb, int wb_f16, float* first_out,
                                                           float* second_out, int hidden, float eps, int w_offset,
                                                           int mode, float scale) {
  __shared__ float red[4];
  const int64_t base = (int64_t)blockIdx.x * hidden;
  float ss = 0.f;
  if (mode == 0) {
    for (int i = threadIdx.x; i < hidden; i += 256) ss = fmaf(x[base + i], x[base + i], ss);
    const float inv_in = 1.0f / sqrtf(block_sum_256(ss, red) / (float)hidden + eps);
    ss = 0.f;
    for (int i = threadIdx.x; i < hidden; i += 256) {
      float post = x[base + i] * inv_in * load_norm_weight(wa, wa_f16, i, w_offset);
      if (residual) post += residual[base + i];
      first_out[base + i] = post;
      ss = fmaf(post, post, ss);
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += 256) {
      const float v = (x[base + i] + residual[base + i]) * scale;
      first_out[base + i] = v;
      ss = fmaf(v, v, ss);
    }
  }
  const float inv = 1.0f / sqrtf(block_sum_256(ss, red) / (float)hidden + eps);
  const void* w2 = mode == 0 ? wb : wa;
  const int w2_f16 = mode == 0 ? wb_f16 : wa_f16;
  for (int i = threadIdx.x; i < hidden; i += 256)
    second_out[base + i] = first_out[base + i] * inv * load_norm_weight(w2, w2_f16, i, w_offset);
}

// Per-head RMSNorm of the q rows and the k rows in one launch: one wave per row of head_dim
// elements (rows q_rows.. are k rows with their own weight).
__global__ __launch_bounds__(256) void rmsnorm_qk_kernel(const float* __restrict__ q, const float* __restrict__ k,
                                                         const void* __restrict__ qw, int qw_f16,
                                                         const void* __restrict__ kw, int kw_f16,
                                                         float* __restrict__ q_out, float* __restrict__ k_out, int q_rows,
                                                         int k_rows, int head_dim, float eps, int w_offset) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= (int64_t)q_rows + k_rows) return;
  const bool is_q = row < q_rows;
  const int64_t base = (is_q ? row : row - q_rows) * head_dim;
  const float* src = (is_q ? q : k) + base;
  float* dst = (is_q ? q_out : k_out) + base;
  const void* w = is_q ? qw : kw;
  const int w_f16 = is_q ? qw_f16 : kw_f16;
  float ss = 0.f;
  for (int i = lane; i < head_dim; i += 64) ss = fmaf(src[i], src[i], ss);
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)head_dim + eps);
  for (int i = lane; i < head_dim; i += 64) dst[i] = src[i] * inv * load_norm_weight(w, w_f16, i, w_offset);
}

// ---------------------------------------------------------------------------------------
// RoPE in place: one thread per rotated pair.
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void rope_kernel(float* __restrict__ x, const float* __restrict__ cos_t,
                                                   const float* __restrict__ sin_t, int64_t total_pairs,
                                                   int heads, int head_dim, int half, int partner,
                                                   int interleaved, int start_pos) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total_pairs) return;
  const int pair = (int)(idx % half);
  const int64_t th = idx / half;  // token * heads + head
  const int64_t token = th / heads;
  const int64_t pos = start_pos + token;
  const float c = cos_t[pos * half + pair], s = sin_t[pos * half + pair];
  float* row = x + th * head_dim;
  const int i0 = interleaved ? 2 * pair : pair;
  const int i1 = interleaved ? 2 * pair + 1 : pair + partner;
  const float x0 = row[i0], x1 = row[i1];
  row[i0] = x0 * c - x1 * s;
  row[i1] = x0 * s + x1 * c;
}

// RoPE in place on separate q [seq][q_heads][head_dim] and k [seq][kv_heads][head_dim] buffers in one
// launch: pairs 0 .. q_pairs-1 belong to q, the rest to k; both read the same tables.
__global__ __launch_bounds__(256) void rope_qk_kernel(float* __restrict__ q, float* __restrict__ k,
                                                      const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                                      int64_t q_pairs, int64_t total_pairs, int q_heads, int kv_heads,
                                                      int head_dim, int half, int partner, int interleaved,
                                                      int start_pos) {
  int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total_pairs) return;
  const bool is_k = idx >= q_pairs;
  if (is_k) idx -= q_pairs;
  const int heads = is_k ? kv_heads : q_heads;
  const int pair = (int)(idx % half);
  const int64_t th = idx / half;  // token * heads + head
  const int64_t pos = start_pos + th / heads;
  const float c = cos_t[pos * half + pair], s = sin_t[pos * half + pair];
  float* row = (is_k ? k : q) + th * head_dim;
  const int i0 = interleaved ? 2 * pair : pair;
  const int i1 = interleaved ? 2 * pair + 1 : pair + partner;
  const float x0 = row[i0], x1 = row[i1];
  row[i0] = x0 * c - x1 * s;
  row[i1] = x0 * s + x1 * c;
}

// ---------------------------------------------------------------------------------------
// Fused split-QKV + per-head RMSNorm + RoPE + f16 KV write.  One wave per (token, head)
// row for Q and K rows; the trailing workgroups narrow V.  D <= 512.
// ---------------------------------------------------------------------------------------
struct QkvArgs {
  const float* qkv;
  const float* qw;
  const float* kw;
  const float* cos_t;
  const float* sin_t;
  float* q_out;
  __half* cache_k;
  __half* cache_v;
  int T, H, Hkv, D, start_pos, rotary_dim, interleaved, w_offset, use_norm;
  float eps;
  int64_t kv_dst;
  int64_t qk_rows;   // T * (H + Hkv)
  int64_t total_v;   // T * Hkv * D
};

__global__ __launch_bounds__(256) void qkv_norm_rope_kernel(const QkvArgs a) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int64_t qk_groups = (a.qk_rows + 3) / 4;
  if ((int64_t)blockIdx.x >= qk_groups) {
    // V: plain narrowing copy
    const int64_t i = ((int64_t)blockIdx.x - qk_groups) * 256 + threadIdx.x;
    if (i < a.total_v) {
      const int64_t v_size = (int64_t)a.Hkv * a.D;
      const int64_t t = i / v_size, e = i - t * v_size;
      const int64_t stride = (int64_t)(a.H + 2 * a.Hkv) * a.D;
      a.cache_v[a.kv_dst + i] = __float2half(a.qkv[t * stride + (int64_t)(a.H + a.Hkv) * a.D + e]);
    }
    return;
  }
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= a.qk_rows) return;
  const int rows_per_tok = a.H + a.Hkv;
  const int64_t t = row / rows_per_tok;
  const int r = (int)(row - t * rows_per_tok);
  const bool is_q = r < a.H;
  const int head = is_q ? r : r - a.H;
  const int64_t stride = (int64_t)(a.H + 2 * a.Hkv) * a.D;
  const float* src = a.qkv + t * stride + (is_q ? 0 : (int64_t)a.H * a.D) + (int64_t)head * a.D;
  const float* w = is_q ? a.qw : a.kw;
  const int D = a.D;
  float inv = 1.0f;
  if (a.use_norm) {
    float ss = 0.f;
    for (int i = lane; i < D; i += 64) ss = fmaf(src[i], src[i], ss);
    ss = wave_sum(ss);
    inv = 1.0f / sqrtf(ss / (float)D + a.eps);
  }
  const int half = a.rotary_dim / 2;
  const int64_t pos = a.start_pos + t;
  float* qdst = a.q_out + (t * a.H + head) * D;
  __half* kdst = a.cache_k + a.kv_dst + (t * a.Hkv + head) * D;
  auto nv = [&](int i) -> float {
    float v = src[i];
    if (a.use_norm) v = v * inv * (a.w_offset ? 1.0f + w[i] : w[i]);
    return v;
  };
  for (int p = lane; p < half; p += 64) {
    const int i0 = a.interleaved ? 2 * p : p;
    const int i1 = a.interleaved ? 2 * p + 1 : p + half;
    const float c = a.cos_t[pos * half + p], s = a.sin_t[pos * half + p];
    const float x0 = nv(i0), x1 = nv(i1);
    const float y0 = x0 * c - x1 * s, y1 = x0 * s + x1 * c;
    if (is_q) { qdst[i0] = y0; qdst[i1] = y1; }
    else { kdst[i0] = __float2half(y0); kdst[i1] = __float2half(y1); }
  }
  for (int i = a.rotary_dim + lane; i < D; i += 64) {
    const float v = nv(i);
    if (is_q) qdst[i] = v; else kdst[i] = __float2half(v);
  }
}

// ---------------------------------------------------------------------------------------
// Elementwise
// ---------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void kv_write_kernel(const float* __restrict__ k, const float* __restrict__ v,
                                                       __half* __restrict__ ck, __half* __restrict__ cv,
                                                       int64_t src, int64_t dst, int64_t count) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= count) return;
  ck[dst + i] = __float2half(k[src + i]);
  cv[dst + i] = __float2half(v[src + i]);
}

__global__ __launch_bounds__(256) void residual_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                       float* __restrict__ out, int64_t n, float scale) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = (a[i] + b[i]) * scale;
}

// Rows of [q | k | v] copied apart into three dense buffers, one element per thread.
__global__ __launch_bounds__(256) void split_qkv_kernel(const float* __restrict__ qkv, float* __restrict__ q,
                                                        float* __restrict__ k, float* __restrict__ v, int64_t total,
                                                        int q_size, int k_size, int v_size) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int row_len = q_size + k_size + v_size;
  const int64_t t = i / row_len;
  const int c = (int)(i % row_len);
  const float x = qkv[i];
  if (c < q_size) q[t * q_size + c] = x;
  else if (c < q_size + k_size) k[t * k_size + (c - q_size)] = x;
  else v[t * v_size + (c - q_size - k_size)] = x;
}

// data[t][d] += bias[d] in place; bias is f32 or f16.
__global__ __launch_bounds__(256) void bias_add_kernel(float* __restrict__ data, const void* __restrict__ bias,
                                                       int bias_f16, int64_t total, int dim) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int d = (int)(i % dim);
  const float b = bias_f16 ? __half2float(((const __half*)bias)[d]) : ((const float*)bias)[d];
  data[i] += b;
}

// out = in * scale; out may be the input itself.
__global__ __launch_bounds__(256) void scale_kernel(const float* in, float* out, int64_t n, float scale) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = in[i] * scale;
}

__global__ __launch_bounds__(256) void gather_f16_kernel(const uint32_t* __restrict__ ids,
                                                         const __half* __restrict__ table,
                                                         float* __restrict__ out, int64_t total, int hidden,
                                                         uint32_t vocab, int index_offset) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / hidden;
  const int d = (int)(i - t * hidden);
  const uint32_t id = ids[t + index_offset];
  out[i] = id >= vocab ? 0.0f : __half2float(table[(int64_t)id * hidden + d]);
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + __expf(-x)); }
__device__ __forceinline__ float gelu_f(float x) {
  const float inner = 0.7978845608f * (x + 0.044715f * x * x * x);
  return 0.5f * x * (1.0f + tanhf(fminf(fmaxf(inner, -15.0f), 15.0f)));
}
__device__ __forceinline__ float gate_mul(float g, float u, int act, float clamp_max) {
  if (act == DH_ACT_SILU) {
    float v = silu_f(g) * u;
    if (clamp_max > 0.f) v = fminf(fmaxf(v, -clamp_max), clamp_max);
    return v;
  }
  return gelu_f(g) * u;
}

__global__ __launch_bounds__(256) void act_gate_kernel(const float* __restrict__ gate, const float* __restrict__ up,
                                                       float* __restrict__ out, int64_t n, int act,
                                                       float clamp_max) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = gate_mul(gate[i], up[i], act, clamp_max);
}

__global__ __launch_bounds__(256) void act_gate_rowsplit_kernel(const float* __restrict__ in,
                                                                float* __restrict__ out, int64_t total, int dim,
                                                                int act, float clamp_max) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / dim;
  const int d = (int)(i - t * dim);
  const float* row = in + t * 2 * dim;
  out[i] = gate_mul(row[d], row[dim + d], act, clamp_max);
}

__global__ __launch_bounds__(256) void cast_f32_f16_kernel(const float* __restrict__ in, __half* __restrict__ out,
                                                           int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = __float2half(in[i]);
}
__global__ __launch_bounds__(256) void cast_f16_f32_kernel(const __half* __restrict__ in, float* __restrict__ out,
                                                           int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = __half2float(in[i]);
}

// status[0] goes 0 -> 1 for the first element that is not finite or whose magnitude exceeds the
// threshold; the launch that wins the exchange records its layer and step beside it.
template <typename T>
__global__ __launch_bounds__(256) void check_finiteness_kernel(const T* __restrict__ in, int64_t n,
                                                               uint32_t* __restrict__ status, uint32_t layer,
                                                               uint32_t step, float abs_threshold) {
  int bad = 0;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float v = static_cast<float>(in[i]);
    const uint32_t bits = __float_as_uint(v);
    bad |= ((bits & 0x7F800000u) == 0x7F800000u) | (fabsf(v) > abs_threshold);
  }
  if (__syncthreads_or(bad) && threadIdx.x == 0) {
    if (atomicCAS(&status[0], 0u, 1u) == 0u) {
      __hip_atomic_store(&status[1], layer, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&status[2], step, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

unsigned grid_for(int64_t n) { return (unsigned)dh::ceil_div(n, 256); }

}  // namespace

namespace dh {

static void* finiteness_kernel_for(int dtype) {
  return dtype == DH_F16 ? reinterpret_cast<void*>(check_finiteness_kernel<__half>)
                         : reinterpret_cast<void*>(check_finiteness_kernel<float>);
}

// Finds the kernel node of every recorded check: same kernel, input, status word, layer and step.
int finite_graph_bind(Graph* g) {
  if (g->n_fin == 0) return 0;
  size_t n = 0;
  DH_CHECK_HIP("dh_graph_end", hipGraphGetNodes(g->graph, nullptr, &n));
  hipGraphNode_t* nodes = new hipGraphNode_t[n ? n : 1];
  hipError_t e = hipGraphGetNodes(g->graph, nodes, &n);
  if (e != hipSuccess) {
    delete[] nodes;
    return fail(2, "[dh_graph_end] hipGraphGetNodes failed: %s", hipGetErrorString(e));
  }
  int found = 0;
  for (size_t i = 0; i < n; i++) {
    hipGraphNodeType type;
    if (hipGraphNodeGetType(nodes[i], &type) != hipSuccess || type != hipGraphNodeTypeKernel) continue;
    hipKernelNodeParams kp{};
    if (hipGraphKernelNodeGetParams(nodes[i], &kp) != hipSuccess || !kp.kernelParams) continue;
    for (int c = 0; c < g->n_fin; c++) {
      GraphFiniteCall& f = g->fin[c];
      if (f.node || kp.func != finiteness_kernel_for(f.dtype)) continue;
      const void* in = *static_cast<const void* const*>(kp.kernelParams[0]);
      const uint32_t* status = *static_cast<uint32_t* const*>(kp.kernelParams[2]);
      const uint32_t layer = *static_cast<const uint32_t*>(kp.kernelParams[3]);
      const uint32_t step = *static_cast<const uint32_t*>(kp.kernelParams[4]);
      if (in == f.input && status == f.status && layer == f.layer && step == f.step) {
        f.node = nodes[i];
        found++;
        break;
      }
    }
  }
  delete[] nodes;
  if (found != g->n_fin)
    return fail(2, "[dh_graph_end] found the kernel nodes of %d of %d finiteness checks in the captured graph", found, g->n_fin);
  return 0;
}

int finite_graph_set_position(Graph* g, int position) {
  const int delta = position - g->captured_position;
  for (int i = 0; i < g->n_fin; i++) {
    const GraphFiniteCall& f = g->fin[i];
    const void* in = f.input;
    int64_t size = f.size;
    uint32_t* status = f.status;
    uint32_t layer = f.layer, step = (uint32_t)((int64_t)f.step + delta);
    float thr = f.abs_threshold;
    void* args[] = {&in, &size, &status, &layer, &step, &thr};
    hipKernelNodeParams kp{};
    kp.func = finiteness_kernel_for(f.dtype);
    kp.gridDim = dim3(f.grid);
    kp.blockDim = dim3(256);
    kp.sharedMemBytes = 0;
    kp.kernelParams = args;
    DH_CHECK_HIP("dh_graph_launch", hipGraphExecKernelNodeSetParams(g->exec, f.node, &kp));
  }
  return 0;
}

}  // namespace dh

extern "C" {

int dh_rmsnorm(const float* d_x, const void* d_weight, int weight_dtype, float* d_out, int batch,
               int hidden, float eps, int weight_offset, const float* d_pre_residual,
               const float* d_post_residual, float* d_prenorm_out, float output_scale) {
  const char* op = "dh_rmsnorm";
  DH_REQUIRE_INIT(op);
  if (batch <= 0 || hidden <= 0) return dh::fail(1, "[%s] batch=%d hidden=%d must be positive", op, batch, hidden);
  if (!d_x || !d_out) return dh::fail(1, "[%s] null pointer", op);
  if (weight_dtype != DH_F32 && weight_dtype != DH_F16)
    return dh::fail(1, "[%s] weight dtype must be f32 or f16", op);
  if (d_prenorm_out && !d_pre_residual)
    return dh::fail(1, "[%s] prenorm output needs a pre-residual input", op);
  const uintptr_t align = reinterpret_cast<uintptr_t>(d_x) | reinterpret_cast<uintptr_t>(d_out) |
                          reinterpret_cast<uintptr_t>(d_pre_residual) | reinterpret_cast<uintptr_t>(d_post_residual) |
                          reinterpret_cast<uintptr_t>(d_prenorm_out);
  const bool vec_ok = hidden % 4 == 0 && (align & 15) == 0;
#define DH_RMS_ARGS d_x, d_weight, weight_dtype == DH_F16, d_out, hidden, eps, weight_offset, d_pre_residual, \
                    d_post_residual, d_prenorm_out, output_scale
  if (vec_ok && hidden <= 1024) {
    hipLaunchKernelGGL(rmsnorm_vec_kernel<1>, dim3(batch), dim3(256), 0, dh::stream(), DH_RMS_ARGS);
  } else if (vec_ok && hidden <= 4096) {
    hipLaunchKernelGGL(rmsnorm_vec_kernel<4>, dim3(batch), dim3(256), 0, dh::stream(), DH_RMS_ARGS);
  } else if (vec_ok && hidden <= 8192) {
    hipLaunchKernelGGL(rmsnorm_vec_kernel<8>, dim3(batch), dim3(256), 0, dh::stream(), DH_RMS_ARGS);
  } else {
    hipLaunchKernelGGL(rmsnorm_kernel, dim3(batch), dim3(256), 0, dh::stream(), DH_RMS_ARGS);
  }
#undef DH_RMS_ARGS
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_rmsnorm_sandwich_pair(const float* d_x, const float* d_residual, const void* d_post_weight,
                             int post_weight_dtype, const void* d_pre_weight, int pre_weight_dtype,
                             float* d_post_out, float* d_pre_out, int batch, int hidden, float eps,
                             int weight_offset) {
  const char* op = "dh_rmsnorm_sandwich_pair";
  DH_REQUIRE_INIT(op);
  if (batch <= 0 || hidden <= 0) return dh::fail(1, "[%s] batch=%d hidden=%d must be positive", op, batch, hidden);
  if (!d_x || !d_post_weight || !d_pre_weight || !d_post_out || !d_pre_out) return dh::fail(1, "[%s] null pointer", op);
  if ((post_weight_dtype != DH_F32 && post_weight_dtype != DH_F16) ||
      (pre_weight_dtype != DH_F32 && pre_weight_dtype != DH_F16))
    return dh::fail(1, "[%s] weight dtype must be f32 or f16", op);
  if (d_post_out == d_pre_out) return dh::fail(1, "[%s] the two outputs must be different buffers", op);
  hipLaunchKernelGGL(rmsnorm_pair_kernel, dim3(batch), dim3(256), 0, dh::stream(), d_x, d_residual, d_post_weight,
                     post_weight_dtype == DH_F16, d_pre_weight, pre_weight_dtype == DH_F16, d_post_out, d_pre_out, hidden,
                     eps, weight_offset, 0, 1.0f);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_residual_rmsnorm_pair(const float* d_x, const float* d_residual, const void* d_norm_weight,
                             int norm_weight_dtype, float* d_residual_out, float* d_norm_out, int batch,
                             int hidden, float eps, int weight_offset, float output_scale) {
  const char* op = "dh_residual_rmsnorm_pair";
  DH_REQUIRE_INIT(op);
  if (batch <= 0 || hidden <= 0) return dh::fail(1, "[%s] batch=%d hidden=%d must be positive", op, batch, hidden);
  if (!d_x || !d_residual || !d_norm_weight || !d_residual_out || !d_norm_out) return dh::fail(1, "[%s] null pointer", op);
  if (norm_weight_dtype != DH_F32 && norm_weight_dtype != DH_F16)
    return dh::fail(1, "[%s] weight dtype must be f32 or f16", op);
  if (!(output_scale == output_scale) || output_scale > 3.0e38f || output_scale < -3.0e38f)
    return dh::fail(1, "[residual_rmsnorm_pair] outputScale must be finite");
  if (d_residual_out == d_norm_out) return dh::fail(1, "[%s] the two outputs must be different buffers", op);
  hipLaunchKernelGGL(rmsnorm_pair_kernel, dim3(batch), dim3(256), 0, dh::stream(), d_x, d_residual, d_norm_weight,
                     norm_weight_dtype == DH_F16, nullptr, 0, d_residual_out, d_norm_out, hidden, eps, weight_offset, 1,
                     output_scale);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_rmsnorm_qk(const float* d_q, const float* d_k, const void* d_q_weight, int q_weight_dtype,
                  const void* d_k_weight, int k_weight_dtype, float* d_q_out, float* d_k_out, int q_rows,
                  int k_rows, int head_dim, float eps, int weight_offset) {
  const char* op = "dh_rmsnorm_qk";
  DH_REQUIRE_INIT(op);
  if (q_rows <= 0 || k_rows <= 0 || head_dim <= 0)
    return dh::fail(1, "[%s] qRows=%d kRows=%d headDim=%d must be positive", op, q_rows, k_rows, head_dim);
  if (!d_q || !d_k || !d_q_out || !d_k_out || !d_q_weight || !d_k_weight) return dh::fail(1, "[%s] null pointer", op);
  if ((q_weight_dtype != DH_F32 && q_weight_dtype != DH_F16) || (k_weight_dtype != DH_F32 && k_weight_dtype != DH_F16))
    return dh::fail(1, "[%s] weight dtype must be f32 or f16", op);
  const int64_t rows = (int64_t)q_rows + k_rows;
  hipLaunchKernelGGL(rmsnorm_qk_kernel, dim3((unsigned)dh::ceil_div(rows, 4)), dim3(256), 0, dh::stream(), d_q, d_k,
                     d_q_weight, q_weight_dtype == DH_F16, d_k_weight, k_weight_dtype == DH_F16, d_q_out, d_k_out,
                     q_rows, k_rows, head_dim, eps, weight_offset);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_rope(float* d_x, const float* d_cos, const float* d_sin, int seq, int heads, int head_dim,
            int rotary_dim, int pair_span_dim, int interleaved, int start_pos) {
  const char* op = "dh_rope";
  DH_REQUIRE_INIT(op);
  if (seq <= 0 || heads <= 0) return dh::fail(1, "[%s] seq=%d heads=%d must be positive", op, seq, heads);
  if (head_dim <= 0 || head_dim % 2) return dh::fail(1, "RoPE headDim must be even, got %d", head_dim);
  if (rotary_dim % 2) return dh::fail(1, "RoPE rotaryDim must be even, got %d", rotary_dim);
  if (rotary_dim <= 0 || rotary_dim > head_dim)
    return dh::fail(1, "RoPE rotaryDim must be in (0, headDim]; got %d for headDim %d", rotary_dim, head_dim);
  if (pair_span_dim % 2) return dh::fail(1, "RoPE pairSpanDim must be even, got %d", pair_span_dim);
  if (pair_span_dim < rotary_dim || pair_span_dim > head_dim)
    return dh::fail(1, "RoPE pairSpanDim must be in [rotaryDim, headDim]; got %d for rotaryDim %d and headDim %d",
                    pair_span_dim, rotary_dim, head_dim);
  if (start_pos < 0) return dh::fail(1, "[%s] startPos must be non-negative", op);
  if (!d_x || !d_cos || !d_sin) return dh::fail(1, "[%s] null pointer", op);
  const int half = rotary_dim / 2;
  const int64_t pairs = (int64_t)seq * heads * half;
  hipLaunchKernelGGL(rope_kernel, dim3(grid_for(pairs)), dim3(256), 0, dh::stream(), d_x, d_cos, d_sin,
                     pairs, heads, head_dim, half, pair_span_dim / 2, interleaved, start_pos);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_rope_qk(float* d_q, float* d_k, const float* d_cos, const float* d_sin, int seq, int q_heads, int kv_heads,
               int head_dim, int rotary_dim, int pair_span_dim, int interleaved, int start_pos) {
  const char* op = "dh_rope_qk";
  DH_REQUIRE_INIT(op);
  if (seq < 0) return dh::fail(1, "RoPE QK requires seqLen to be a non-negative integer.");
  if (start_pos < 0) return dh::fail(1, "RoPE QK requires startPos to be a non-negative integer.");
  if (q_heads <= 0) return dh::fail(1, "RoPE QK requires numQHeads to be a positive integer.");
  if (kv_heads <= 0) return dh::fail(1, "RoPE QK requires numKVHeads to be a positive integer.");
  if (head_dim <= 0) return dh::fail(1, "RoPE QK requires headDim to be a positive integer.");
  if (head_dim % 2) return dh::fail(1, "RoPE QK headDim must be even, got %d.", head_dim);
  if (rotary_dim <= 0) return dh::fail(1, "RoPE QK requires rotaryDim to be a positive integer.");
  if (rotary_dim % 2) return dh::fail(1, "RoPE QK rotaryDim must be even, got %d.", rotary_dim);
  if (rotary_dim > head_dim)
    return dh::fail(1, "RoPE QK rotaryDim must be <= headDim; got %d for headDim %d.", rotary_dim, head_dim);
  if (pair_span_dim <= 0) return dh::fail(1, "RoPE QK requires pairSpanDim to be a positive integer.");
  if (pair_span_dim % 2) return dh::fail(1, "RoPE QK pairSpanDim must be even, got %d.", pair_span_dim);
  if (pair_span_dim < rotary_dim || pair_span_dim > head_dim)
    return dh::fail(1, "RoPE QK pairSpanDim must be in [rotaryDim, headDim]; got %d for rotaryDim %d and headDim %d.",
                    pair_span_dim, rotary_dim, head_dim);
  if (seq == 0) return 0;
  if (!d_q || !d_k || !d_cos || !d_sin) return dh::fail(1, "[%s] null pointer", op);
  if (d_q == d_k) return dh::fail(1, "[%s] q and k must be different buffers", op);
  const int half = rotary_dim / 2;
  const int64_t q_pairs = (int64_t)seq * q_heads * half;
  const int64_t total = q_pairs + (int64_t)seq * kv_heads * half;
  hipLaunchKernelGGL(rope_qk_kernel, dim3(grid_for(total)), dim3(256), 0, dh::stream(), d_q, d_k, d_cos, d_sin, q_pairs,
                     total, q_heads, kv_heads, head_dim, half, pair_span_dim / 2, interleaved, start_pos);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_qkv_norm_rope_kvwrite(const float* d_qkv, const float* d_q_weight, const float* d_k_weight,
                             const float* d_cos, const float* d_sin, float* d_q_out, void* d_cache_k,
                             void* d_cache_v, int T, int H, int Hkv, int D, int start_pos,
                             int rotary_dim, int interleaved, float eps, int weight_offset,
                             int64_t kv_dst_offset, int use_norm) {
  const char* op = "dh_qkv_norm_rope_kvwrite";
  DH_REQUIRE_INIT(op);
  if (T <= 0 || H <= 0 || Hkv <= 0 || D <= 0)
    return dh::fail(1, "[%s] numTokens/numHeads/numKVHeads/headDim must be positive integers", op);
  if (D % 2 || rotary_dim % 2 || rotary_dim <= 0 || rotary_dim > D)
    return dh::fail(1, "[%s] rotaryDim %d must be even and in (0, headDim=%d]", op, rotary_dim, D);
  if (start_pos < 0 || kv_dst_offset < 0) return dh::fail(1, "[%s] startPos and dstOffset must be non-negative", op);
  if (!d_qkv || !d_cos || !d_sin || !d_q_out || !d_cache_k || !d_cache_v)
    return dh::fail(1, "[%s] null pointer", op);
  if (use_norm && (!d_q_weight || !d_k_weight)) return dh::fail(1, "[%s] q/k norm weights are required", op);
  QkvArgs a{};
  a.qkv = d_qkv; a.qw = d_q_weight; a.kw = d_k_weight; a.cos_t = d_cos; a.sin_t = d_sin;
  a.q_out = d_q_out; a.cache_k = static_cast<__half*>(d_cache_k); a.cache_v = static_cast<__half*>(d_cache_v);
  a.T = T; a.H = H; a.Hkv = Hkv; a.D = D; a.start_pos = start_pos; a.rotary_dim = rotary_dim;
  a.interleaved = interleaved; a.w_offset = weight_offset; a.use_norm = use_norm; a.eps = eps;
  a.kv_dst = kv_dst_offset;
  a.qk_rows = (int64_t)T * (H + Hkv);
  a.total_v = (int64_t)T * Hkv * D;
  const int64_t groups = dh::ceil_div(a.qk_rows, 4) + dh::ceil_div(a.total_v, 256);
  hipLaunchKernelGGL(qkv_norm_rope_kernel, dim3((unsigned)groups), dim3(256), 0, dh::stream(), a);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_kv_write_f16(const float* d_k, const float* d_v, void* d_cache_k, void* d_cache_v,
                    int64_t src_offset, int64_t dst_offset, int64_t count) {
  const char* op = "dh_kv_write_f16";
  DH_REQUIRE_INIT(op);
  if (src_offset < 0 || dst_offset < 0 || count < 0)
    return dh::fail(1, "[%s] srcOffset, dstOffset and elementCount must be non-negative integers", op);
  if (count == 0) return 0;
  if (!d_k || !d_v || !d_cache_k || !d_cache_v) return dh::fail(1, "[%s] null pointer", op);
  hipLaunchKernelGGL(kv_write_kernel, dim3(grid_for(count)), dim3(256), 0, dh::stream(), d_k, d_v,
                     static_cast<__half*>(d_cache_k), static_cast<__half*>(d_cache_v), src_offset,
                     dst_offset, count);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_residual_add(const float* d_a, const float* d_b, float* d_out, int64_t n, float scale) {
  const char* op = "dh_residual_add";
  DH_REQUIRE_INIT(op);
  if (n < 0) return dh::fail(1, "[%s] size must be non-negative", op);
  if (n == 0) return 0;
  if (!d_a || !d_b || !d_out) return dh::fail(1, "[%s] null pointer", op);
  if (!(scale == scale) || scale > 3.0e38f || scale < -3.0e38f)
    return dh::fail(1, "[Residual] outputScale must be finite");
  hipLaunchKernelGGL(residual_kernel, dim3(grid_for(n)), dim3(256), 0, dh::stream(), d_a, d_b, d_out, n, scale);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_split_qkv(const float* d_qkv, float* d_q, float* d_k, float* d_v, int num_tokens, int q_size, int k_size,
                 int v_size) {
  const char* op = "dh_split_qkv";
  DH_REQUIRE_INIT(op);
  if (num_tokens < 0 || q_size <= 0 || k_size <= 0 || v_size <= 0)
    return dh::fail(1, "[%s] numTokens=%d qSize=%d kSize=%d vSize=%d: need numTokens >= 0 and positive sizes", op,
                    num_tokens, q_size, k_size, v_size);
  if (num_tokens == 0) return 0;
  if (!d_qkv || !d_q || !d_k || !d_v) return dh::fail(1, "[%s] null pointer", op);
  const int64_t total = (int64_t)num_tokens * ((int64_t)q_size + k_size + v_size);
  hipLaunchKernelGGL(split_qkv_kernel, dim3(grid_for(total)), dim3(256), 0, dh::stream(), d_qkv, d_q, d_k, d_v, total,
                     q_size, k_size, v_size);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_bias_add(float* d_data, const void* d_bias, int bias_dtype, int64_t num_tokens, int dim,
                int64_t data_offset_bytes, int64_t bias_offset_bytes) {
  const char* op = "dh_bias_add";
  DH_REQUIRE_INIT(op);
  if (num_tokens < 0 || dim <= 0)
    return dh::fail(1, "[%s] numTokens=%lld dim=%d: need numTokens >= 0 and dim > 0", op, (long long)num_tokens, dim);
  if (bias_dtype != DH_F32 && bias_dtype != DH_F16) return dh::fail(1, "[%s] bias dtype must be f32 or f16", op);
  const int64_t bias_elem = bias_dtype == DH_F16 ? 2 : 4;
  if (data_offset_bytes < 0 || data_offset_bytes % 4 || bias_offset_bytes < 0 || bias_offset_bytes % bias_elem)
    return dh::fail(1, "[%s] dataOffset=%lld / biasOffset=%lld must be non-negative multiples of the element size", op,
                    (long long)data_offset_bytes, (long long)bias_offset_bytes);
  if (num_tokens == 0) return 0;
  if (!d_data || !d_bias) return dh::fail(1, "[%s] null pointer", op);
  const int64_t total = num_tokens * dim;
  hipLaunchKernelGGL(bias_add_kernel, dim3(grid_for(total)), dim3(256), 0, dh::stream(),
                     (float*)((char*)d_data + data_offset_bytes), (const void*)((const char*)d_bias + bias_offset_bytes),
                     bias_dtype == DH_F16, total, dim);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_scale(const float* d_in, float* d_out, int64_t n, float scale) {
  const char* op = "dh_scale";
  DH_REQUIRE_INIT(op);
  if (n < 0) return dh::fail(1, "[%s] count must be non-negative", op);
  if (n == 0) return 0;
  if (!d_in || !d_out) return dh::fail(1, "[%s] null pointer", op);
  hipLaunchKernelGGL(scale_kernel, dim3(grid_for(n)), dim3(256), 0, dh::stream(), d_in, d_out, n, scale);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_gather_f16(const uint32_t* d_ids, const void* d_table, float* d_out, int T, int hidden, int vocab,
                  int index_offset) {
  const char* op = "dh_gather_f16";
  DH_REQUIRE_INIT(op);
  if (T <= 0 || hidden <= 0 || vocab <= 0 || index_offset < 0)
    return dh::fail(1, "[%s] numTokens/hiddenSize/vocabSize must be positive", op);
  if (!d_ids || !d_table || !d_out) return dh::fail(1, "[%s] null pointer", op);
  const int64_t total = (int64_t)T * hidden;
  hipLaunchKernelGGL(gather_f16_kernel, dim3(grid_for(total)), dim3(256), 0, dh::stream(), d_ids,
                     static_cast<const __half*>(d_table), d_out, total, hidden, (uint32_t)vocab, index_offset);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_act_gate(const float* d_gate, const float* d_up, float* d_out, int64_t n, int activation,
                float swiglu_limit) {
  const char* op = "dh_act_gate";
  DH_REQUIRE_INIT(op);
  if (n < 0) return dh::fail(1, "[%s] size must be non-negative", op);
  if (activation != DH_ACT_SILU && activation != DH_ACT_GELU) return dh::fail(1, "[%s] unknown activation %d", op, activation);
  if (n == 0) return 0;
  if (!d_gate || !d_up || !d_out) return dh::fail(1, "[%s] null pointer", op);
  hipLaunchKernelGGL(act_gate_kernel, dim3(grid_for(n)), dim3(256), 0, dh::stream(), d_gate, d_up, d_out, n,
                     activation, swiglu_limit);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_act_gate_rowsplit(const float* d_in, float* d_out, int T, int dim, int activation, float swiglu_limit) {
  const char* op = "dh_act_gate_rowsplit";
  DH_REQUIRE_INIT(op);
  if (T <= 0 || dim <= 0) return dh::fail(1, "[%s] numTokens=%d dim=%d must be positive", op, T, dim);
  if (activation != DH_ACT_SILU && activation != DH_ACT_GELU) return dh::fail(1, "[%s] unknown activation %d", op, activation);
  if (!d_in || !d_out) return dh::fail(1, "[%s] null pointer", op);
  const int64_t total = (int64_t)T * dim;
  hipLaunchKernelGGL(act_gate_rowsplit_kernel, dim3(grid_for(total)), dim3(256), 0, dh::stream(), d_in, d_out,
                     total, dim, activation, swiglu_limit);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_cast_f32_to_f16(const float* d_in, void* d_out, int64_t n) {
  const char* op = "dh_cast_f32_to_f16";
  DH_REQUIRE_INIT(op);
  if (n < 0) return dh::fail(1, "[%s] size must be non-negative", op);
  if (n == 0) return 0;
  if (!d_in || !d_out) return dh::fail(1, "[%s] null pointer", op);
  hipLaunchKernelGGL(cast_f32_f16_kernel, dim3(grid_for(n)), dim3(256), 0, dh::stream(), d_in,
                     static_cast<__half*>(d_out), n);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_cast_f16_to_f32(const void* d_in, float* d_out, int64_t n) {
  const char* op = "dh_cast_f16_to_f32";
  DH_REQUIRE_INIT(op);
  if (n < 0) return dh::fail(1, "[%s] size must be non-negative", op);
  if (n == 0) return 0;
  if (!d_in || !d_out) return dh::fail(1, "[%s] null pointer", op);
  hipLaunchKernelGGL(cast_f16_f32_kernel, dim3(grid_for(n)), dim3(256), 0, dh::stream(),
                     static_cast<const __half*>(d_in), d_out, n);
  DH_CHECK_LAUNCH(op);
  return 0;
}

int dh_check_finiteness(const void* d_input, int dtype, int64_t size, uint32_t* d_status, uint32_t layer,
                        uint32_t step, float abs_threshold) {
  const char* op = "dh_check_finiteness";
  DH_REQUIRE_INIT(op);
  if (size < 0) return dh::fail(1, "[%s] size must be non-negative", op);
  if (dtype != DH_F32 && dtype != DH_F16) return dh::fail(1, "[%s] input dtype must be f32 or f16", op);
  if (!d_status) return dh::fail(1, "[%s] status pointer is null", op);
  if (size == 0) return 0;
  if (!d_input) return dh::fail(1, "[%s] null pointer", op);
  if (!(abs_threshold > 0.f) || !std::isfinite(abs_threshold)) abs_threshold = 65500.f;
  const unsigned grid = (unsigned)std::min<int64_t>(dh::ceil_div(size, 256), 4096);
  if (dtype == DH_F16)
    hipLaunchKernelGGL(check_finiteness_kernel<__half>, dim3(grid), dim3(256), 0, dh::stream(),
                       static_cast<const __half*>(d_input), size, d_status, layer, step, abs_threshold);
  else
    hipLaunchKernelGGL(check_finiteness_kernel<float>, dim3(grid), dim3(256), 0, dh::stream(),
                       static_cast<const float*>(d_input), size, d_status, layer, step, abs_threshold);
  DH_CHECK_LAUNCH(op);
  dh::graph_note_finiteness(dh::GraphFiniteCall{d_input, dtype, size, d_status, layer, step, abs_threshold, grid, nullptr});
  return 0;
}

}  // extern "C"
