// Dense f32 GEMV with an RMSNorm over its output row, for one activation row:
//   y[n] = sum_k x[k] * W(n, k);  out[n] = y[n] / sqrt(mean_n(y^2) + eps) * (w[n] | 1 + w[n]) (+ residual[n])
// (reference: src/gpu/kernels/fused_matmul_rmsnorm.wgsl:166-213 small, :215-272 medium; host
// src/gpu/kernels/fused_matmul_rmsnorm.js:50-170).  The reference runs the whole row in one
// workgroup; here the product is spread over the chip in K slices (it is a read of N*K*4 bytes of
// weights, bound by HBM), the slices are summed in a fixed order (by a launch of its own when there
// are more than 8) and a single-workgroup launch on the same stream reduces the squares and writes
// the normalised row.
#include <algorithm>

#include "dh_common.h"

namespace {

constexpr int kFinishThreads = 1024;
constexpr int kMaxN = 4096;   // the reference's maxMediumN (src/config/schema/kernel-thresholds.schema.js:87)

// Element types of activations, weights, residual and output: f32, or f16 widened on load and
// rounded once on the final store (all sums run in f32 either way).
// The weight matrix is read once per call, every wave whole cache lines of it: those loads carry the
// non-temporal hint (STREAM), the activations' do not.
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
template <bool STREAM>
__device__ __forceinline__ u32x4_t load_16(const void* p) {
  return STREAM ? __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p)) : *reinterpret_cast<const u32x4_t*>(p);
}
template <bool STREAM>
__device__ __forceinline__ u32x2_t load_8(const void* p) {
  return STREAM ? __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p)) : *reinterpret_cast<const u32x2_t*>(p);
}
template <typename T> struct Vec16;   // a 16-byte piece
template <> struct Vec16<float> {
  static constexpr int N = 4;
  template <bool STREAM = false>
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const u32x4_t t = load_16<STREAM>(p);
#pragma unroll
    for (int i = 0; i < 4; i++) v[i] = __uint_as_float(t[i]);
  }
};
template <> struct Vec16<__half> {
  static constexpr int N = 8;
  template <bool STREAM = false>
  static __device__ __forceinline__ void load(const __half* p, float (&v)[8]) {
    const u32x4_t w = load_16<STREAM>(p);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[2 * i] = __half2float(__ushort_as_half((unsigned short)(w[i] & 0xffffu)));
      v[2 * i + 1] = __half2float(__ushort_as_half((unsigned short)(w[i] >> 16)));
    }
  }
};
__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(__half v) { return __half2float(v); }
// four consecutive elements
template <bool STREAM = false>
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) { Vec16<float>::load<STREAM>(p, v); }
template <bool STREAM = false>
__device__ __forceinline__ void load4(const __half* p, float (&v)[4]) {
  const u32x2_t t = load_8<STREAM>(p);
  v[0] = __half2float(__ushort_as_half((unsigned short)(t[0] & 0xffffu)));
  v[1] = __half2float(__ushort_as_half((unsigned short)(t[0] >> 16)));
  v[2] = __half2float(__ushort_as_half((unsigned short)(t[1] & 0xffffu)));
  v[3] = __half2float(__ushort_as_half((unsigned short)(t[1] >> 16)));
}

// W is [N, K]: a wave per output row and K slice, lanes stride over the slice in 16-byte pieces,
// four loads in flight per lane.  parts[slice][n] receives the wave's sum.
template <typename T>
__global__ __launch_bounds__(256) void gemv_rows_kernel(const T* __restrict__ x, const T* __restrict__ W,
                                                        float* __restrict__ parts, int N, int K, int k_per_slice,
                                                        int vec) {
  constexpr int V = Vec16<T>::N;
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= N) return;
  const int k0 = blockIdx.y * k_per_slice;
  const int k1 = min(K, k0 + k_per_slice);
  const T* row = W + (int64_t)n * K;
  float acc = 0.f;
  if (vec) {
    // k_per_slice and K are multiples of V here; pieces q0 .. q1 - 1 of the row
    const int q1 = k1 / V;
    int q = k0 / V + lane;
    float a[4] = {0.f, 0.f, 0.f, 0.f};
    for (; q + 192 < q1; q += 256) {
      float w[4][V], v[4][V];
#pragma unroll
      for (int u = 0; u < 4; u++) {
        Vec16<T>::template load<true>(row + (int64_t)(q + 64 * u) * V, w[u]);
        Vec16<T>::load(x + (int64_t)(q + 64 * u) * V, v[u]);
      }
#pragma unroll
      for (int u = 0; u < 4; u++)
#pragma unroll
        for (int e = 0; e < V; e++) a[u] = fmaf(w[u][e], v[u][e], a[u]);
    }
    for (; q < q1; q += 64) {
      float w[V], v[V];
      Vec16<T>::template load<true>(row + (int64_t)q * V, w);
      Vec16<T>::load(x + (int64_t)q * V, v);
#pragma unroll
      for (int e = 0; e < V; e++) a[0] = fmaf(w[e], v[e], a[0]);
    }
    acc = (a[0] + a[1]) + (a[2] + a[3]);
  } else {
    for (int k = k0 + lane; k < k1; k += 64) acc = fmaf(to_f32(row[k]), to_f32(x[k]), acc);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0) parts[(int64_t)blockIdx.y * N + n] = acc;
}

// W is [K, N]: a workgroup of 16 waves covers 256 output columns (64 lanes x 4) and one slice of K;
// wave w takes rows w, w + 16, ... of the slice, four rows in flight, and the waves meet in LDS in
// wave order.  parts[slice][n] receives the sum.
constexpr int kColsWaves = 16;
template <typename T>
__global__ __launch_bounds__(kColsWaves * 64) void gemv_cols_kernel(const T* __restrict__ x, const T* __restrict__ W,
                                                                    float* __restrict__ parts, int N, int K,
                                                                    int k_per_slice, int vec) {
  __shared__ float red[kColsWaves][64][4];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * 256 + lane * 4;
  const int k0 = blockIdx.y * k_per_slice;
  const int k1 = min(K, k0 + k_per_slice);
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  if (vec) {
    if (n0 < N) {
      const T* col = W + n0;
      int k = k0 + wave;
      for (; k + 3 * kColsWaves < k1; k += 4 * kColsWaves) {
        float w[4][4];
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
          load4<true>(col + (int64_t)(k + u * kColsWaves) * N, w[u]);
          v[u] = to_f32(x[k + u * kColsWaves]);
        }
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
          for (int j = 0; j < 4; j++) acc[j] = fmaf(w[u][j], v[u], acc[j]);
      }
      for (; k < k1; k += kColsWaves) {
        float w[4];
        load4<true>(col + (int64_t)k * N, w);
        const float v = to_f32(x[k]);
#pragma unroll
        for (int j = 0; j < 4; j++) acc[j] = fmaf(w[j], v, acc[j]);
      }
    }
  } else {
    for (int k = k0 + wave; k < k1; k += kColsWaves) {
      const float v = to_f32(x[k]);
      const T* row = W + (int64_t)k * N;
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (n0 + j < N) acc[j] = fmaf(to_f32(row[n0 + j]), v, acc[j]);
    }
  }
#pragma unroll
  for (int j = 0; j < 4; j++) red[wave][lane][j] = acc[j];
  __syncthreads();
  if (threadIdx.x < 256) {
    // thread t finishes column t of the block: lane t / 4, element t % 4
    const int l = threadIdx.x >> 2, j = threadIdx.x & 3;
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kColsWaves; w++) s += red[w][l][j];
    const int n = blockIdx.x * 256 + threadIdx.x;
    if (n < N) parts[(int64_t)blockIdx.y * N + n] = s;
  }
}

// More slices than one workgroup should read: 64 columns per workgroup, four groups of slices per
// column summed in slice order and met in LDS in group order.  y[n] receives the sum.
__global__ __launch_bounds__(256) void slices_sum_kernel(const float* __restrict__ parts, int slices,
                                                         float* __restrict__ y, int N) {
  __shared__ float red[4][64];
  const int c = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int n = blockIdx.x * 64 + c;
  float s = 0.f;
  if (n < N)
    for (int p = g; p < slices; p += 4) s += parts[(int64_t)p * N + n];
  red[g][c] = s;
  __syncthreads();
  if (g == 0 && n < N) y[n] = ((red[0][c] + red[1][c]) + red[2][c]) + red[3][c];
}

// One workgroup: y[n] = sum over slices (in slice order), mean of squares, scale, weight, residual.
template <typename T>
__global__ __launch_bounds__(kFinishThreads) void rmsnorm_finish_kernel(const float* __restrict__ parts, int slices,
                                                                        const void* __restrict__ norm_weight,
                                                                        int weight_f16, int weight_offset,
                                                                        const T* __restrict__ residual,
                                                                        T* __restrict__ out, int N, float eps) {
  __shared__ float red[kFinishThreads / 64];
  float y[kMaxN / kFinishThreads];
  float ssq = 0.f;
#pragma unroll
  for (int c = 0; c < kMaxN / kFinishThreads; c++) {
    const int n = threadIdx.x + c * kFinishThreads;
    float s = 0.f;
    if (n < N)
      for (int p = 0; p < slices; p++) s += parts[(int64_t)p * N + n];
    y[c] = s;
    ssq += s * s;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ssq += __shfl_xor(ssq, off, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ssq;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < kFinishThreads / 64; w++) total += red[w];
  const float inv_rms = 1.0f / sqrtf(total / (float)N + eps);
#pragma unroll
  for (int c = 0; c < kMaxN / kFinishThreads; c++) {
    const int n = threadIdx.x + c * kFinishThreads;
    if (n >= N) continue;
    float w = weight_f16 ? __half2float(static_cast<const __half*>(norm_weight)[n])
                         : static_cast<const float*>(norm_weight)[n];
    if (weight_offset) w += 1.0f;
    float r = y[c] * inv_rms * w;
    if (residual) r += to_f32(residual[n]);
    out[n] = static_cast<T>(r);
  }
}

template <typename T>
int matmul_rmsnorm_impl(const char* op, const T* d_x, const T* d_W, int transpose_b, const void* d_norm_weight,
                        int norm_weight_dtype, float eps, int weight_offset, const T* d_residual, T* d_out, int N, int K) {
  DH_REQUIRE_INIT(op);
  constexpr int V = Vec16<T>::N;
  if (N <= 0 || K <= 0) return dh::fail(1, "[%s] Dimensions must be positive: N=%d, K=%d", op, N, K);
  if (N > kMaxN)
    return dh::fail(1, "[%s] N=%d exceeds maxMediumN=%d; the RMSNorm over the output row is one workgroup", op, N, kMaxN);
  if (!d_x || !d_W || !d_norm_weight || !d_out) return dh::fail(1, "[%s] null pointer", op);
  if (norm_weight_dtype != DH_F32 && norm_weight_dtype != DH_F16)
    return dh::fail(1, "[%s] norm weight dtype must be f32 or f16", op);
  size_t ws_bytes = 0;
  float* parts = dh::splitk_workspace(&ws_bytes);
  int slices = 1;
  if (transpose_b) {
    const int vec = (K % V == 0) && ((reinterpret_cast<uintptr_t>(d_W) | reinterpret_cast<uintptr_t>(d_x)) % 16 == 0);
    // about 16 waves per compute unit, at least 256 16-byte pieces of a row per wave
    slices = std::max(1, std::min<int>((int)(K / (256 * V)), (int)dh::ceil_div(16 * dh::num_cus(), N)));
    const int k_per_slice = (int)dh::ceil_div(dh::ceil_div(K, slices), V) * V;
    slices = (int)dh::ceil_div(K, k_per_slice);
    if ((size_t)(slices + 1) * N * sizeof(float) > ws_bytes)
      return dh::fail(2, "[%s] internal: %d slices of %d floats do not fit the workspace", op, slices, N);
    hipLaunchKernelGGL(gemv_rows_kernel<T>, dim3((unsigned)dh::ceil_div(N, 4), slices), dim3(256), 0, dh::stream(), d_x,
                       d_W, parts, N, K, k_per_slice, vec);
  } else {
    const int col_blocks = (int)dh::ceil_div(N, 256);
    // about two workgroups of 16 waves per compute unit, at least 64 rows of W each
    slices = std::max(1, std::min<int>((int)(K / 64), (int)dh::ceil_div(2 * dh::num_cus(), col_blocks)));
    const int k_per_slice = (int)dh::ceil_div(K, slices);
    slices = (int)dh::ceil_div(K, k_per_slice);
    if ((size_t)(slices + 1) * N * sizeof(float) > ws_bytes)
      return dh::fail(2, "[%s] internal: %d slices of %d floats do not fit the workspace", op, slices, N);
    const int vec = (N % 4 == 0) && (reinterpret_cast<uintptr_t>(d_W) % (4 * sizeof(T)) == 0);
    hipLaunchKernelGGL(gemv_cols_kernel<T>, dim3(col_blocks, slices), dim3(kColsWaves * 64), 0, dh::stream(), d_x, d_W,
                       parts, N, K, k_per_slice, vec);
  }
  DH_CHECK_LAUNCH(op);
  if (slices > 8) {
    float* y = parts + (size_t)slices * N;
    hipLaunchKernelGGL(slices_sum_kernel, dim3((unsigned)dh::ceil_div(N, 64)), dim3(256), 0, dh::stream(), parts, slices,
                       y, N);
    DH_CHECK_LAUNCH(op);
    parts = y;
    slices = 1;
  }
  hipLaunchKernelGGL(rmsnorm_finish_kernel<T>, dim3(1), dim3(kFinishThreads), 0, dh::stream(), parts, slices,
                     d_norm_weight, norm_weight_dtype == DH_F16, weight_offset, d_residual, d_out, N, eps);
  DH_CHECK_LAUNCH(op);
  return 0;
}

}  // namespace

extern "C" int dh_matmul_rmsnorm_f32(const float* d_x, const float* d_W, int transpose_b, const void* d_norm_weight,
                                     int norm_weight_dtype, float eps, int weight_offset, const float* d_residual,
                                     float* d_out, int N, int K) {
  return matmul_rmsnorm_impl<float>("dh_matmul_rmsnorm_f32", d_x, d_W, transpose_b, d_norm_weight, norm_weight_dtype, eps,
                                    weight_offset, d_residual, d_out, N, K);
}

extern "C" int dh_matmul_rmsnorm_f16(const void* d_x, const void* d_W, int transpose_b, const void* d_norm_weight,
                                     int norm_weight_dtype, float eps, int weight_offset, const void* d_residual,
                                     void* d_out, int N, int K) {
  return matmul_rmsnorm_impl<__half>("dh_matmul_rmsnorm_f16", static_cast<const __half*>(d_x),
                                     static_cast<const __half*>(d_W), transpose_b, d_norm_weight, norm_weight_dtype, eps,
                                     weight_offset, static_cast<const __half*>(d_residual), static_cast<__half*>(d_out), N, K);
}
