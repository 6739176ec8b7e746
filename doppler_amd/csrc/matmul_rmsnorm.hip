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

// W is [N, K]: a wave per output row and K slice, lanes stride over the slice in 16-byte pieces,
// four loads in flight per lane.  parts[slice][n] receives the wave's sum.
__global__ __launch_bounds__(256) void gemv_rows_kernel(const float* __restrict__ x, const float* __restrict__ W,
                                                        float* __restrict__ parts, int N, int K, int k_per_slice,
                                                        int vec) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= N) return;
  const int k0 = blockIdx.y * k_per_slice;
  const int k1 = min(K, k0 + k_per_slice);
  const float* row = W + (int64_t)n * K;
  float acc = 0.f;
  if (vec) {
    // k_per_slice is a multiple of 4 here, so is K
    const float4* row4 = reinterpret_cast<const float4*>(row);
    const float4* x4 = reinterpret_cast<const float4*>(x);
    const int q1 = k1 >> 2;
    int k = (k0 >> 2) + lane;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
    for (; k + 192 < q1; k += 256) {
      const float4 w0 = row4[k], w1 = row4[k + 64], w2 = row4[k + 128], w3 = row4[k + 192];
      const float4 v0 = x4[k], v1 = x4[k + 64], v2 = x4[k + 128], v3 = x4[k + 192];
      a0 += w0.x * v0.x + w0.y * v0.y + w0.z * v0.z + w0.w * v0.w;
      a1 += w1.x * v1.x + w1.y * v1.y + w1.z * v1.z + w1.w * v1.w;
      a2 += w2.x * v2.x + w2.y * v2.y + w2.z * v2.z + w2.w * v2.w;
      a3 += w3.x * v3.x + w3.y * v3.y + w3.z * v3.z + w3.w * v3.w;
    }
    for (; k < q1; k += 64) {
      const float4 w = row4[k];
      const float4 v = x4[k];
      a0 += w.x * v.x + w.y * v.y + w.z * v.z + w.w * v.w;
    }
    acc = (a0 + a1) + (a2 + a3);
  } else {
    for (int k = k0 + lane; k < k1; k += 64) acc += row[k] * x[k];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
  if (lane == 0) parts[(int64_t)blockIdx.y * N + n] = acc;
}

// W is [K, N]: a workgroup of 16 waves covers 256 output columns (64 lanes x 4) and one slice of K;
// wave w takes rows w, w + 16, ... of the slice, four rows in flight, and the waves meet in LDS in
// wave order.  parts[slice][n] receives the sum.
constexpr int kColsWaves = 16;
__global__ __launch_bounds__(kColsWaves * 64) void gemv_cols_kernel(const float* __restrict__ x,
                                                                    const float* __restrict__ W,
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
      const float* col = W + n0;
      int k = k0 + wave;
      for (; k + 3 * kColsWaves < k1; k += 4 * kColsWaves) {
        float4 w[4];
        float v[4];
#pragma unroll
        for (int u = 0; u < 4; u++) {
          w[u] = *reinterpret_cast<const float4*>(col + (int64_t)(k + u * kColsWaves) * N);
          v[u] = x[k + u * kColsWaves];
        }
#pragma unroll
        for (int u = 0; u < 4; u++) {
          acc[0] += w[u].x * v[u]; acc[1] += w[u].y * v[u]; acc[2] += w[u].z * v[u]; acc[3] += w[u].w * v[u];
        }
      }
      for (; k < k1; k += kColsWaves) {
        const float4 w = *reinterpret_cast<const float4*>(col + (int64_t)k * N);
        const float v = x[k];
        acc[0] += w.x * v; acc[1] += w.y * v; acc[2] += w.z * v; acc[3] += w.w * v;
      }
    }
  } else {
    for (int k = k0 + wave; k < k1; k += kColsWaves) {
      const float v = x[k];
      const float* row = W + (int64_t)k * N;
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (n0 + j < N) acc[j] += row[n0 + j] * v;
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
__global__ __launch_bounds__(kFinishThreads) void rmsnorm_finish_kernel(const float* __restrict__ parts, int slices,
                                                                        const void* __restrict__ norm_weight,
                                                                        int weight_f16, int weight_offset,
                                                                        const float* __restrict__ residual,
                                                                        float* __restrict__ out, int N, float eps) {
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
    if (residual) r += residual[n];
    out[n] = r;
  }
}

}  // namespace

extern "C" int dh_matmul_rmsnorm_f32(const float* d_x, const float* d_W, int transpose_b, const void* d_norm_weight,
                                     int norm_weight_dtype, float eps, int weight_offset, const float* d_residual,
                                     float* d_out, int N, int K) {
  const char* op = "dh_matmul_rmsnorm_f32";
  DH_REQUIRE_INIT(op);
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
    const int vec = (K % 4 == 0) && ((reinterpret_cast<uintptr_t>(d_W) | reinterpret_cast<uintptr_t>(d_x)) % 16 == 0);
    // about 16 waves per compute unit, at least 1024 elements of a row per wave
    slices = std::max(1, std::min<int>((int)(K / 1024), (int)dh::ceil_div(16 * dh::num_cus(), N)));
    const int k_per_slice = (int)dh::ceil_div(dh::ceil_div(K, slices), 4) * 4;
    slices = (int)dh::ceil_div(K, k_per_slice);
    if ((size_t)(slices + 1) * N * sizeof(float) > ws_bytes)
      return dh::fail(2, "[%s] internal: %d slices of %d floats do not fit the workspace", op, slices, N);
    hipLaunchKernelGGL(gemv_rows_kernel, dim3((unsigned)dh::ceil_div(N, 4), slices), dim3(256), 0, dh::stream(), d_x,
                       d_W, parts, N, K, k_per_slice, vec);
  } else {
    const int col_blocks = (int)dh::ceil_div(N, 256);
    // about two workgroups of 16 waves per compute unit, at least 64 rows of W each
    slices = std::max(1, std::min<int>((int)(K / 64), (int)dh::ceil_div(2 * dh::num_cus(), col_blocks)));
    const int k_per_slice = (int)dh::ceil_div(K, slices);
    slices = (int)dh::ceil_div(K, k_per_slice);
    if ((size_t)(slices + 1) * N * sizeof(float) > ws_bytes)
      return dh::fail(2, "[%s] internal: %d slices of %d floats do not fit the workspace", op, slices, N);
    const int vec = (N % 4 == 0) && (reinterpret_cast<uintptr_t>(d_W) % 16 == 0);
    hipLaunchKernelGGL(gemv_cols_kernel, dim3(col_blocks, slices), dim3(kColsWaves * 64), 0, dh::stream(), d_x, d_W,
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
  hipLaunchKernelGGL(rmsnorm_finish_kernel, dim3(1), dim3(kFinishThreads), 0, dh::stream(), parts, slices,
                     d_norm_weight, norm_weight_dtype == DH_F16, weight_offset, d_residual, d_out, N, eps);
  DH_CHECK_LAUNCH(op);
  return 0;
}
