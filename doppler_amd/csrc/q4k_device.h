// Device helpers shared by the Q4_K kernels (GEMV and GEMM): f16 field access, 6-bit
// scale/min decode, gated activations.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include <cstdint>

namespace {

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

__device__ __forceinline__ float act_silu(float x) { return x / (1.0f + __expf(-x)); }
__device__ __forceinline__ float act_gelu(float x) {
  const float inner = 0.7978845608f * (x + 0.044715f * x * x * x);
  return 0.5f * x * (1.0f + tanhf(fminf(fmaxf(inner, -15.0f), 15.0f)));
}

}  // namespace
