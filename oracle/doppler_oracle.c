/*
 * doppler_oracle.c -- CPU restatement of Doppler's per-op JavaScript references.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the HIP library, the Node addon,
 * the JS/Python host code) may link, load or call this file; it exists so that
 * tests, the smoke check and the benchmark's cpu_baseline leg have an independent
 * statement of what every op must compute.
 *
 * Each function follows one reference file (cited as path:line, relative to the
 * reference checkout).  JavaScript numbers are doubles, so every accumulator that
 * is a plain `let sum = 0` in the reference is a `double` here, and every store
 * into a Float32Array is an explicit (float) rounding at the same place.
 *
 * How each function is pinned (all checks live in tests/test_oracle_pins.py):
 *   f16 -> f32            exhaustive 65,536 patterns vs numpy float16; sha256 of the
 *                         9B receipt's block-d.f32 / block-dmin.f32
 *   f32 -> f16 (rne)      vs numpy float16 cast on all f16 midpoints + random grid
 *   6-bit scale unpack    round trip through the reference quantizer's packing rule
 *                         (a different function of the reference) on the real
 *                         Qwen3.5-9B scale/min bits from the receipt
 *   scale = f32(d*sc)     sha256 of 1.57 M decoded scales / minima recorded in the
 *   min   = f32(dmin*mn)  receipt (layer0-ffn-gate-oracle.json: decodedScales,
 *                         decodedMinima)
 *   w = scale*q - min     closed form: single correctly rounded f32 of the exact
 *                         value; brute force vs exact rational arithmetic
 *   nibble order          hand-built blocks: one-hot nibble at a known byte must land
 *                         at element 64*chunk + j (+32 for the high nibble)
 *   q4k matmul            == dequant rows then naive f64 dot; linearity; one-hot
 *                         activation returns a dequantized column; K tail masked
 *   rmsnorm/silu/gelu/
 *   residual/softmax      torch float64 closed forms
 *   rope                  complex multiply; norm preservation; pos 0 == identity
 *   attention             torch scaled_dot_product_attention (f64, repeated KV heads);
 *                         kvLen==1 => O==V; uniform scores => mean of V
 *   argmax                brute force incl. ties -> lowest index, pad excluded
 *   (numpy, oracle/__init__.py)
 *   matmul + rmsnorm      torch float64 matmul and rms_norm; unit weight and identity matrix
 *                         give x / rms(x); both weight layouts agree on W and W^T
 *   finiteness guard      the reference's own vectors (finiteness-overflow-gate.test.js,
 *                         finiteness-guard-status.test.js); first trigger wins
 *
 * Build: see oracle/Makefile (gcc -O2 -fopenmp -shared).
 */
#define _GNU_SOURCE
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define QK_K 256
#define Q4K_BLOCK_BYTES 144

/* ------------------------------------------------------------------------- */
/* f16 helpers                                                                */
/* ------------------------------------------------------------------------- */

/* tests/kernels/reference/dequant.js:6-22, src/converter/quantizer.js:48-65.
 * sign * 2^-14 * frac/1024 for subnormals, sign * 2^(e-15) * (1+frac/1024) otherwise;
 * every intermediate is exact in double, and the result fits f32 exactly. */
float dor_f16_to_f32(uint16_t bits) {
  const int sign = (bits >> 15) & 1;
  const int exp = (bits >> 10) & 0x1f;
  const int frac = bits & 0x3ff;
  double v;
  if (exp == 0) {
    if (frac == 0) return sign ? -0.0f : 0.0f;
    v = ldexp((double)frac / 1024.0, -14);
  } else if (exp == 31) {
    if (frac) return NAN;
    return sign ? -INFINITY : INFINITY;
  } else {
    v = ldexp(1.0 + (double)frac / 1024.0, exp - 15);
  }
  return (float)(sign ? -v : v);
}

/* Round-to-nearest-even f32 -> f16: what WGSL `f16(x)` does on the reference's GPU
 * path for the KV-cache write (src/gpu/kernels/kv_cache_write_f32_to_f16.wgsl:30-31)
 * and what v_cvt_f16_f32 does on gfx950. */
uint16_t dor_f32_to_f16_rne(float value) {
  uint32_t x;
  memcpy(&x, &value, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  const uint32_t absx = x & 0x7fffffffu;
  if (absx > 0x7f800000u) return (uint16_t)(sign | 0x7e00u);       /* NaN */
  if (absx >= 0x477ff000u) return (uint16_t)(sign | 0x7c00u);      /* >= 65520 -> Inf */
  if (absx < 0x33000001u) return (uint16_t)sign;                   /* <= 2^-25 -> 0 */
  int exp = (int)(absx >> 23) - 127;
  uint32_t mant = (absx & 0x7fffffu) | 0x800000u;
  int shift;
  uint32_t base;
  if (exp < -14) {          /* subnormal result: value = mant * 2^(exp-23), unit 2^-24 */
    shift = -exp - 14 + 13; /* 14..24 */
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(exp + 15) << 10;
    mant &= 0x7fffffu;
  }
  uint32_t q = mant >> shift;
  const uint32_t rem = mant & ((1u << shift) - 1u);
  const uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u))) q += 1;
  return (uint16_t)(sign | (base + q));  /* carry into the exponent is the right answer */
}

/* src/inference/kv-cache/types.js:25-43: the reference's host-side KV conversion,
 * round-half-up on the magnitude ((mant + 0x1000) >> 13). Kept so tests can show
 * where it differs from RNE (exact ties only). */
uint16_t dor_f32_to_f16_half_up(float value) {
  uint32_t x;
  memcpy(&x, &value, 4);
  const uint32_t sign = (x >> 16) & 0x8000u;
  int exp = (int)((x >> 23) & 0xff) - 127 + 15;
  uint32_t mant = x & 0x7fffffu;
  if (exp <= 0) {
    if (exp < -10) return (uint16_t)sign;
    mant = (mant | 0x800000u) >> (1 - exp);
    return (uint16_t)(sign | ((mant + 0x1000u) >> 13));
  }
  if (exp >= 31) return (uint16_t)(sign | 0x7c00u | (mant ? 0x200u : 0u));
  return (uint16_t)(sign | ((uint32_t)exp << 10) | ((mant + 0x1000u) >> 13));
}

/* src/converter/quantizer.js:15-46: the converter's truncating conversion. */
uint16_t dor_f32_to_f16_trunc(float value) {
  uint32_t f;
  memcpy(&f, &value, 4);
  const uint32_t sign = (f >> 31) & 1u;
  int exp = (int)((f >> 23) & 0xff);
  uint32_t frac = f & 0x7fffffu;
  if (exp == 0xff) return (uint16_t)((sign << 15) | 0x7c00u | (frac ? 0x200u : 0u));
  if (exp == 0) return (uint16_t)(sign << 15);
  exp = exp - 127 + 15;
  if (exp >= 31) return (uint16_t)((sign << 15) | 0x7c00u);
  if (exp <= 0) {
    if (exp < -10) return (uint16_t)(sign << 15);
    frac = (frac | 0x800000u) >> (1 - exp);
    return (uint16_t)((sign << 15) | (frac >> 13));
  }
  return (uint16_t)((sign << 15) | ((uint32_t)exp << 10) | (frac >> 13));
}

/* Table of all 65,536 widenings, filled from dor_f16_to_f32 by dor_init_tables(); the bulk
 * loops (LM head, attention over the KV cache) read it instead of calling ldexp per element. */
static float g_f16_lut[65536];
static int g_f16_lut_ready = 0;

void dor_init_tables(void) {
  if (g_f16_lut_ready) return;
  for (int i = 0; i < 65536; i++) g_f16_lut[i] = dor_f16_to_f32((uint16_t)i);
  g_f16_lut_ready = 1;
}

static inline float f16_widen(uint16_t bits) {
  return g_f16_lut_ready ? g_f16_lut[bits] : dor_f16_to_f32(bits);
}

void dor_f16_to_f32_array(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = dor_f16_to_f32(in[i]);
}

void dor_f32_to_f16_rne_array(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = dor_f32_to_f16_rne(in[i]);
}

/* ------------------------------------------------------------------------- */
/* Q4_K super-block                                                           */
/* ------------------------------------------------------------------------- */

/* tests/kernels/reference/dequant.js:259-272 (same in
 * tools/lib/q4k-projection-reference.js:26-36): the twelve bytes at block offset 4
 * hold eight 6-bit scales and eight 6-bit mins. */
void dor_q4k_unpack_scale_bits(const uint8_t* block, uint8_t sc[8], uint8_t mn[8]) {
  for (int i = 0; i < 4; i++) {
    sc[i] = block[4 + i] & 0x3f;
    sc[i + 4] = (uint8_t)(((block[4 + i] >> 6) & 0x03) << 4);
    mn[i] = block[8 + i] & 0x3f;
    mn[i + 4] = (uint8_t)(((block[8 + i] >> 6) & 0x03) << 4);
  }
  for (int i = 0; i < 4; i++) {
    sc[i + 4] |= block[12 + i] & 0x0f;
    mn[i + 4] |= (block[12 + i] >> 4) & 0x0f;
  }
}

/* tests/kernels/reference/dequant.js:274-279: `scales` and `mins` are Float32Arrays,
 * so d*bits is rounded to f32 when stored (the product is exact anyway). */
void dor_q4k_block_scales(const uint8_t* block, float scales[8], float mins[8]) {
  uint8_t sc[8], mn[8];
  const double d = dor_f16_to_f32((uint16_t)(block[0] | (block[1] << 8)));
  const double dmin = dor_f16_to_f32((uint16_t)(block[2] | (block[3] << 8)));
  dor_q4k_unpack_scale_bits(block, sc, mn);
  for (int i = 0; i < 8; i++) {
    scales[i] = (float)(d * (double)sc[i]);
    mins[i] = (float)(dmin * (double)mn[i]);
  }
}

/* tests/kernels/reference/dequant.js:253-300 dequantizeQ4_KBlockRef: four chunks of
 * 32 bytes; byte i of chunk c carries element 64c+i (low nibble, sub-block 2c) and
 * element 64c+32+i (high nibble, sub-block 2c+1).  `scale*q - min` is evaluated in
 * double and rounded once to f32 by the Float32Array store. */
void dor_q4k_dequant_block(const uint8_t* block, float out[QK_K]) {
  float scales[8], mins[8];
  dor_q4k_block_scales(block, scales, mins);
  for (int chunk = 0; chunk < 4; chunk++) {
    const int base = chunk * 64;
    const uint8_t* q = block + 16 + chunk * 32;
    const int sb0 = chunk * 2, sb1 = chunk * 2 + 1;
    for (int i = 0; i < 32; i++) {
      const int lo = q[i] & 0x0f;
      const int hi = (q[i] >> 4) & 0x0f;
      out[base + i] = (float)((double)scales[sb0] * lo - (double)mins[sb0]);
      out[base + 32 + i] = (float)((double)scales[sb1] * hi - (double)mins[sb1]);
    }
  }
}

/* Same values as dor_q4k_dequant_block, computed in f32: scale*q is exact in f32 (at most
 * 21 significant bits) so `scale*q - min` rounds once, to the same f32 the double expression
 * rounds to.  Compiled without FMA contraction; tests assert bit equality with the double
 * version.  Used by the matmul loops, where the per-element double arithmetic dominated. */
static void q4k_dequant_block_fast(const uint8_t* block, float* out) {
  float scales[8], mins[8];
  dor_q4k_block_scales(block, scales, mins);
  for (int chunk = 0; chunk < 4; chunk++) {
    const uint8_t* q = block + 16 + chunk * 32;
    float* o = out + chunk * 64;
    const float s0 = scales[chunk * 2], s1 = scales[chunk * 2 + 1];
    const float m0 = mins[chunk * 2], m1 = mins[chunk * 2 + 1];
    for (int i = 0; i < 32; i++) {
      o[i] = s0 * (float)(q[i] & 0x0f) - m0;
      o[32 + i] = s1 * (float)(q[i] >> 4) - m1;
    }
  }
}

void dor_q4k_dequant_blocks_fast(const uint8_t* packed, int64_t num_blocks, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < num_blocks; b++)
    q4k_dequant_block_fast(packed + b * Q4K_BLOCK_BYTES, out + b * QK_K);
}

void dor_q4k_dequant_blocks(const uint8_t* packed, int64_t num_blocks, float* out) {
#pragma omp parallel for schedule(static)
  for (int64_t b = 0; b < num_blocks; b++)
    dor_q4k_dequant_block(packed + b * Q4K_BLOCK_BYTES, out + b * QK_K);
}

/* Decoded per-sub-block scales/minima in `block*8 + sub` order, as
 * tools/lib/q4k-projection-reference.js:134-139 records them. */
void dor_q4k_decoded_scales(const uint8_t* packed, int64_t num_blocks, float* scales,
                            float* mins) {
  for (int64_t b = 0; b < num_blocks; b++)
    dor_q4k_block_scales(packed + b * Q4K_BLOCK_BYTES, scales + b * 8, mins + b * 8);
}

/* tests/kernels/reference/fused-ffn-q4k.js:24-40 dequantQ4KRowsRef: W[N,K] is
 * N*ceil(K/256) blocks, row n starts at block n*ceil(K/256); the padded tail of the
 * last block of a row is dropped. */
void dor_q4k_dequant_rows(const uint8_t* packed, int64_t N, int64_t K, float* out) {
  const int64_t nb = (K + QK_K - 1) / QK_K;
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; n++) {
    float tmp[QK_K];
    for (int64_t b = 0; b < nb; b++) {
      dor_q4k_dequant_block(packed + (n * nb + b) * Q4K_BLOCK_BYTES, tmp);
      const int64_t kbase = b * QK_K;
      const int64_t len = (K - kbase) < QK_K ? (K - kbase) : QK_K;
      memcpy(out + n * K + kbase, tmp, (size_t)len * sizeof(float));
    }
  }
}

/* ------------------------------------------------------------------------- */
/* Q4_K matmul  C[M,N] = alpha * A[M,K] . dequant(W)[N,K]^T                     */
/* ------------------------------------------------------------------------- */

/* tools/lib/q4k-projection-reference.js:82-175 projectQ4KRowWiseReference (M=1) and
 * tests/kernels/reference/fused-ffn-q4k.js:57-68 (M>1): one f64 accumulator per
 * output, k ascending, products of two f32 values (exact in double), only the first
 * K elements of each padded row take part; result stored to f32.  alpha as in
 * tests/kernels/reference/matmul.js:13 (`sum * alpha`). */
void dor_q4k_matmul(const float* A, const uint8_t* W, int64_t M, int64_t N, int64_t K,
                    float alpha, float* C) {
  const int64_t nb = (K + QK_K - 1) / QK_K;
  const int64_t kp = nb * QK_K;
  /* Four rows at a time: four independent accumulators keep the adder busy; each row's own
   * sum still runs over k in ascending order, one f64 add per element. */
#pragma omp parallel
  {
    float* wrow = (float*)malloc((size_t)4 * kp * sizeof(float));
#pragma omp for schedule(static)
    for (int64_t n0 = 0; n0 < N; n0 += 4) {
      const int64_t rows = (N - n0) < 4 ? (N - n0) : 4;
      for (int64_t r = 0; r < rows; r++)
        for (int64_t b = 0; b < nb; b++)
          q4k_dequant_block_fast(W + ((n0 + r) * nb + b) * Q4K_BLOCK_BYTES, wrow + r * kp + b * QK_K);
      for (int64_t m = 0; m < M; m++) {
        const float* a = A + m * K;
        if (rows == 4) {
          double s0 = 0.0, s1 = 0.0, s2 = 0.0, s3 = 0.0;
          const float *w0 = wrow, *w1 = wrow + kp, *w2 = wrow + 2 * kp, *w3 = wrow + 3 * kp;
          for (int64_t k = 0; k < K; k++) {
            const double av = (double)a[k];
            s0 += av * (double)w0[k];
            s1 += av * (double)w1[k];
            s2 += av * (double)w2[k];
            s3 += av * (double)w3[k];
          }
          C[m * N + n0] = (float)(s0 * (double)alpha);
          C[m * N + n0 + 1] = (float)(s1 * (double)alpha);
          C[m * N + n0 + 2] = (float)(s2 * (double)alpha);
          C[m * N + n0 + 3] = (float)(s3 * (double)alpha);
        } else {
          for (int64_t r = 0; r < rows; r++) {
            double sum = 0.0;
            for (int64_t k = 0; k < K; k++) sum += (double)a[k] * (double)wrow[r * kp + k];
            C[m * N + n0 + r] = (float)(sum * (double)alpha);
          }
        }
      }
    }
    free(wrow);
  }
}

/* Dense f16-weight matmul, weights row-major [N,K] ("row" layout):
 * src/inference/pipelines/text/logits/cpu.js:61-88 matmulCPU and
 * tools/lib/q4k-projection-reference.js:177-203 projectF16RowWiseReference. */
void dor_f16w_matmul(const float* A, const uint16_t* W, int64_t M, int64_t N, int64_t K,
                     float alpha, float* C) {
#pragma omp parallel for schedule(static)
  for (int64_t n = 0; n < N; n++) {
    for (int64_t m = 0; m < M; m++) {
      double sum = 0.0;
      const float* a = A + m * K;
      const uint16_t* w = W + n * K;
      for (int64_t k = 0; k < K; k++) sum += (double)a[k] * (double)f16_widen(w[k]);
      C[m * N + n] = (float)(sum * (double)alpha);
    }
  }
}

/* ------------------------------------------------------------------------- */
/* Activations                                                                */
/* ------------------------------------------------------------------------- */

/* tests/kernels/reference/silu.js:1-3 */
static double silu_d(double x) { return x / (1.0 + exp(-x)); }

/* tests/kernels/reference/fused-ffn-q4k.js:12-15 (constant 0.7978845608) */
static double gelu_ffn_d(double x) {
  const double c = 0.7978845608;
  return 0.5 * x * (1.0 + tanh(c * (x + 0.044715 * x * x * x)));
}

/* tests/kernels/reference/gelu.js:4-5,28-37: sqrt(2/pi) in full double precision. */
static double gelu_std_d(double x) {
  const double c = sqrt(2.0 / M_PI);
  const double cdf = 0.5 * (1.0 + tanh(c * (x + 0.044715 * x * x * x)));
  return x * cdf;
}

/* tests/kernels/reference/fused-ffn-q4k.js:17-22 */
static double clamp_swiglu_d(double x, int activation_code, double clamp_max) {
  if (clamp_max <= 0.0 || activation_code != 0) return x;
  if (x < -clamp_max) return -clamp_max;
  if (x > clamp_max) return clamp_max;
  return x;
}

/* tests/kernels/reference/fused-ffn-q4k.js:42-73 fusedFfnQ4KRef:
 * out[m,c] = clamp(act(x.Wg[c]) * (x.Wu[c]) * alpha); activation 0 = silu, 1 = gelu. */
void dor_q4k_ffn_gate_up(const float* X, const uint8_t* Wg, const uint8_t* Wu, int64_t M,
                         int64_t hidden, int64_t inter, float alpha, int activation,
                         float swiglu_limit, float* out) {
  const int64_t nb = (hidden + QK_K - 1) / QK_K;
#pragma omp parallel for schedule(static)
  for (int64_t c = 0; c < inter; c++) {
    float* g = (float*)malloc((size_t)nb * QK_K * sizeof(float));
    float* u = (float*)malloc((size_t)nb * QK_K * sizeof(float));
    for (int64_t b = 0; b < nb; b++) {
      dor_q4k_dequant_block(Wg + (c * nb + b) * Q4K_BLOCK_BYTES, g + b * QK_K);
      dor_q4k_dequant_block(Wu + (c * nb + b) * Q4K_BLOCK_BYTES, u + b * QK_K);
    }
    for (int64_t m = 0; m < M; m++) {
      double gs = 0.0, us = 0.0;
      const float* a = X + m * hidden;
      for (int64_t k = 0; k < hidden; k++) {
        gs += (double)a[k] * (double)g[k];
        us += (double)a[k] * (double)u[k];
      }
      const double act = activation == 0 ? silu_d(gs) : gelu_ffn_d(gs);
      out[m * inter + c] =
          (float)clamp_swiglu_d(act * us * (double)alpha, activation, (double)swiglu_limit);
    }
    free(g);
    free(u);
  }
}

/* Gated activation on two buffers: tests/kernels/reference/silu.js:20-28 siluGatedRef
 * (activation 0) and tests/kernels/reference/gelu.js:28-37 gegluRef (activation 1);
 * the optional clamp is the SwiGLU limit of src/gpu/kernels/silu.wgsl:44-49. */
void dor_act_gate(const float* gate, const float* up, int64_t n, int activation,
                  float swiglu_limit, float* out) {
  for (int64_t i = 0; i < n; i++) {
    const double g = gate[i];
    double v = (activation == 0 ? silu_d(g) : gelu_std_d(g)) * (double)up[i];
    if (activation == 0) v = clamp_swiglu_d(v, 0, (double)swiglu_limit);
    out[i] = (float)v;
  }
}

/* Row-split form [T, 2*dim] -> [T, dim] (src/gpu/kernels/silu.wgsl:83-98,
 * gelu.wgsl:37-52): gate = row[0:dim], up = row[dim:2dim]. */
void dor_act_gate_rowsplit(const float* in, int64_t T, int64_t dim, int activation,
                           float swiglu_limit, float* out) {
  for (int64_t t = 0; t < T; t++)
    dor_act_gate(in + t * 2 * dim, in + t * 2 * dim + dim, dim, activation, swiglu_limit,
                 out + t * dim);
}

/* tests/kernels/reference/residual.js:55-63 outputScaledResidualAddRef:
 * (x + r) * scale (scale 1 gives residualAddRef :3-11). */
void dor_residual_add(const float* a, const float* b, int64_t n, float scale, float* out) {
  for (int64_t i = 0; i < n; i++) out[i] = (float)(((double)a[i] + (double)b[i]) * (double)scale);
}

/* ------------------------------------------------------------------------- */
/* RMSNorm                                                                    */
/* ------------------------------------------------------------------------- */

/* tests/kernels/reference/rmsnorm.js:4-28 rmsNormRef with the wrapper's options
 * (src/gpu/kernels/rmsnorm.js:152-156, rmsnorm.wgsl:88-111,166-185):
 *   x      = input (+ pre_residual)           [PRE_RESIDUAL]
 *   prenorm_out = x                            [OUTPUT_PRENORM]
 *   y      = x * 1/sqrt(mean(x^2)+eps) * (w | 1+w)
 *   y     += post_residual                     [has_residual]
 *   y     *= output_scale
 * Arithmetic is double with one f32 rounding at the store, like the reference. */
void dor_rmsnorm(const float* input, const float* weight, int64_t batch, int64_t hidden,
                 float eps, int weight_offset, const float* pre_residual,
                 const float* post_residual, float* prenorm_out, float output_scale,
                 float* out) {
  for (int64_t b = 0; b < batch; b++) {
    const int64_t off = b * hidden;
    double sum_sq = 0.0;
    for (int64_t i = 0; i < hidden; i++) {
      double v = input[off + i];
      if (pre_residual) v = (double)(float)(v + (double)pre_residual[off + i]);
      sum_sq += v * v;
    }
    const double scale = 1.0 / sqrt(sum_sq / (double)hidden + (double)eps);
    for (int64_t i = 0; i < hidden; i++) {
      double v = input[off + i];
      if (pre_residual) v = (double)(float)(v + (double)pre_residual[off + i]);
      if (prenorm_out) prenorm_out[off + i] = (float)v;
      const double w = weight ? (weight_offset ? 1.0 + (double)weight[i] : (double)weight[i]) : 1.0;
      double y = v * scale * w;
      if (post_residual) y += (double)post_residual[off + i];
      out[off + i] = (float)(y * (double)output_scale);
    }
  }
}

/* ------------------------------------------------------------------------- */
/* RoPE                                                                       */
/* ------------------------------------------------------------------------- */

/* Table builders.  recipe 0: tests/kernels/reference/rope.js:4-19 computeRopeFreqs
 * (frequency kept in double).  recipe 1: src/inference/pipelines/text/init-rope.js:
 * 21-26,120-133 (frequency rounded to f32 first, linear scale `rope_scale`,
 * magnitude 1).  Both store cos/sin as f32, layout [pos][dim/2]. */
void dor_rope_tables(int64_t rotary_dim, int64_t max_seq, double theta, int recipe,
                     double rope_scale, float* cos_out, float* sin_out) {
  const int64_t half = rotary_dim / 2;
  for (int64_t pos = 0; pos < max_seq; pos++) {
    for (int64_t i = 0; i < half; i++) {
      double freq = 1.0 / pow(theta, (double)(2 * i) / (double)rotary_dim);
      double angle;
      if (recipe == 1) {
        freq = (double)(float)freq;
        const double scaled_pos = (double)pos / (double)(float)rope_scale;
        angle = scaled_pos * freq;
      } else {
        angle = (double)pos * freq;
      }
      cos_out[pos * half + i] = (float)cos(angle);
      sin_out[pos * half + i] = (float)sin(angle);
    }
  }
}

/* tests/kernels/reference/rope.js:22-49 ropeRef (rotate-half; partner at
 * +pairSpanDim/2) and :52-77 ropeInterleavedRef (adjacent pairs).  x is
 * [seq][heads][head_dim] f32; out may alias a copy of x, not x itself. */
void dor_rope_apply(const float* x, const float* cos_t, const float* sin_t, int64_t seq,
                    int64_t heads, int64_t head_dim, int64_t start_pos, int64_t rotary_dim,
                    int64_t pair_span_dim, int interleaved, float* out) {
  const int64_t half = rotary_dim / 2;
  const int64_t partner = pair_span_dim / 2;
  memcpy(out, x, (size_t)(seq * heads * head_dim) * sizeof(float));
  for (int64_t s = 0; s < seq; s++) {
    const int64_t pos = s + start_pos;
    for (int64_t h = 0; h < heads; h++) {
      const int64_t off = (s * heads + h) * head_dim;
      for (int64_t i = 0; i < half; i++) {
        const int64_t i0 = interleaved ? 2 * i : i;
        const int64_t i1 = interleaved ? 2 * i + 1 : i + partner;
        const double x0 = x[off + i0], x1 = x[off + i1];
        const double c = cos_t[pos * half + i], sn = sin_t[pos * half + i];
        out[off + i0] = (float)(x0 * c - x1 * sn);
        out[off + i1] = (float)(x0 * sn + x1 * c);
      }
    }
  }
}

/* ------------------------------------------------------------------------- */
/* Attention                                                                  */
/* ------------------------------------------------------------------------- */

/* tests/kernels/reference/attention.js:4-63 attentionRef, with the rounding points of
 * its Float32Array `scores` kept (score*scale, exp(), p/sum are each stored as f32)
 * and an additive mask [seq][kvLen] (0 / -inf, createCausalMask :129-144).
 * Q [seq][H][D], K,V [kvLen][Hkv][D], all f32; scale is 1/sqrt(D) when scale<=0. */
void dor_attention_ref(const float* Q, const float* K, const float* V, int64_t seq,
                       int64_t kv_len, int64_t H, int64_t Hkv, int64_t D, const float* mask,
                       float scale_in, float* out) {
  const double scale = scale_in > 0.0f ? (double)scale_in : 1.0 / sqrt((double)D);
  const int64_t per_kv = H / Hkv;
#pragma omp parallel for collapse(2) schedule(static)
  for (int64_t h = 0; h < H; h++) {
    for (int64_t q = 0; q < seq; q++) {
      const int64_t kvh = h / per_kv;
      float* scores = (float*)malloc((size_t)kv_len * sizeof(float));
      for (int64_t k = 0; k < kv_len; k++) {
        double s = 0.0;
        const float* qv = Q + (q * H + h) * D;
        const float* kv = K + (k * Hkv + kvh) * D;
        for (int64_t d = 0; d < D; d++) s += (double)qv[d] * (double)kv[d];
        scores[k] = (float)(s * scale);
        if (mask) scores[k] = (float)((double)scores[k] + (double)mask[q * kv_len + k]);
      }
      double mx = -INFINITY;
      for (int64_t k = 0; k < kv_len; k++) mx = fmax(mx, (double)scores[k]);
      double sum = 0.0;
      for (int64_t k = 0; k < kv_len; k++) {
        scores[k] = (float)exp((double)scores[k] - mx);
        sum += (double)scores[k];
      }
      for (int64_t k = 0; k < kv_len; k++) scores[k] = (float)((double)scores[k] / sum);
      for (int64_t d = 0; d < D; d++) {
        double val = 0.0;
        for (int64_t k = 0; k < kv_len; k++)
          val += (double)scores[k] * (double)V[(k * Hkv + kvh) * D + d];
        out[(q * H + h) * D + d] = (float)val;
      }
      free(scores);
    }
  }
}

/* Decode attention (one query token) over an f16 KV cache with the options of
 * src/gpu/kernels/attention_decode_online_f16kv.wgsl:61-82,140-243 that attentionRef
 * lacks: explicit scale, soft cap, causal and sliding-window masking on absolute
 * positions (abs_key = kv_start + k, abs_query = start_pos), ring layout
 * (kv_layout 1: physical row = abs_key % sliding_window).  Softmax as attentionRef.
 * kv_len == 0 or every key masked gives zeros (:105-113,236). */
void dor_attention_decode_f16kv(const float* Q, const uint16_t* K, const uint16_t* V,
                                int64_t H, int64_t Hkv, int64_t D, int64_t kv_len,
                                float scale_in, int causal, int64_t start_pos, float softcap,
                                int64_t sliding_window, int64_t kv_start, int kv_layout,
                                float* out) {
  const double scale = (double)scale_in;
  const int64_t per_kv = H / Hkv;
#pragma omp parallel for schedule(static)
  for (int64_t h = 0; h < H; h++) {
    const int64_t kvh = h / per_kv;
    float* scores = (float*)malloc((size_t)(kv_len > 0 ? kv_len : 1) * sizeof(float));
    int64_t* rows = (int64_t*)malloc((size_t)(kv_len > 0 ? kv_len : 1) * sizeof(int64_t));
    int any = 0;
    for (int64_t k = 0; k < kv_len; k++) {
      const int64_t abs_key = kv_start + k;
      int masked = 0;
      if (causal && abs_key > start_pos) masked = 1;
      if (sliding_window > 0 && start_pos >= sliding_window &&
          abs_key < start_pos - sliding_window + 1)
        masked = 1;
      int64_t row = abs_key;
      if (kv_layout == 1 && sliding_window > 0) row = abs_key % sliding_window;
      rows[k] = row;
      if (masked) {
        scores[k] = -INFINITY;
        continue;
      }
      any = 1;
      double s = 0.0;
      const float* qv = Q + h * D;
      const uint16_t* kv = K + (row * Hkv + kvh) * D;
      for (int64_t d = 0; d < D; d++) s += (double)qv[d] * (double)f16_widen(kv[d]);
      s = (double)(float)(s * scale);
      if (softcap > 0.0f) s = (double)(float)(tanh(s / (double)softcap) * (double)softcap);
      scores[k] = (float)s;
    }
    if (!any) {
      for (int64_t d = 0; d < D; d++) out[h * D + d] = 0.0f;
    } else {
      double mx = -INFINITY;
      for (int64_t k = 0; k < kv_len; k++) mx = fmax(mx, (double)scores[k]);
      double sum = 0.0;
      for (int64_t k = 0; k < kv_len; k++) {
        scores[k] = (float)exp((double)scores[k] - mx);
        sum += (double)scores[k];
      }
      for (int64_t k = 0; k < kv_len; k++) scores[k] = (float)((double)scores[k] / sum);
      for (int64_t d = 0; d < D; d++) {
        double val = 0.0;
        for (int64_t k = 0; k < kv_len; k++)
          val += (double)scores[k] * (double)f16_widen(V[(rows[k] * Hkv + kvh) * D + d]);
        out[h * D + d] = (float)val;
      }
    }
    free(scores);
    free(rows);
  }
}

/* ------------------------------------------------------------------------- */
/* KV-cache write, fused q/k-norm + RoPE + KV write, gather, argmax           */
/* ------------------------------------------------------------------------- */

/* src/gpu/kernels/kv_cache_write_f32_to_f16.wgsl:18-32 */
void dor_kv_write_f16(const float* k, const float* v, int64_t src_off, int64_t dst_off,
                      int64_t count, uint16_t* out_k, uint16_t* out_v) {
  for (int64_t i = 0; i < count; i++) {
    out_k[dst_off + i] = dor_f32_to_f16_rne(k[src_off + i]);
    out_v[dst_off + i] = dor_f32_to_f16_rne(v[src_off + i]);
  }
}

/* src/gpu/kernels/split_qkv_rmsnorm_rope_qk_f16kv_cache.wgsl:168-217: from the fused
 * projection qkv[T][q_size+k_size+v_size] (f32): per-head RMSNorm with q/k weights,
 * RoPE at position start_pos+t (rotate-half partner at +rotary_dim/2, or interleaved),
 * Q out f32 [T*H][D]; K and V narrowed to f16 at element kv_dst_offset of the caches.
 * Composition of dor_rmsnorm and dor_rope_apply with one f32 rounding after the norm
 * is NOT what the kernel does: it rotates the unrounded normalised values, so this
 * function does the same in double and rounds once at the store. */
void dor_qkv_norm_rope_kvwrite(const float* qkv, const float* q_weight, const float* k_weight,
                               const float* cos_t, const float* sin_t, int64_t T, int64_t H,
                               int64_t Hkv, int64_t D, int64_t start_pos, int64_t rotary_dim,
                               int interleaved, float eps, int weight_offset,
                               int64_t kv_dst_offset, float* q_out, uint16_t* cache_k,
                               uint16_t* cache_v) {
  const int64_t q_size = H * D, k_size = Hkv * D, v_size = Hkv * D;
  const int64_t stride = q_size + k_size + v_size;
  const int64_t half = rotary_dim / 2;
  double* tmp = (double*)malloc((size_t)D * sizeof(double));
  for (int64_t t = 0; t < T; t++) {
    for (int64_t r = 0; r < H + Hkv; r++) {
      const int is_q = r < H;
      const int64_t head = is_q ? r : r - H;
      const float* src = qkv + t * stride + (is_q ? 0 : q_size) + head * D;
      const float* w = is_q ? q_weight : k_weight;
      double ss = 0.0;
      for (int64_t i = 0; i < D; i++) ss += (double)src[i] * (double)src[i];
      const double inv = 1.0 / sqrt(ss / (double)D + (double)eps);
      for (int64_t i = 0; i < D; i++)
        tmp[i] = (double)src[i] * inv * (weight_offset ? 1.0 + (double)w[i] : (double)w[i]);
      const int64_t pos = start_pos + t;
      for (int64_t i = 0; i < half; i++) {
        const int64_t i0 = interleaved ? 2 * i : i;
        const int64_t i1 = interleaved ? 2 * i + 1 : i + half;
        const double c = cos_t[pos * half + i], sn = sin_t[pos * half + i];
        const double x0 = tmp[i0], x1 = tmp[i1];
        tmp[i0] = x0 * c - x1 * sn;
        tmp[i1] = x0 * sn + x1 * c;
      }
      for (int64_t i = 0; i < D; i++) {
        if (is_q)
          q_out[(t * H + head) * D + i] = (float)tmp[i];
        else
          cache_k[kv_dst_offset + (t * Hkv + head) * D + i] = dor_f32_to_f16_rne((float)tmp[i]);
      }
    }
    for (int64_t i = 0; i < v_size; i++)
      cache_v[kv_dst_offset + t * v_size + i] =
          dor_f32_to_f16_rne(qkv[t * stride + q_size + k_size + i]);
  }
  free(tmp);
}

/* src/gpu/kernels/gather_f16.wgsl:35-66: out[t,:] = f32(E[id_t, :]); an id outside
 * the vocabulary gives a zero row. */
void dor_gather_f16(const uint32_t* ids, const uint16_t* table, int64_t T, int64_t hidden,
                    int64_t vocab, float* out) {
  for (int64_t t = 0; t < T; t++) {
    for (int64_t i = 0; i < hidden; i++)
      out[t * hidden + i] =
          ids[t] >= (uint32_t)vocab ? 0.0f : f16_widen(table[(int64_t)ids[t] * hidden + i]);
  }
}

/* tests/kernels/reference/sample.js:4-16 argmaxRef (strict `>`: first maximum wins)
 * with the kernel's extras (src/gpu/kernels/sample.wgsl:35-51,311-335): optional soft
 * cap softcap*tanh(x/softcap), and a pad id that can never win (pad_id < 0: none).
 * Starting point is (-3.402823e38, index 0) as in the kernel. */
int64_t dor_argmax(const float* logits, int64_t vocab, int64_t pad_id, float softcap) {
  int64_t best = 0;
  float best_val = -3.402823e+38f;
  for (int64_t i = 0; i < vocab; i++) {
    if (i == pad_id) continue;
    float v = logits[i];
    if (softcap > 0.0f) v = (float)((double)softcap * tanh((double)v / (double)softcap));
    if (v > best_val) {
      best_val = v;
      best = i;
    }
  }
  return best;
}

/* Top-k temperature sampling.  tests/kernels/reference/sample.js:62-92 (sampleTopKRef):
 * below temperature 0.01 plain argmax; otherwise the top_k logits by value (stable: among
 * equal values the lower index first, as Array.prototype.sort on {val, idx} gives), softmax of
 * value / temperature over those in f64, then the first candidate at which the running sum of
 * probabilities reaches random_value (last candidate if none does).  Soft cap and pad id as in
 * dor_argmax (the kernel's extras). */
int64_t dor_sample_topk(const float* logits, int64_t vocab, double temperature, int64_t top_k,
                        double random_value, int64_t pad_id, float softcap) {
  if (temperature < 0.01) return dor_argmax(logits, vocab, pad_id, softcap);
  if (top_k > vocab) top_k = vocab;
  int64_t* idx = (int64_t*)malloc((size_t)top_k * sizeof(int64_t));
  double* val = (double*)malloc((size_t)top_k * sizeof(double));
  int64_t n = 0;
  for (int64_t i = 0; i < vocab; i++) {            /* insertion into the sorted top-k list */
    if (i == pad_id) continue;
    float v = logits[i];
    if (softcap > 0.0f) v = (float)((double)softcap * tanh((double)v / (double)softcap));
    if (n == top_k && !((double)v > val[n - 1])) continue;   /* equal to the last: later index loses */
    int64_t p = n < top_k ? n : top_k - 1;
    while (p > 0 && (double)v > val[p - 1]) {
      val[p] = val[p - 1];
      idx[p] = idx[p - 1];
      p--;
    }
    val[p] = (double)v;
    idx[p] = i;
    if (n < top_k) n++;
  }
  double mx = -INFINITY, sum = 0.0;
  for (int64_t i = 0; i < n; i++) {
    val[i] = val[i] / temperature;
    if (val[i] > mx) mx = val[i];
  }
  for (int64_t i = 0; i < n; i++) {
    val[i] = exp(val[i] - mx);
    sum += val[i];
  }
  int64_t pick = n > 0 ? idx[n - 1] : 0;
  double cum = 0.0;
  for (int64_t i = 0; i < n; i++) {
    cum += val[i] / sum;
    if (cum >= random_value) {
      pick = idx[i];
      break;
    }
  }
  free(idx);
  free(val);
  return pick;
}

/* Math.sin based generator of the reference, tests/kernels/reference/sample.js:94-97. */
double dor_seeded_random(double seed) {
  const double x = sin(seed) * 10000.0;
  return x - floor(x);
}

/* ------------------------------------------------------------------------- */
/* Whole decoder step (test/bench driver; op order follows the execution graph */
/* src/config/conversion/qwen3/qwen-3-embedding-0-6b-q4k-ehf16-af32.json       */
/* `execution.decode`: input_norm -> q,k,v -> q/k-norm + rope -> KV write ->   */
/* attention -> o_proj -> +residual -> post_attn_norm -> gate,up -> silu*up -> */
/* down -> +residual; then final_norm -> tied LM head -> argmax)               */
/* ------------------------------------------------------------------------- */

typedef struct {
  int64_t layers, hidden, inter, heads, kv_heads, head_dim, vocab, max_seq;
  float eps;
  int qk_norm; /* per-head q/k RMSNorm (Qwen3); 0 = plain RoPE */
} dor_model_cfg;

typedef struct {
  const uint8_t *wq, *wk, *wv, *wo, *wgate, *wup, *wdown; /* Q4_K rows */
  const float *input_norm, *post_attn_norm, *q_norm, *k_norm;
  uint16_t *cache_k, *cache_v; /* [max_seq][kv_heads][head_dim] f16 */
} dor_layer;

/* One token: id at position pos (KV rows 0..pos-1 already present).  logits_out may
 * be NULL.  Returns the greedy token. */
int64_t dor_decode_step(const dor_model_cfg* cfg, const dor_layer* layers,
                        const uint16_t* embed, const float* final_norm, const float* cos_t,
                        const float* sin_t, uint32_t token, int64_t pos, float* logits_out) {
  const int64_t Hd = cfg->hidden, H = cfg->heads, Hkv = cfg->kv_heads, D = cfg->head_dim;
  const int64_t qs = H * D, ks = Hkv * D;
  float* x = (float*)malloc((size_t)Hd * 4);
  float* normed = (float*)malloc((size_t)Hd * 4);
  float* qkv = (float*)malloc((size_t)(qs + 2 * ks) * 4);
  float* q = (float*)malloc((size_t)qs * 4);
  float* attn = (float*)malloc((size_t)qs * 4);
  float* proj = (float*)malloc((size_t)Hd * 4);
  float* gate = (float*)malloc((size_t)cfg->inter * 4);
  float* up = (float*)malloc((size_t)cfg->inter * 4);
  float* act = (float*)malloc((size_t)cfg->inter * 4);
  dor_gather_f16(&token, embed, 1, Hd, cfg->vocab, x);
  for (int64_t l = 0; l < cfg->layers; l++) {
    const dor_layer* L = &layers[l];
    dor_rmsnorm(x, L->input_norm, 1, Hd, cfg->eps, 0, NULL, NULL, NULL, 1.0f, normed);
    dor_q4k_matmul(normed, L->wq, 1, qs, Hd, 1.0f, qkv);
    dor_q4k_matmul(normed, L->wk, 1, ks, Hd, 1.0f, qkv + qs);
    dor_q4k_matmul(normed, L->wv, 1, ks, Hd, 1.0f, qkv + qs + ks);
    if (cfg->qk_norm) {
      dor_qkv_norm_rope_kvwrite(qkv, L->q_norm, L->k_norm, cos_t, sin_t, 1, H, Hkv, D, pos, D,
                                0, cfg->eps, 0, pos * ks, q, L->cache_k, L->cache_v);
    } else {
      /* unit-weight norm is not the same as no norm: rotate raw q,k instead */
      float* kr = (float*)malloc((size_t)ks * 4);
      dor_rope_apply(qkv, cos_t, sin_t, 1, H, D, pos, D, D, 0, q);
      dor_rope_apply(qkv + qs, cos_t, sin_t, 1, Hkv, D, pos, D, D, 0, kr);
      dor_kv_write_f16(kr, qkv + qs + ks, 0, pos * ks, ks, L->cache_k, L->cache_v);
      free(kr);
    }
    dor_attention_decode_f16kv(q, L->cache_k, L->cache_v, H, Hkv, D, pos + 1,
                               (float)(1.0 / sqrt((double)D)), 1, pos, 0.0f, 0, 0, 0, attn);
    dor_q4k_matmul(attn, L->wo, 1, Hd, qs, 1.0f, proj);
    dor_residual_add(proj, x, Hd, 1.0f, x);
    dor_rmsnorm(x, L->post_attn_norm, 1, Hd, cfg->eps, 0, NULL, NULL, NULL, 1.0f, normed);
    dor_q4k_matmul(normed, L->wgate, 1, cfg->inter, Hd, 1.0f, gate);
    dor_q4k_matmul(normed, L->wup, 1, cfg->inter, Hd, 1.0f, up);
    dor_act_gate(gate, up, cfg->inter, 0, 0.0f, act);
    dor_q4k_matmul(act, L->wdown, 1, Hd, cfg->inter, 1.0f, proj);
    dor_residual_add(proj, x, Hd, 1.0f, x);
  }
  dor_rmsnorm(x, final_norm, 1, Hd, cfg->eps, 0, NULL, NULL, NULL, 1.0f, normed);
  float* logits = logits_out ? logits_out : (float*)malloc((size_t)cfg->vocab * 4);
  dor_f16w_matmul(normed, embed, 1, cfg->vocab, Hd, 1.0f, logits);
  const int64_t tok = dor_argmax(logits, cfg->vocab, -1, 0.0f);
  if (!logits_out) free(logits);
  free(x); free(normed); free(qkv); free(q); free(attn); free(proj);
  free(gate); free(up); free(act);
  return tok;
}
