// runMatmulRMSNormFused / recordMatmulRMSNormFused / shouldUseFusedMatmulRMSNorm /
// selectMatmulRMSNormFusedVariant: reference src/gpu/kernels/fused_matmul_rmsnorm.js:30-312.
// One activation row through a dense weight, RMSNorm over the N outputs, the residual added after
// the norm; all f32, or all f16 with f32 sums (the reference's *_f16 variants).
import { getNative, DTYPE } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { getBuffer, getWeightDtype } from '../weight-buffer.js';
import { ptrOf, noteDispatch } from './constants.js';

// src/config/schema/kernel-thresholds.schema.js:87-88
export const FUSED_MATMUL_THRESHOLDS = Object.freeze({ maxMediumN: 4096, maxMediumK: 8192 });
const WORKGROUP_SIZE_DEFAULT = 256;

// The reference tells an f16 norm weight from an f32 one by the buffer's size (:14-28).
function resolveNormWeightDtype(byteSize, hiddenSize) {
  if (!byteSize || hiddenSize == null) return null;
  if (byteSize >= hiddenSize * 4) return 'f32';
  if (byteSize >= hiddenSize * 2) return 'f16';
  return null;
}

export function selectMatmulRMSNormFusedVariant(N, dtype) {
  if (!dtype) {
    throw new Error('[MatmulRMSNormFused] dtype is required for variant selection.');
  }
  // src/rules/kernels/fused-matmul-rmsnorm.rules.json; informational here, one pair of kernels serves every N
  return (N <= WORKGROUP_SIZE_DEFAULT ? 'small' : 'medium') + (dtype === 'f16' ? '_f16' : '');
}

function assertFusedOptions(options) {
  if (!options || options.transposeB === undefined) {
    throw new Error('[MatmulRMSNormFused] transposeB is required.');
  }
  if (!options || options.rmsNormWeightOffset === undefined) {
    throw new Error('[MatmulRMSNormFused] rmsNormWeightOffset is required.');
  }
}

async function matmulRMSNormFused(recorder, input, weight, normWeight, options) {
  assertFusedOptions(options);
  const { N, K, eps, residual = null, outputBuffer = null, transposeB, rmsNormWeightOffset, label = null } = options;
  if (eps == null) {
    throw new Error('[MatmulRMSNormFused] eps is required.');
  }
  if (!Number.isInteger(N) || !Number.isInteger(K) || N <= 0 || K <= 0) {
    throw new Error(`[MatmulRMSNormFused] N and K must be positive integers: N=${N}, K=${K}`);
  }
  const { maxMediumN } = FUSED_MATMUL_THRESHOLDS;
  if (N > maxMediumN) {
    throw new Error(`[MatmulRMSNormFused] N=${N} exceeds maxMediumN=${maxMediumN}; kernel only supports single-workgroup RMSNorm.`);
  }
  const weightBuffer = getBuffer(weight);
  const normWeightBuffer = getBuffer(normWeight);
  const normWeightDtype = resolveNormWeightDtype(normWeightBuffer.size, N);
  if (!normWeightDtype) {
    throw new Error(
      `[MatmulRMSNormFused] norm weight size (${normWeightBuffer.size} bytes) does not match ` +
      `hiddenSize=${N} (expected ${N * 2} or ${N * 4} bytes).`
    );
  }
  if (!input.dtype) {
    throw new Error('[MatmulRMSNormFused] input dtype is required.');
  }
  selectMatmulRMSNormFusedVariant(N, input.dtype);
  const dtype = input.dtype;
  if (dtype !== 'f32' && dtype !== 'f16') {
    throw new Error(`[MatmulRMSNormFused] the HIP path takes f32 or f16 activations, got ${dtype}.`);
  }
  const elem = dtype === 'f16' ? 2 : 4;
  // the f16 variants take f16 weights, residual and output as well (fused_matmul_rmsnorm_f16.wgsl:41-45)
  const weightDtype = getWeightDtype(weight) || weight.dtype || dtype;
  if (weightDtype !== dtype) {
    throw new Error(`[MatmulRMSNormFused] the HIP path takes dense ${dtype} weights for ${dtype} activations, got ${weightDtype}.`);
  }
  if (input.buffer.size < K * elem || weightBuffer.size < N * K * elem) {
    throw new Error(`[MatmulRMSNormFused] input or weight buffer too small for N=${N}, K=${K}.`);
  }
  const residualBuffer = residual ? (residual.buffer || residual) : null;
  if (residualBuffer && residualBuffer.size < N * elem) {
    throw new Error(`[MatmulRMSNormFused] residual buffer smaller than N=${N} elements.`);
  }
  if (residual && residual.dtype && residual.dtype !== dtype) {
    throw new Error(`[MatmulRMSNormFused] residual dtype must match the input's (${dtype}).`);
  }
  const output = outputBuffer || acquireBuffer(N * elem, undefined, 'matmul_rmsnorm_fused_output');
  const owned = outputBuffer ? null : output;
  try {
    const native = getNative();
    (dtype === 'f16' ? native.matmulRmsnormF16 : native.matmulRmsnormF32)(input.buffer.ptr, weightBuffer.ptr, transposeB ? 1 : 0, normWeightBuffer.ptr,
      DTYPE[normWeightDtype], eps, rmsNormWeightOffset ? 1 : 0, residualBuffer ? residualBuffer.ptr : ptrOf(null),
      output.ptr, N, K);
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
  noteDispatch(recorder, label ? `matmul_rmsnorm_fused:${label}` : 'matmul_rmsnorm_fused');
  return createTensor(output, input.dtype, [1, N], 'matmul_rmsnorm_fused_output');
}

export async function runMatmulRMSNormFused(input, weight, normWeight, options) {
  return matmulRMSNormFused(null, input, weight, normWeight, options);
}

export async function recordMatmulRMSNormFused(recorder, input, weight, normWeight, options) {
  return matmulRMSNormFused(recorder, input, weight, normWeight, options);
}

export function shouldUseFusedMatmulRMSNorm(M, N, K) {
  if (M !== 1) return false;
  const { maxMediumN, maxMediumK } = FUSED_MATMUL_THRESHOLDS;
  if (N > maxMediumN) return false;
  if (typeof K === 'number' && K > maxMediumK) return false;
  return true;
}
