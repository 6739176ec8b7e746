// runRMSNorm / recordRMSNorm: reference src/gpu/kernels/rmsnorm.js:146-297.
import { getNative, DTYPE } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { getBuffer, getWeightDtype } from '../weight-buffer.js';
import { padToQ4KBlock, ptrOf, noteDispatch } from './constants.js';

function resolveOutputScale(outputScale) {
  if (outputScale === null || outputScale === undefined) return 1;
  const value = Number(outputScale);
  if (!Number.isFinite(value)) {
    throw new Error(`[RMSNorm] outputScale must be finite; got "${String(outputScale)}".`);
  }
  return value;
}

async function rmsnorm(recorder, input, weight, eps, options = {}) {
  const {
    batchSize = 1, hiddenSize = null, residual = null, outputBuffer = null,
    rmsNormWeightOffset = false, preResidual = null, residualSumOutput = null, outputScale = null,
  } = options;
  const scale = resolveOutputScale(outputScale);
  if (input.dtype !== 'f32') {
    throw new Error(`[RMSNorm] the HIP path takes f32 activations, got ${input.dtype}.`);
  }
  const hidden = hiddenSize || input.shape[input.shape.length - 1];
  const weightBuffer = getBuffer(weight);
  const weightDtype = getWeightDtype(weight) === 'f16' ? 'f16' : 'f32';
  if (weightBuffer && weightBuffer.size < hidden * (weightDtype === 'f16' ? 2 : 4)) {
    throw new Error(`[RMSNorm] weight buffer (${weightBuffer.size} bytes) is smaller than hiddenSize=${hidden}.`);
  }
  const outputSize = batchSize * padToQ4KBlock(hidden) * 4;
  const output = outputBuffer || acquireBuffer(outputSize, undefined, 'rmsnorm_output');
  const owned = outputBuffer ? null : output;
  const hasPrenorm = !!preResidual && !!residualSumOutput;
  try {
    getNative().rmsnorm(getBuffer(input).ptr, weightBuffer ? weightBuffer.ptr : null, DTYPE[weightDtype], output.ptr,
      batchSize, hidden, eps, rmsNormWeightOffset ? 1 : 0, ptrOf(preResidual), ptrOf(residual),
      hasPrenorm ? ptrOf(residualSumOutput) : null, scale);
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
  noteDispatch(recorder, 'rmsnorm');
  return createTensor(output, input.dtype, [batchSize, hidden], 'rmsnorm_output');
}

export async function runRMSNorm(input, weight, eps, options = {}) {
  return rmsnorm(null, input, weight, eps, options);
}

export async function recordRMSNorm(recorder, input, weight, eps, options = {}) {
  return rmsnorm(recorder, input, weight, eps, options);
}
