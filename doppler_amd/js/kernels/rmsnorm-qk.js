// runRMSNormQK / recordRMSNormQK: reference src/gpu/kernels/rmsnorm-qk.js:29-128.
import { getNative, DTYPE } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { getBuffer, getWeightDtype } from '../weight-buffer.js';
import { padToQ4KBlock, noteDispatch } from './constants.js';

function assertPositiveInteger(value, name) {
  if (!Number.isInteger(value) || value <= 0) {
    throw new Error(`RMSNorm QK requires a positive integer ${name}, got ${String(value)}.`);
  }
}

export function canUseRMSNormQK(qTensor, kTensor, options = {}) {
  if (options.skipKNorm === true) return false;
  if (!qTensor || !kTensor || qTensor.buffer === kTensor.buffer) return false;
  return qTensor.dtype === kTensor.dtype && qTensor.dtype === 'f32';
}

async function rmsNormQK(recorder, qTensor, kTensor, qWeight, kWeight, eps, options = {}) {
  const { numTokens, numHeads, numKVHeads, headDim, rmsNormWeightOffset = false } = options;
  assertPositiveInteger(numTokens, 'numTokens');
  assertPositiveInteger(numHeads, 'numHeads');
  assertPositiveInteger(numKVHeads, 'numKVHeads');
  assertPositiveInteger(headDim, 'headDim');
  if (qTensor.dtype !== kTensor.dtype) {
    throw new Error(`RMSNorm QK requires matching Q/K dtypes, got ${qTensor.dtype} and ${kTensor.dtype}.`);
  }
  if (qTensor.dtype !== 'f32') {
    throw new Error(`RMSNorm QK: the HIP path takes f32 tensors, got ${qTensor.dtype}.`);
  }
  const qRows = numTokens * numHeads;
  const kRows = numTokens * numKVHeads;
  const qBuffer = getBuffer(qTensor);
  const kBuffer = getBuffer(kTensor);
  if (qBuffer.size < qRows * headDim * 4) throw new Error(`RMSNorm QK: Q input buffer (${qBuffer.size} bytes) is too small.`);
  if (kBuffer.size < kRows * headDim * 4) throw new Error(`RMSNorm QK: K input buffer (${kBuffer.size} bytes) is too small.`);
  const weights = [qWeight, kWeight].map((w, i) => {
    const buffer = getBuffer(w);
    const dtype = getWeightDtype(w) === 'f16' ? 'f16' : 'f32';
    if (!buffer || buffer.size < headDim * (dtype === 'f16' ? 2 : 4)) {
      throw new Error(`RMSNorm QK: ${i ? 'K' : 'Q'} weight buffer is smaller than headDim=${headDim}.`);
    }
    return { buffer, dtype };
  });
  const padded = padToQ4KBlock(headDim);
  let qOut = null;
  let kOut = null;
  try {
    qOut = acquireBuffer(qRows * padded * 4, undefined, 'rmsnorm_qk_q_output');
    kOut = acquireBuffer(kRows * padded * 4, undefined, 'rmsnorm_qk_k_output');
    getNative().rmsnormQK(qBuffer.ptr, kBuffer.ptr, weights[0].buffer.ptr, DTYPE[weights[0].dtype], weights[1].buffer.ptr,
      DTYPE[weights[1].dtype], qOut.ptr, kOut.ptr, qRows, kRows, headDim, eps, rmsNormWeightOffset ? 1 : 0);
  } catch (error) {
    if (qOut) releaseBuffer(qOut);
    if (kOut) releaseBuffer(kOut);
    throw error;
  }
  noteDispatch(recorder, 'rmsnorm_qk');
  return {
    q: createTensor(qOut, qTensor.dtype, [qRows, headDim], 'rmsnorm_qk_q_output'),
    k: createTensor(kOut, kTensor.dtype, [kRows, headDim], 'rmsnorm_qk_k_output'),
  };
}

export async function runRMSNormQK(qTensor, kTensor, qWeight, kWeight, eps, options = {}) {
  return rmsNormQK(null, qTensor, kTensor, qWeight, kWeight, eps, options);
}

export async function recordRMSNormQK(recorder, qTensor, kTensor, qWeight, kWeight, eps, options = {}) {
  return rmsNormQK(recorder, qTensor, kTensor, qWeight, kWeight, eps, options);
}
