// runSandwichRMSNormPair / runResidualNextRMSNormPair (+ record forms): reference
// src/gpu/kernels/rmsnorm-pair.js:147-266.
import { getNative, DTYPE } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { getBuffer, getWeightDtype } from '../weight-buffer.js';
import { padToQ4KBlock, ptrOf, noteDispatch } from './constants.js';

function inferHiddenSize(input, hiddenSize) {
  if (hiddenSize != null) return hiddenSize;
  const shape = input && input.shape;
  return Array.isArray(shape) && shape.length > 0 ? shape[shape.length - 1] : null;
}

function assertInputs(input, residual, hiddenSize) {
  if (!input || input.dtype !== 'f32') {
    throw new Error(`[rmsnorm_pair] input dtype must be f32; got "${String(input && input.dtype)}".`);
  }
  if (residual && residual.dtype && residual.dtype !== 'f32') {
    throw new Error(`[rmsnorm_pair] residual dtype must be f32; got "${String(residual.dtype)}".`);
  }
  if (!Number.isInteger(hiddenSize) || hiddenSize <= 0) {
    throw new Error('[rmsnorm_pair] hiddenSize must be a positive integer.');
  }
}

function normWeight(weight, hidden, what) {
  const buffer = getBuffer(weight);
  const dtype = getWeightDtype(weight) === 'f16' ? 'f16' : 'f32';
  if (!buffer || buffer.size < hidden * (dtype === 'f16' ? 2 : 4)) {
    throw new Error(`[rmsnorm_pair] ${what} weight buffer is smaller than hiddenSize=${hidden}.`);
  }
  return { ptr: buffer.ptr, dtype: DTYPE[dtype] };
}

async function sandwich(recorder, input, residual, postWeight, preWeight, eps, options = {}) {
  const { batchSize = 1, hiddenSize = null, rmsNormWeightOffset = false, postOutputBuffer = null, preOutputBuffer = null } = options;
  const hidden = inferHiddenSize(input, hiddenSize);
  assertInputs(input, residual, hidden);
  const post = normWeight(postWeight, hidden, 'post');
  const pre = normWeight(preWeight, hidden, 'pre');
  const outputSize = batchSize * padToQ4KBlock(hidden) * 4;
  const postOutput = postOutputBuffer || acquireBuffer(outputSize, undefined, 'rmsnorm_pair_post_output');
  const preOutput = preOutputBuffer || acquireBuffer(outputSize, undefined, 'rmsnorm_pair_pre_output');
  try {
    getNative().rmsnormSandwichPair(getBuffer(input).ptr, ptrOf(residual), post.ptr, post.dtype, pre.ptr, pre.dtype,
      postOutput.ptr, preOutput.ptr, batchSize, hidden, eps, rmsNormWeightOffset ? 1 : 0);
  } catch (error) {
    if (!postOutputBuffer) releaseBuffer(postOutput);
    if (!preOutputBuffer) releaseBuffer(preOutput);
    throw error;
  }
  noteDispatch(recorder, 'rmsnorm_pair');
  return {
    postAttn: createTensor(postOutput, 'f32', [batchSize, hidden], 'rmsnorm_pair_post_output'),
    ffnInput: createTensor(preOutput, 'f32', [batchSize, hidden], 'rmsnorm_pair_pre_output'),
  };
}

async function residualNext(recorder, input, residual, weight, eps, options = {}) {
  const {
    batchSize = 1, hiddenSize = null, rmsNormWeightOffset = false, residualOutputBuffer = null, normOutputBuffer = null,
    outputScale = 1,
  } = options;
  const hidden = inferHiddenSize(input, hiddenSize);
  assertInputs(input, residual, hidden);
  if (!residual) throw new Error('[residual_rmsnorm_pair] a residual tensor is required.');
  const scale = Number(outputScale);
  if (!Number.isFinite(scale)) {
    throw new Error(`[residual_rmsnorm_pair] outputScale must be finite; got "${String(outputScale)}".`);
  }
  const w = normWeight(weight, hidden, 'norm');
  const outputSize = batchSize * padToQ4KBlock(hidden) * 4;
  const residualOutput = residualOutputBuffer || acquireBuffer(outputSize, undefined, 'residual_rmsnorm_pair_residual_output');
  const normOutput = normOutputBuffer || acquireBuffer(outputSize, undefined, 'residual_rmsnorm_pair_norm_output');
  try {
    getNative().residualRmsnormPair(getBuffer(input).ptr, ptrOf(residual), w.ptr, w.dtype, residualOutput.ptr, normOutput.ptr,
      batchSize, hidden, eps, rmsNormWeightOffset ? 1 : 0, scale);
  } catch (error) {
    if (!residualOutputBuffer) releaseBuffer(residualOutput);
    if (!normOutputBuffer) releaseBuffer(normOutput);
    throw error;
  }
  noteDispatch(recorder, 'residual_rmsnorm_pair');
  return {
    residual: createTensor(residualOutput, 'f32', [batchSize, hidden], 'residual_rmsnorm_pair_residual_output'),
    nextInput: createTensor(normOutput, 'f32', [batchSize, hidden], 'residual_rmsnorm_pair_norm_output'),
  };
}

export async function runSandwichRMSNormPair(input, residual, postWeight, preWeight, eps, options = {}) {
  return sandwich(null, input, residual, postWeight, preWeight, eps, options);
}
export async function recordSandwichRMSNormPair(recorder, input, residual, postWeight, preWeight, eps, options = {}) {
  return sandwich(recorder, input, residual, postWeight, preWeight, eps, options);
}
export async function runResidualNextRMSNormPair(input, residual, normWeightTensor, eps, options = {}) {
  return residualNext(null, input, residual, normWeightTensor, eps, options);
}
export async function recordResidualNextRMSNormPair(recorder, input, residual, normWeightTensor, eps, options = {}) {
  return residualNext(recorder, input, residual, normWeightTensor, eps, options);
}
