// runFusedFFN / recordFusedFFN: reference src/gpu/kernels/fused_ffn.js:501-700 (Q4_K weights).
import { getNative, ACT } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { getBuffer, getWeightDtype } from '../weight-buffer.js';
import { noteDispatch } from './constants.js';

function resolveSwigluLimit(value, label) {
  if (value === null || value === undefined) return 0;
  if (!Number.isFinite(value) || value < 0) {
    throw new Error(`[${label}] swigluLimit must be a non-negative finite number, got ${value}.`);
  }
  return value;
}

async function fusedFFN(recorder, input, W_gate, W_up, hiddenSize, intermediateSize, options = {}) {
  const { batchSize = 1, activation = 'silu', alpha = 1.0, outputBuffer = null, swigluLimit } = options;
  const limit = resolveSwigluLimit(swigluLimit, 'FusedFFN');
  const gateDtype = getWeightDtype(W_gate);
  const upDtype = getWeightDtype(W_up);
  if (!gateDtype || !upDtype) {
    throw new Error('Fused FFN requires explicit gate/up weight dtypes');
  }
  if (gateDtype !== upDtype) {
    throw new Error(`Fused FFN requires matching gate/up dtypes (gate=${gateDtype}, up=${upDtype})`);
  }
  if (gateDtype !== 'q4k') {
    throw new Error(`Fused FFN does not support ${gateDtype} weights`);
  }
  if (input.dtype !== 'f32') {
    throw new Error('Fused FFN requires f32 activations');
  }
  if (activation !== 'silu' && activation !== 'gelu') {
    throw new Error(`Fused FFN does not support activation "${activation}"`);
  }
  const outputSize = batchSize * intermediateSize * 4;
  const owned = outputBuffer ? null : acquireBuffer(outputSize, undefined, 'fused_ffn_output');
  const output = outputBuffer || owned;
  try {
    getNative().q4kFfnGateUp(
      getBuffer(input).ptr, getBuffer(W_gate).ptr, getBuffer(W_up).ptr, output.ptr,
      batchSize, hiddenSize, intermediateSize, ACT[activation], alpha, activation === 'silu' ? limit : 0
    );
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
  noteDispatch(recorder, 'fused_ffn');
  return createTensor(output, 'f32', [batchSize, intermediateSize], 'fused_ffn_output');
}

// Gate/up projection + gated activation over RMSNorm(input) in one launch.  Stands in for the
// reference's runFusedFFNFromRMSNormStats / recordFusedFFNFromRMSNormStats
// (src/gpu/kernels/fused_ffn.js:770-860); the inverse RMS the reference takes as a buffer from
// its rmsnorm-stats pass is computed in the kernel prologue, so the argument is `eps` instead.
async function fusedNormedFFN(recorder, input, normWeight, eps, W_gate, W_up, hiddenSize, intermediateSize, options = {}) {
  const { batchSize = 1, activation = 'silu', alpha = 1.0, outputBuffer = null, swigluLimit } = options;
  if (!Number.isInteger(batchSize) || batchSize <= 0) {
    throw new Error(`Fused normed FFN batchSize must be a positive integer; got ${String(batchSize)}.`);
  }
  if (!input || input.dtype !== 'f32') {
    throw new Error(`Fused normed FFN requires f32 prenorm input; got ${String(input && input.dtype)}.`);
  }
  if (!normWeight) {
    throw new Error('Fused normed FFN requires a norm weight buffer.');
  }
  const gateDtype = getWeightDtype(W_gate);
  const upDtype = getWeightDtype(W_up);
  if (gateDtype !== 'q4k' || upDtype !== 'q4k') {
    throw new Error(`Fused normed FFN requires Q4_K gate/up weights; got gate=${gateDtype}, up=${upDtype}.`);
  }
  if (activation !== 'silu' && activation !== 'gelu') {
    throw new Error(`Fused normed FFN activation must be silu|gelu; got ${String(activation)}.`);
  }
  const limit = resolveSwigluLimit(swigluLimit, 'FusedNormedFFN');
  const outputSize = batchSize * intermediateSize * 4;
  const owned = outputBuffer ? null : acquireBuffer(outputSize, undefined, 'fused_normed_ffn_output');
  const output = outputBuffer || owned;
  try {
    getNative().q4kFfnGateUpRmsnorm(
      getBuffer(input).ptr, getBuffer(normWeight).ptr, eps, options.rmsNormWeightOffset === true ? 1 : 0,
      getBuffer(W_gate).ptr, getBuffer(W_up).ptr, output.ptr,
      batchSize, hiddenSize, intermediateSize, ACT[activation], alpha, activation === 'silu' ? limit : 0
    );
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
  noteDispatch(recorder, 'fused_normed_ffn');
  return createTensor(output, 'f32', [batchSize, intermediateSize], 'fused_normed_ffn_output');
}

export async function runFusedNormedFFN(input, normWeight, eps, W_gate, W_up, hiddenSize, intermediateSize, options = {}) {
  return fusedNormedFFN(null, input, normWeight, eps, W_gate, W_up, hiddenSize, intermediateSize, options);
}

export async function recordFusedNormedFFN(recorder, input, normWeight, eps, W_gate, W_up, hiddenSize, intermediateSize, options = {}) {
  return fusedNormedFFN(recorder, input, normWeight, eps, W_gate, W_up, hiddenSize, intermediateSize, options);
}

export async function runFusedFFN(input, W_gate, W_up, hiddenSize, intermediateSize, options = {}) {
  return fusedFFN(null, input, W_gate, W_up, hiddenSize, intermediateSize, options);
}

export async function recordFusedFFN(recorder, input, W_gate, W_up, hiddenSize, intermediateSize, options = {}) {
  return fusedFFN(recorder, input, W_gate, W_up, hiddenSize, intermediateSize, options);
}
