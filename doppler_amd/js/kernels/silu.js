// Gated SiLU ops: reference src/gpu/kernels/silu.js:95-169 (runSiLU with `gate`),
// :230-347 (runSiLURowSplit / recordSiLURowSplit), :349+ (recordSiLU).
import { getNative, ACT } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { bufferOf, noteDispatch } from './constants.js';

function resolveSwigluLimit(value, label) {
  if (value === null || value === undefined) return 0;
  if (!Number.isFinite(value) || value < 0) {
    throw new Error(`[${label}] swigluLimit must be a non-negative finite number, got ${value}.`);
  }
  return value;
}

async function silu(recorder, input, options = {}) {
  const { size, gate = null, outputBuffer = null, swigluLimit, gateActivation = 'silu' } = options;
  const limit = resolveSwigluLimit(swigluLimit, 'SiLU');
  if (!gate) {
    throw new Error('[SiLU] the HIP path implements the gated form (options.gate) only.');
  }
  if (gateActivation !== 'silu') {
    throw new Error(`[SiLU] gateActivation "${gateActivation}" is not supported by the HIP path.`);
  }
  if (input.dtype !== 'f32') {
    throw new Error(`[SiLU] the HIP path takes f32 activations, got ${input.dtype}.`);
  }
  const n = size || (input.buffer.size / 4);
  const output = outputBuffer || acquireBuffer(n * 4, undefined, 'silu_output');
  const owned = outputBuffer ? null : output;
  try {
    getNative().actGate(bufferOf(gate).ptr, input.buffer.ptr, output.ptr, n, ACT.silu, limit);
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
  noteDispatch(recorder, 'silu');
  return createTensor(output, input.dtype, [n], 'silu_output');
}

export async function runSiLU(input, options = {}) {
  return silu(null, input, options);
}

export async function recordSiLU(recorder, input, options = {}) {
  return silu(recorder, input, options);
}

async function siluRowSplit(recorder, input, options) {
  const { numTokens, dim, activation = 'silu', outputBuffer = null, swigluLimit } = options;
  const limit = resolveSwigluLimit(swigluLimit, 'SiLU row-split');
  if (!(activation in ACT)) {
    throw new Error(`[SiLU row-split] activation "${activation}" is not supported by the HIP path.`);
  }
  if (input.dtype !== 'f32') {
    throw new Error(`[SiLU row-split] the HIP path takes f32 activations, got ${input.dtype}.`);
  }
  if (input.buffer.size < numTokens * dim * 2 * 4) {
    throw new Error(`[SiLU row-split] input buffer smaller than [${numTokens}, ${2 * dim}] f32.`);
  }
  const output = outputBuffer || acquireBuffer(numTokens * dim * 4, undefined, 'silu_rowsplit_output');
  const owned = outputBuffer ? null : output;
  try {
    getNative().actGateRowsplit(input.buffer.ptr, output.ptr, numTokens, dim, ACT[activation], activation === 'silu' ? limit : 0);
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
  noteDispatch(recorder, 'silu_rowsplit');
  return createTensor(output, input.dtype, [numTokens, dim], 'silu_rowsplit_output');
}

export async function runSiLURowSplit(input, options) {
  return siluRowSplit(null, input, options);
}

export async function recordSiLURowSplit(recorder, input, options) {
  return siluRowSplit(recorder, input, options);
}
