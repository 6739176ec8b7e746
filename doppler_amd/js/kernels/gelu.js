// runGeLU / recordGeLU (gated form): reference src/gpu/kernels/gelu.js:49-56, gelu.wgsl:24-65.
import { getNative, ACT } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { bufferOf, noteDispatch } from './constants.js';

async function gelu(recorder, input, options = {}) {
  const { size, gate = null, outputBuffer = null } = options;
  if (!gate) {
    throw new Error('[GeLU] the HIP path implements the gated form (options.gate) only.');
  }
  if (input.dtype !== 'f32') {
    throw new Error(`[GeLU] the HIP path takes f32 activations, got ${input.dtype}.`);
  }
  const n = size || (input.buffer.size / 4);
  const output = outputBuffer || acquireBuffer(n * 4, undefined, 'gelu_output');
  const owned = outputBuffer ? null : output;
  try {
    getNative().actGate(bufferOf(gate).ptr, input.buffer.ptr, output.ptr, n, ACT.gelu, 0);
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
  noteDispatch(recorder, 'gelu');
  return createTensor(output, input.dtype, [n], 'gelu_output');
}

export async function runGeLU(input, options = {}) {
  return gelu(null, input, options);
}

export async function recordGeLU(recorder, input, options = {}) {
  return gelu(recorder, input, options);
}
