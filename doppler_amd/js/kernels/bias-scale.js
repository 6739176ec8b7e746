// runBiasAdd / recordBiasAdd (reference src/gpu/kernels/residual.js:165-224) and runScale / recordScale
// (reference src/gpu/kernels/scale.js:13-46) on f32 activations.
import { getNative, DTYPE } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { bufferOf, noteDispatch } from './constants.js';

async function biasAdd(recorder, data, bias, numTokens, dim, options = {}) {
  const { dataOffset = 0, biasOffset = 0 } = options;
  if (data.dtype !== 'f32') {
    throw new Error(`[BiasAdd] the HIP path takes f32 data, got ${data.dtype}.`);
  }
  const biasDtype = bias.dtype === undefined ? 'f32' : bias.dtype;
  if (biasDtype !== 'f32' && biasDtype !== 'f16') {
    throw new Error(`[BiasAdd] bias dtype must be f32 or f16, got ${biasDtype}.`);
  }
  const biasBuffer = bufferOf(bias);
  if (dataOffset + numTokens * dim * 4 > data.buffer.size) {
    throw new Error(`[BiasAdd] data buffer is smaller than numTokens=${numTokens} x dim=${dim} at offset ${dataOffset}.`);
  }
  if (biasOffset + dim * (biasDtype === 'f16' ? 2 : 4) > biasBuffer.size) {
    throw new Error(`[BiasAdd] bias buffer is smaller than dim=${dim} at offset ${biasOffset}.`);
  }
  // An f16 bias is widened inside the kernel, so no aligned temporary copy is made.
  getNative().biasAdd(data.buffer.ptr, biasBuffer.ptr, DTYPE[biasDtype], numTokens, dim, dataOffset, biasOffset);
  noteDispatch(recorder, 'bias_add');
  return createTensor(data.buffer, data.dtype, [numTokens, dim], 'bias_add_output');
}

export async function runBiasAdd(data, bias, numTokens, dim, options = {}) {
  return biasAdd(null, data, bias, numTokens, dim, options);
}

export async function recordBiasAdd(recorder, data, bias, numTokens, dim, options = {}) {
  return biasAdd(recorder, data, bias, numTokens, dim, options);
}

async function scaleTensor(recorder, input, scale, options = {}) {
  const { outputBuffer = null, inplace = false } = options;
  if (input.dtype !== 'f32') {
    throw new Error(`[Scale] the HIP path takes f32 tensors, got ${input.dtype}.`);
  }
  const count = options.count === undefined || options.count === null ? Math.floor(input.buffer.size / 4) : options.count;
  if (count * 4 > input.buffer.size) {
    throw new Error(`[Scale] count=${count} exceeds the input buffer.`);
  }
  const owned = !inplace && !outputBuffer ? acquireBuffer(count * 4, undefined, 'scale_output') : null;
  const output = inplace ? input.buffer : (outputBuffer || owned);
  try {
    getNative().scale(input.buffer.ptr, output.ptr, count, scale);
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
  noteDispatch(recorder, 'scale');
  return createTensor(output, input.dtype, [...input.shape], 'scale_output');
}

export async function runScale(input, scale, options = {}) {
  return scaleTensor(null, input, scale, options);
}

export async function recordScale(recorder, input, scale, options = {}) {
  return scaleTensor(recorder, input, scale, options);
}
