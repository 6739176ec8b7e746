// runResidualAdd / recordResidualAdd: reference src/gpu/kernels/residual.js:122-216.
import { getNative } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { noteDispatch } from './constants.js';

function resolveOutputScale(outputScale) {
  if (outputScale === null || outputScale === undefined) return 1;
  const value = Number(outputScale);
  if (!Number.isFinite(value)) {
    throw new Error(`[Residual] outputScale must be finite; got "${String(outputScale)}".`);
  }
  return value;
}

async function residualAdd(recorder, a, b, size, options = {}) {
  const { outputBuffer = null } = options;
  const scale = resolveOutputScale(options.outputScale);
  if (a.dtype !== 'f32' || b.dtype !== 'f32') {
    throw new Error(`[Residual] the HIP path takes f32 tensors, got ${a.dtype}/${b.dtype}.`);
  }
  if (a.buffer.size < size * 4 || b.buffer.size < size * 4) {
    throw new Error(`[Residual] input buffers are smaller than ${size} f32 elements.`);
  }
  const output = outputBuffer || acquireBuffer(size * 4, undefined, 'residual_output');
  const owned = outputBuffer ? null : output;
  try {
    getNative().residualAdd(a.buffer.ptr, b.buffer.ptr, output.ptr, size, scale);
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
  noteDispatch(recorder, 'residual');
  return createTensor(output, 'f32', [size], 'residual_output');
}

export async function runResidualAdd(a, b, size, options = {}) {
  return residualAdd(null, a, b, size, options);
}

export async function recordResidualAdd(recorder, a, b, size, options = {}) {
  return residualAdd(recorder, a, b, size, options);
}
