// castF32ToF16 / castF16ToF32 (+record forms): reference src/gpu/kernels/cast.js:98-116.
import { getNative } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer } from '../buffer-pool.js';

function count(input) {
  return input.shape.reduce((a, b) => a * b, 1);
}

export async function castF32ToF16(input, options = {}) {
  const n = count(input);
  const output = options.outputBuffer || acquireBuffer(n * 2, undefined, 'cast_f32_to_f16_output');
  getNative().castF32ToF16(input.buffer.ptr, output.ptr, n);
  return createTensor(output, 'f16', [...input.shape], 'cast_f32_to_f16_output');
}

export async function castF16ToF32(input, options = {}) {
  const n = count(input);
  const output = options.outputBuffer || acquireBuffer(n * 4, undefined, 'cast_f16_to_f32_output');
  getNative().castF16ToF32(input.buffer.ptr, output.ptr, n);
  return createTensor(output, 'f32', [...input.shape], 'cast_f16_to_f32_output');
}

export async function recordCastF32ToF16(recorder, input, options = {}) {
  return castF32ToF16(input, options);
}

export async function recordCastF16ToF32(recorder, input, options = {}) {
  return castF16ToF32(input, options);
}
