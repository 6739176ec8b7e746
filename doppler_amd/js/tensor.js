// Tensor handle of the op API: a plain record {buffer, dtype, shape, label} whose shape cannot be
// changed afterwards.  Same fields and helper names as the reference's src/gpu/tensor.js:7-31.

const BYTES_PER_ELEMENT = { f16: 2, f32: 4 };

export function createTensor(buffer, dtype, shape, label) {
  const dims = Object.freeze(Array.from(shape));
  return { buffer, dtype, shape: dims, label };
}

// Every dtype other than 'f16' is stored as four bytes per element, as in the reference.
export function dtypeBytes(dtype) {
  return BYTES_PER_ELEMENT[dtype] === 2 ? 2 : 4;
}

export function tensorBytes(shape, dtype) {
  let elements = 1;
  for (const d of shape) elements *= d;
  return elements * dtypeBytes(dtype);
}
