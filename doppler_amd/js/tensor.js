// Tensor handle: reference src/gpu/tensor.js:7-31.

export function createTensor(buffer, dtype, shape, label) {
  return {
    buffer,
    dtype,
    shape: Object.freeze([...shape]),
    label,
  };
}

export function dtypeBytes(dtype) {
  return dtype === 'f16' ? 2 : 4;
}

export function tensorBytes(shape, dtype) {
  return shape.reduce((a, b) => a * b, 1) * dtypeBytes(dtype);
}
