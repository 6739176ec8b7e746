// runKVCacheWriteF32ToF16 / recordKVCacheWriteF32ToF16:
// reference src/gpu/kernels/kv-cache-write.js:35-126.
import { getNative } from '../native.js';
import { noteDispatch } from './constants.js';

function assertNonNegativeInteger(value, label) {
  if (!Number.isInteger(value) || value < 0) {
    throw new Error(`KV cache write ${label} must be a non-negative integer, got ${value}.`);
  }
}

function assertBufferCapacity(buffer, offset, elementCount, bytesPerElement, label) {
  const requiredBytes = (offset + elementCount) * bytesPerElement;
  if (!buffer || !Number.isFinite(buffer.size) || requiredBytes > buffer.size) {
    throw new Error(
      `KV cache write ${label} buffer is smaller than requested range ` +
      `(${requiredBytes} > ${buffer && buffer.size !== undefined ? buffer.size : 'unknown'} bytes).`
    );
  }
}

async function kvWrite(recorder, keys, values, outputKeys, outputValues, options = {}) {
  const srcOffset = options.srcOffset === undefined ? 0 : options.srcOffset;
  const dstOffset = options.dstOffset === undefined ? 0 : options.dstOffset;
  const elementCount = options.elementCount;
  assertNonNegativeInteger(srcOffset, 'srcOffset');
  assertNonNegativeInteger(dstOffset, 'dstOffset');
  assertNonNegativeInteger(elementCount, 'elementCount');
  if (elementCount === 0) return;
  assertBufferCapacity(keys, srcOffset, elementCount, 4, 'keys input');
  assertBufferCapacity(values, srcOffset, elementCount, 4, 'values input');
  assertBufferCapacity(outputKeys, dstOffset, elementCount, 2, 'keys output');
  assertBufferCapacity(outputValues, dstOffset, elementCount, 2, 'values output');
  getNative().kvWriteF16(keys.ptr, values.ptr, outputKeys.ptr, outputValues.ptr, srcOffset, dstOffset, elementCount);
  noteDispatch(recorder, 'kv_cache_write:f32_to_f16');
}

export async function runKVCacheWriteF32ToF16(keys, values, outputKeys, outputValues, options = {}) {
  return kvWrite(null, keys, values, outputKeys, outputValues, options);
}

export async function recordKVCacheWriteF32ToF16(recorder, keys, values, outputKeys, outputValues, options = {}) {
  return kvWrite(recorder, keys, values, outputKeys, outputValues, options);
}
