// Format constants shared by the op wrappers (reference:
// src/config/schema/quantization.schema.js:5-33).
export const QK_K = 256;
export const Q4K_BLOCK_BYTES = 144;

export function padToQ4KBlock(size) {
  return Math.ceil(size / QK_K) * QK_K;
}

export function bufferOf(x) {
  return x && typeof x === 'object' && 'buffer' in x && x.buffer && 'ptr' in x.buffer ? x.buffer : x;
}

export function ptrOf(x) {
  if (x === null || x === undefined) return null;
  const b = bufferOf(x);
  if (!b || typeof b.ptr !== 'bigint') {
    throw new Error('[doppler-hip] expected a device buffer');
  }
  return b.ptr;
}

export function sizeOf(x) {
  const b = bufferOf(x);
  return b ? b.size : NaN;
}

export function noteDispatch(recorder, label) {
  if (recorder && typeof recorder.noteDispatch === 'function') recorder.noteDispatch(label);
}
