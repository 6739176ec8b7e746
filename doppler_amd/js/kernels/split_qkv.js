// runSplitQKV / recordSplitQKV: reference src/gpu/kernels/split_qkv.js:6-45.  Copies the rows of the
// stacked projection [numTokens][qSize + kSize + vSize] apart into Q, K and V.
import { getNative } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { noteDispatch } from './constants.js';

async function splitQKV(recorder, qkvTensor, options) {
  const { numTokens, qSize, kSize, vSize } = options;
  if (qkvTensor.dtype !== 'f32') {
    throw new Error(`[SplitQKV] the HIP path takes f32 tensors, got ${qkvTensor.dtype}.`);
  }
  const rowLength = qSize + kSize + vSize;
  if (numTokens * rowLength * 4 > qkvTensor.buffer.size) {
    throw new Error(`[SplitQKV] qkv buffer is smaller than numTokens=${numTokens} x ${rowLength} elements.`);
  }
  const parts = [
    { given: options.qTensor || null, size: qSize, label: 'Q' },
    { given: options.kTensor || null, size: kSize, label: 'K' },
    { given: options.vTensor || null, size: vSize, label: 'V' },
  ];
  const owned = [];
  try {
    for (const part of parts) {
      const bytes = numTokens * part.size * 4;
      if (part.given && part.given.buffer.size < bytes) {
        throw new Error(`[SplitQKV] ${part.label} tensor is smaller than numTokens=${numTokens} x ${part.size} elements.`);
      }
      part.buffer = part.given ? part.given.buffer : acquireBuffer(bytes, undefined, part.label);
      if (!part.given) owned.push(part.buffer);
    }
    getNative().splitQKV(qkvTensor.buffer.ptr, parts[0].buffer.ptr, parts[1].buffer.ptr, parts[2].buffer.ptr, numTokens,
      qSize, kSize, vSize);
  } catch (error) {
    owned.forEach((buffer) => releaseBuffer(buffer));
    throw error;
  }
  noteDispatch(recorder, 'split_qkv');
  const [Q, K, V] = parts.map((part) => part.given || createTensor(part.buffer, 'f32', [numTokens, part.size], part.label));
  return { Q, K, V };
}

export async function runSplitQKV(qkvTensor, options) {
  return splitQKV(null, qkvTensor, options);
}

export async function recordSplitQKV(recorder, qkvTensor, options) {
  return splitQKV(recorder, qkvTensor, options);
}
