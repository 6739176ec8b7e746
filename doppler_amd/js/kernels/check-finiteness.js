// recordCheckFiniteness and its host helpers: reference src/gpu/kernels/check-finiteness.js:5-150;
// parseFinitenessStatusWords: src/inference/pipelines/text/finiteness-guard-status.js:1-21.
// The status buffer is 4 u32 words [status, layer, step, pad] that the caller zeroes before a step
// and reads back beside the sampled token (src/inference/pipelines/text/generator-steps.js:786-798).
import { getNative, DTYPE } from '../native.js';
import { acquireBuffer } from '../buffer-pool.js';
import { noteDispatch } from './constants.js';

export const DEFAULT_FINITENESS_ABS_THRESHOLD = 65500;
export const FINITENESS_STATUS_BYTES = 16;

export function resolveFinitenessAbsThreshold(value) {
  if (Number.isFinite(value) && value > 0) {
    return value;
  }
  return DEFAULT_FINITENESS_ABS_THRESHOLD;
}

export function shouldTriggerFinitenessValue(value, absThreshold = DEFAULT_FINITENESS_ABS_THRESHOLD) {
  if (!Number.isFinite(value)) {
    return true;
  }
  return Math.abs(value) > resolveFinitenessAbsThreshold(absThreshold);
}

export function parseFinitenessStatusWords(words, offset = 0) {
  const word = (i) => (words[i] === undefined || words[i] === null ? 0 : Number(words[i]));
  const status = word(offset);
  if (status <= 0) {
    return { triggered: false, layer: 0, step: 0, metadata: '' };
  }
  const layer = word(offset + 1);
  const step = word(offset + 2);
  return { triggered: true, layer, step, metadata: ` (layer ${layer}, step ${step})` };
}

export function createFinitenessStatusBuffer() {
  const buffer = acquireBuffer(FINITENESS_STATUS_BYTES, undefined, 'finiteness_status');
  getNative().fillZero(buffer.ptr, 0, FINITENESS_STATUS_BYTES);
  return buffer;
}

// inputBuffer: a tensor ({buffer, dtype}) or a bare buffer; a bare buffer is read as f16, the
// element type of the reference's shader, unless `inputDtype` says f32.
export function recordCheckFiniteness(
  target,
  inputBuffer,
  size,
  statusBuffer,
  layerIdx = 0,
  step = 0,
  absThreshold = DEFAULT_FINITENESS_ABS_THRESHOLD,
  inputDtype = null
) {
  const buffer = inputBuffer && inputBuffer.buffer ? inputBuffer.buffer : inputBuffer;
  const dtype = inputDtype || (inputBuffer && typeof inputBuffer.dtype === 'string' ? inputBuffer.dtype : 'f16');
  if (dtype !== 'f16' && dtype !== 'f32') {
    throw new Error(`[check_finiteness] input dtype must be f16 or f32, got ${dtype}.`);
  }
  if (buffer.size < size * (dtype === 'f16' ? 2 : 4)) {
    throw new Error(`[check_finiteness] input buffer smaller than size=${size}.`);
  }
  if (!statusBuffer || statusBuffer.size < FINITENESS_STATUS_BYTES) {
    throw new Error('[check_finiteness] status buffer must hold 4 u32 words.');
  }
  getNative().checkFiniteness(buffer.ptr, DTYPE[dtype], size, statusBuffer.ptr, layerIdx, step,
    resolveFinitenessAbsThreshold(absThreshold));
  noteDispatch(target, 'check_finiteness');
}
