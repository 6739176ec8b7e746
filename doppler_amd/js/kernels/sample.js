// runArgmax / recordArgmax: reference src/gpu/kernels/sample.js:258-341,459-466;
// runGPUSample / recordGPUSample (top-k temperature sampling): sample.js:343-568.
// runArgmax returns the token id (it reads 4 bytes back); recordArgmax returns the output
// buffer holding the id at `outputIndex`.
import { getNative } from '../native.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { bufferOf } from './constants.js';

function assertArgmaxOptions(options) {
  const idx = options.outputIndex === undefined ? 0 : options.outputIndex;
  if (!Number.isInteger(idx) || idx < 0) {
    throw new Error(`[Argmax] outputIndex must be a non-negative integer, got ${idx}.`);
  }
  const dtype = options.logitsDtype === undefined ? 'f32' : options.logitsDtype;
  if (dtype !== 'f32') {
    throw new Error(`[Argmax] logitsDtype "${dtype}" is not supported by the HIP path (f32).`);
  }
  return idx;
}

function enqueueArgmax(recorder, logits, vocabSize, options) {
  const outputIndex = assertArgmaxOptions(options);
  const native = getNative();
  const src = bufferOf(logits);
  if (src.size < vocabSize * 4) {
    throw new Error(`[Argmax] logits buffer smaller than vocabSize=${vocabSize} f32 values.`);
  }
  const minOutputBytes = Math.max(4, (outputIndex + 1) * 4);
  const output = options.outputBuffer || acquireBuffer(minOutputBytes, undefined, 'argmax_output');
  if (output.size < minOutputBytes) {
    throw new Error(`[Argmax] output buffer too small for outputIndex ${outputIndex}.`);
  }
  const workspace = acquireBuffer(native.argmaxWorkspaceBytes(), undefined, 'argmax_temp');
  const pad = options.padTokenId === null || options.padTokenId === undefined ? -1 : options.padTokenId;
  try {
    native.argmax(src.ptr, vocabSize, pad, options.logitSoftcap || 0, workspace.ptr, output.ptr, outputIndex);
  } catch (error) {
    if (!options.outputBuffer) releaseBuffer(output);
    releaseBuffer(workspace);
    throw error;
  }
  if (recorder) recorder.trackTemporaryBuffer(workspace); else releaseBuffer(workspace);
  return { output, outputIndex };
}

export async function runArgmax(logits, vocabSize, options = {}) {
  const { output, outputIndex } = enqueueArgmax(null, logits, vocabSize, options);
  const bytes = getNative().download(output.ptr, outputIndex * 4, 4);
  if (!options.outputBuffer) releaseBuffer(output);
  return new Uint32Array(bytes)[0];
}

export async function recordArgmax(recorder, logits, vocabSize, options = {}) {
  return enqueueArgmax(recorder, logits, vocabSize, options).output;
}

// src/gpu/kernels/sample.js:569-572
export function seededRandom(seed) {
  const x = Math.sin(seed) * 10000;
  return x - Math.floor(x);
}

function enqueueSample(recorder, logits, vocabSize, options) {
  const { temperature, topK, randomSeed, randomValue, padTokenId, logitSoftcap, greedyThreshold = 0.01 } = options;
  if (!(temperature >= 0) || !Number.isInteger(topK)) {
    throw new Error('[Sample] temperature and topK are required.');
  }
  if (temperature < greedyThreshold || topK <= 1) return enqueueArgmax(recorder, logits, vocabSize, options);
  const outputIndex = assertArgmaxOptions(options);
  const r = randomValue !== undefined ? randomValue : (randomSeed !== undefined ? seededRandom(randomSeed) : Math.random());
  const native = getNative();
  const src = bufferOf(logits);
  if (src.size < vocabSize * 4) {
    throw new Error(`[Sample] logits buffer smaller than vocabSize=${vocabSize} f32 values.`);
  }
  const minOutputBytes = Math.max(4, (outputIndex + 1) * 4);
  const output = options.outputBuffer || acquireBuffer(minOutputBytes, undefined, 'sample_output');
  if (output.size < minOutputBytes) {
    throw new Error(`[Sample] output buffer too small for outputIndex ${outputIndex}.`);
  }
  const workspace = acquireBuffer(native.sampleTopkWorkspaceBytes(vocabSize, topK), undefined, 'topk_candidates');
  const pad = padTokenId === null || padTokenId === undefined ? -1 : padTokenId;
  try {
    native.sampleTopk(src.ptr, vocabSize, temperature, topK, r, pad, logitSoftcap || 0, workspace.ptr, output.ptr, outputIndex);
  } catch (error) {
    if (!options.outputBuffer) releaseBuffer(output);
    releaseBuffer(workspace);
    throw error;
  }
  if (recorder) recorder.trackTemporaryBuffer(workspace); else releaseBuffer(workspace);
  return { output, outputIndex };
}

export async function runGPUSample(logits, vocabSize, options = {}) {
  const { output, outputIndex } = enqueueSample(null, logits, vocabSize, options);
  const bytes = getNative().download(output.ptr, outputIndex * 4, 4);
  if (!options.outputBuffer) releaseBuffer(output);
  return new Uint32Array(bytes)[0];
}

export async function recordGPUSample(recorder, logits, vocabSize, options = {}) {
  return enqueueSample(recorder, logits, vocabSize, options).output;
}
