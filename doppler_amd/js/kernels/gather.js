// runGather / recordGather for f16 embedding tables: reference src/gpu/kernels/gather.js:238-391.
// outputDtype 'f16' (the reference's f16-activation plan) hands the rows back as they are stored: they are
// gathered into an f32 temporary and narrowed again, which is exact for values that were f16.
import { getNative } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { padToQ4KBlock, bufferOf, noteDispatch } from './constants.js';

async function gather(recorder, indices, embeddings, numTokens, hiddenSize, vocabSize, options = {}) {
  const {
    outputBuffer = null, embeddingDtype, outputDtype, transpose = false, indexOffset = 0,
    inputHiddenSize = hiddenSize, hiddenOffset = 0,
  } = options;
  if (embeddingDtype === null || embeddingDtype === undefined) {
    throw new Error('[Gather] embeddingDtype is required.');
  }
  if (outputDtype === null || outputDtype === undefined) {
    throw new Error('[Gather] outputDtype is required.');
  }
  if (embeddingDtype !== 'f16') {
    throw new Error(`[Gather] unsupported embeddingDtype="${embeddingDtype}".`);
  }
  if (outputDtype !== 'f32' && outputDtype !== 'f16') {
    throw new Error(`[Gather] outputDtype="${outputDtype}" is not supported by the HIP path (f32, f16).`);
  }
  if (transpose || inputHiddenSize !== hiddenSize || hiddenOffset !== 0) {
    throw new Error('[Gather] transposed tables and hidden slices are not supported by the HIP path.');
  }
  const idx = bufferOf(indices);
  const table = bufferOf(embeddings);
  if (idx.size < (indexOffset + numTokens) * 4) {
    throw new Error(`[Gather] indices buffer smaller than ${indexOffset + numTokens} ids.`);
  }
  if (table.size < vocabSize * hiddenSize * 2) {
    throw new Error(`[Gather] embedding buffer smaller than [${vocabSize}, ${hiddenSize}] f16.`);
  }
  const narrow = outputDtype === 'f16';
  const outBytes = numTokens * padToQ4KBlock(hiddenSize) * (narrow ? 2 : 4);
  if (outputBuffer && outputBuffer.size < numTokens * hiddenSize * (narrow ? 2 : 4)) {
    throw new Error(`[Gather] outputBuffer smaller than [${numTokens}, ${hiddenSize}] ${outputDtype}.`);
  }
  const output = outputBuffer || acquireBuffer(outBytes, undefined, 'gather_output');
  const owned = outputBuffer ? null : output;
  const wide = narrow ? acquireBuffer(numTokens * hiddenSize * 4, undefined, 'gather_f32_temp') : null;
  try {
    getNative().gatherF16(idx.ptr, table.ptr, (wide || output).ptr, numTokens, hiddenSize, vocabSize, indexOffset);
    if (wide) getNative().castF32ToF16(wide.ptr, output.ptr, numTokens * hiddenSize);
  } catch (error) {
    if (owned) releaseBuffer(owned);
    if (wide) releaseBuffer(wide);
    throw error;
  }
  if (wide) {
    if (recorder) recorder.trackTemporaryBuffer(wide); else releaseBuffer(wide);
  }
  noteDispatch(recorder, 'gather');
  return createTensor(output, outputDtype, [numTokens, hiddenSize], 'gather_output');
}

export async function runGather(indices, embeddings, numTokens, hiddenSize, vocabSize, options = {}) {
  return gather(null, indices, embeddings, numTokens, hiddenSize, vocabSize, options);
}

export async function recordGather(recorder, indices, embeddings, numTokens, hiddenSize, vocabSize, options = {}) {
  return gather(recorder, indices, embeddings, numTokens, hiddenSize, vocabSize, options);
}
