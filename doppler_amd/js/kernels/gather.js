// runGather / recordGather for f16 embedding tables: reference src/gpu/kernels/gather.js:238-391.
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
  if (outputDtype !== 'f32') {
    throw new Error(`[Gather] outputDtype="${outputDtype}" is not supported by the HIP path (f32).`);
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
  const output = outputBuffer || acquireBuffer(numTokens * padToQ4KBlock(hiddenSize) * 4, undefined, 'gather_output');
  const owned = outputBuffer ? null : output;
  try {
    getNative().gatherF16(idx.ptr, table.ptr, output.ptr, numTokens, hiddenSize, vocabSize, indexOffset);
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
  noteDispatch(recorder, 'gather');
  return createTensor(output, 'f32', [numTokens, hiddenSize], 'gather_output');
}

export async function runGather(indices, embeddings, numTokens, hiddenSize, vocabSize, options = {}) {
  return gather(null, indices, embeddings, numTokens, hiddenSize, vocabSize, options);
}

export async function recordGather(recorder, indices, embeddings, numTokens, hiddenSize, vocabSize, options = {}) {
  return gather(recorder, indices, embeddings, numTokens, hiddenSize, vocabSize, options);
}
