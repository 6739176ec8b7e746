// One decode step of recordSplitQKVRMSNormRoPEQK (f16KVCacheWrite at the row of startPos) followed by
// recordAttention with seqLen == 1, in one launch: reference
// src/gpu/kernels/split-qkv-rmsnorm-rope-qk.js:244-250 then src/gpu/kernels/attention.js:2007-2030.
// The attention kernel norms and rotates the step's q and k itself, appends k/v to the f16 cache and
// attends to rows up to and including the new one.
import { getNative, KV_LAYOUT } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { getBuffer } from '../weight-buffer.js';
import { padToQ4KBlock, bufferOf, noteDispatch } from './constants.js';

export function decodeAttentionFromQKVSupported(numHeads, numKVHeads, headDim, rotaryDim = headDim, interleaved = false) {
  return getNative().attnDecodeQkvSupported(numHeads, numKVHeads, headDim, rotaryDim, interleaved ? 1 : 0) === 1;
}

async function execute(recorder, qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, keys, values, options = {}) {
  const {
    numHeads, numKVHeads = numHeads, headDim, startPos,
    rotaryDim = headDim, interleaved = false, rmsNormWeightOffset = false, useNorm = true,
    scale = 1.0 / Math.sqrt(headDim), attnSoftcap = 0, slidingWindow = 0, kvStart = 0, kvLayout = 'contiguous',
    outputBuffer = null,
    kvLenBuffer = null, maxKvLen = 0,
  } = options;
  for (const [label, v] of [['numHeads', numHeads], ['numKVHeads', numKVHeads], ['headDim', headDim]]) {
    if (!Number.isInteger(v) || v <= 0) throw new Error(`[Attention] fused decode ${label} must be a positive integer, got ${v}.`);
  }
  // kvLenBuffer: the key count (the step's position - kvStart + 1) is read on the device, as with
  // runAttention's option of that name; maxKvLen bounds it and sizes tables, caches and workspace
  if (kvLenBuffer) {
    if (!Number.isInteger(maxKvLen) || maxKvLen < 1) {
      throw new Error(`[Attention] fused decode with kvLenBuffer needs a positive maxKvLen, got ${maxKvLen}.`);
    }
    if (!(kvLenBuffer.size >= 4)) throw new Error('[Attention] kvLenBuffer must hold one u32.');
  } else if (!Number.isInteger(startPos) || startPos < 0) {
    throw new Error(`[Attention] fused decode startPos must be a non-negative integer, got ${startPos}.`);
  }
  const lastPos = kvLenBuffer ? kvStart + maxKvLen - 1 : startPos;
  if (!(kvLayout in KV_LAYOUT)) {
    throw new Error(`[Attention] kvLayout "${kvLayout}" is not supported by the HIP path (contiguous, ring).`);
  }
  if (qkvTensor.dtype !== 'f32') {
    throw new Error(`[Attention] fused decode requires f32 QKV input, got ${qkvTensor.dtype}.`);
  }
  if (qkvTensor.buffer.size < (numHeads + 2 * numKVHeads) * headDim * 4) {
    throw new Error('[Attention] fused decode: QKV buffer is smaller than (numHeads + 2 numKVHeads) * headDim floats.');
  }
  const cos = bufferOf(freqsCos);
  const sin = bufferOf(freqsSin);
  const freqBytes = (lastPos + 1) * (rotaryDim / 2) * 4;
  if (cos.size < freqBytes || sin.size < freqBytes) {
    throw new Error(`[Attention] fused decode: rotary tables end before position ${lastPos}.`);
  }
  const rows = kvLayout === 'ring' ? slidingWindow : lastPos + 1;
  const kvBytes = rows * numKVHeads * headDim * 2;
  if (keys.buffer.size < kvBytes || values.buffer.size < kvBytes) {
    throw new Error(`[Attention] KV buffers are smaller than ${rows} rows (${kvBytes} bytes).`);
  }
  const native = getNative();
  const output = outputBuffer || acquireBuffer(padToQ4KBlock(numHeads * headDim) * 4, undefined, 'attention_output');
  const workspace = acquireBuffer(native.attnDecodeWorkspaceBytes(numHeads, headDim, lastPos - kvStart + 1), undefined,
    'attention_splitk_workspace');
  try {
    if (kvLenBuffer) {
      native.attnDecodeQkvKvLen(qkvTensor.buffer.ptr, useNorm ? getBuffer(qWeight).ptr : 0, useNorm ? getBuffer(kWeight).ptr : 0,
        cos.ptr, sin.ptr, keys.buffer.ptr, values.buffer.ptr, output.ptr, numHeads, numKVHeads, headDim, kvLenBuffer.ptr,
        maxKvLen, rotaryDim, interleaved ? 1 : 0, eps, rmsNormWeightOffset ? 1 : 0, useNorm ? 1 : 0, scale, attnSoftcap,
        slidingWindow, kvStart, KV_LAYOUT[kvLayout], workspace.ptr);
    } else native.attnDecodeQkv(qkvTensor.buffer.ptr, useNorm ? getBuffer(qWeight).ptr : 0, useNorm ? getBuffer(kWeight).ptr : 0,
      cos.ptr, sin.ptr, keys.buffer.ptr, values.buffer.ptr, output.ptr, numHeads, numKVHeads, headDim, startPos,
      rotaryDim, interleaved ? 1 : 0, eps, rmsNormWeightOffset ? 1 : 0, useNorm ? 1 : 0, scale, attnSoftcap,
      slidingWindow, kvStart, KV_LAYOUT[kvLayout], workspace.ptr);
  } catch (error) {
    if (!outputBuffer) releaseBuffer(output);
    releaseBuffer(workspace);
    throw error;
  }
  if (recorder) recorder.trackTemporaryBuffer(workspace); else releaseBuffer(workspace);
  noteDispatch(recorder, 'attention:from_qkv');
  return createTensor(output, 'f32', [1, numHeads, headDim], 'attention_output');
}

export async function runDecodeAttentionFromQKV(qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, keys, values, options = {}) {
  return execute(null, qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, keys, values, options);
}

export async function recordDecodeAttentionFromQKV(recorder, qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, keys, values, options = {}) {
  return execute(recorder, qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, keys, values, options);
}
