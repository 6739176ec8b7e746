// runAttention / recordAttention over an f16 KV cache, decode (seqLen 1) and prefill (seqLen > 1):
// reference src/gpu/kernels/attention.js:1047-1310,2007-2030.
import { getNative, KV_LAYOUT } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { padToQ4KBlock, noteDispatch } from './constants.js';

async function executeAttention(recorder, Q, K, V, mask, numHeads, headDim, options = {}) {
  const {
    seqLen = 1,
    kvLen = seqLen,
    numKVHeads = numHeads,
    scale = 1.0 / Math.sqrt(headDim),
    causal = true,
    startPos = 0,
    outputBuffer = null,
    attnSoftcap = 0,
    slidingWindow = 0,
    kvStart = 0,
    kvLayout = 'contiguous',
    kvLenBuffer = null,
  } = options;
  if (!(seqLen >= 1)) {
    throw new Error(`[Attention] seqLen must be positive, got ${seqLen}.`);
  }
  if (mask) {
    throw new Error('[Attention] explicit masks are not supported on the HIP path.');
  }
  if (!(kvLayout in KV_LAYOUT)) {
    throw new Error(`[Attention] kvLayout "${kvLayout}" is not supported by the HIP path (contiguous, ring).`);
  }
  if (Q.dtype !== 'f32' || K.dtype !== 'f16' || V.dtype !== 'f16') {
    throw new Error(`[Attention] decode needs f32 Q and f16 K/V, got ${Q.dtype}/${K.dtype}/${V.dtype}.`);
  }
  const rows = kvLayout === 'ring' ? slidingWindow : kvStart + kvLen;
  const kvBytes = rows * numKVHeads * headDim * 2;
  if (kvLen > 0 && (K.buffer.size < kvBytes || V.buffer.size < kvBytes)) {
    throw new Error(`[Attention] KV buffers are smaller than kvLen=${kvLen} rows (${kvBytes} bytes).`);
  }
  const native = getNative();
  if (kvLenBuffer && seqLen > 1) {
    throw new Error(`[Attention] kvLenBuffer is served for decode (seqLen 1) only, got seqLen=${seqLen}.`);
  }
  if (kvLenBuffer && !(kvLenBuffer.size >= 4)) {
    throw new Error('[Attention] kvLenBuffer must hold one u32.');
  }
  if (seqLen > 1) {
    if (kvLayout !== 'contiguous' || kvStart !== 0) {
      throw new Error(`[Attention] prefill (seqLen=${seqLen}) needs a contiguous cache with kvStart=0.`);
    }
    const out = outputBuffer || acquireBuffer(seqLen * numHeads * headDim * 4, undefined, 'attention_output');
    try {
      native.attnPrefill(Q.buffer.ptr, K.buffer.ptr, V.buffer.ptr, out.ptr, seqLen, numHeads, numKVHeads, headDim, kvLen,
        scale, causal ? 1 : 0, startPos, attnSoftcap, slidingWindow);
    } catch (error) {
      if (!outputBuffer) releaseBuffer(out);
      throw error;
    }
    noteDispatch(recorder, 'attention');
    return createTensor(out, 'f32', [seqLen, numHeads, headDim], 'attention_output');
  }
  const outputSize = seqLen * padToQ4KBlock(numHeads * headDim) * 4;
  const output = outputBuffer || acquireBuffer(outputSize, undefined, 'attention_output');
  const owned = outputBuffer ? null : output;
  const workspace = acquireBuffer(native.attnDecodeWorkspaceBytes(numHeads, headDim, Math.max(kvLen, 1)), undefined,
    'attention_splitk_workspace');
  try {
    if (kvLenBuffer) {
      // the key count is read on the device (reference: kv_len_source == 1); kvLen bounds it, and
      // startPos < 0 places the query at the last key (a decode step replayed for the next token)
      native.attnDecodeKvLen(Q.buffer.ptr, K.buffer.ptr, V.buffer.ptr, output.ptr, numHeads, numKVHeads, headDim,
        kvLenBuffer.ptr, Math.max(kvLen, 1), scale, causal ? 1 : 0, startPos, attnSoftcap, slidingWindow, kvStart,
        KV_LAYOUT[kvLayout], workspace.ptr);
    } else {
      native.attnDecode(Q.buffer.ptr, K.buffer.ptr, V.buffer.ptr, output.ptr, numHeads, numKVHeads, headDim, kvLen,
        scale, causal ? 1 : 0, startPos, attnSoftcap, slidingWindow, kvStart, KV_LAYOUT[kvLayout], workspace.ptr);
    }
  } catch (error) {
    if (owned) releaseBuffer(owned);
    releaseBuffer(workspace);
    throw error;
  }
  if (recorder) recorder.trackTemporaryBuffer(workspace); else releaseBuffer(workspace);
  noteDispatch(recorder, 'attention');
  return createTensor(output, 'f32', [seqLen, numHeads, headDim], 'attention_output');
}

export async function runAttention(Q, K, V, mask, numHeads, headDim, options = {}) {
  return executeAttention(null, Q, K, V, mask, numHeads, headDim, options);
}

export async function recordAttention(recorder, Q, K, V, mask, numHeads, headDim, options = {}) {
  return executeAttention(recorder, Q, K, V, mask, numHeads, headDim, options);
}
