// runAttention / recordAttention over an f16 KV cache, decode (seqLen 1) and prefill (seqLen > 1):
// reference src/gpu/kernels/attention.js:1047-1310,2007-2030.  An f16 Q (the reference's f16-activation
// plan: variants *_f16 with outputDtype f16, src/config/kernels/registry.json) is widened into a temporary
// (exact), the kernels run as for f32 and the output is narrowed to f16 once.
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
  if ((Q.dtype !== 'f32' && Q.dtype !== 'f16') || K.dtype !== 'f16' || V.dtype !== 'f16') {
    throw new Error(`[Attention] the HIP path needs f32 or f16 Q and f16 K/V, got ${Q.dtype}/${K.dtype}/${V.dtype}.`);
  }
  if (Q.dtype === 'f16') {
    // widened Q and an f32 output of our own; the caller's outputBuffer (if any) takes the f16 result
    const n = seqLen * numHeads * headDim;
    if (Q.buffer.size < n * 2) {
      throw new Error(`[Attention] Q buffer is smaller than [${seqLen}, ${numHeads}, ${headDim}] f16.`);
    }
    if (outputBuffer && outputBuffer.size < n * 2) {
      throw new Error(`[Attention] outputBuffer is smaller than [${seqLen}, ${numHeads}, ${headDim}] f16.`);
    }
    const wideQ = acquireBuffer(n * 4, undefined, 'attention_q_f32_temp');
    let wideOut = null;
    let out16 = null;
    try {
      getNative().castF16ToF32(Q.buffer.ptr, wideQ.ptr, n);
      const r = await executeAttention(recorder, createTensor(wideQ, 'f32', [...Q.shape], 'attention_q_f32'), K, V, mask,
        numHeads, headDim, { ...options, outputBuffer: null });
      wideOut = r.buffer;
      out16 = outputBuffer || acquireBuffer(n * 2, undefined, 'attention_output');
      getNative().castF32ToF16(wideOut.ptr, out16.ptr, n);
    } catch (error) {
      releaseBuffer(wideQ);
      if (wideOut) releaseBuffer(wideOut);
      if (out16 && !outputBuffer) releaseBuffer(out16);
      throw error;
    }
    for (const b of [wideQ, wideOut]) {
      if (recorder) recorder.trackTemporaryBuffer(b); else releaseBuffer(b);
    }
    return createTensor(out16, 'f16', [seqLen, numHeads, headDim], 'attention_output');
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
