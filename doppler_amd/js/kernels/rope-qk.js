// runRoPEQK / recordRoPEQK / canUseRoPEQK: reference src/gpu/kernels/rope-qk.js:56-143.  Rotates
// separate q and k buffers in place with one launch; the returned Tensors alias the inputs.
import { getNative } from '../native.js';
import { createTensor } from '../tensor.js';
import { bufferOf, noteDispatch } from './constants.js';

function requireInteger(value, label, minimum, kind) {
  if (!Number.isInteger(value) || value < minimum) {
    throw new Error(`RoPE QK requires ${label} to be a ${kind} integer.`);
  }
}

function requireRange(buffer, bytes, label) {
  if (buffer && Number.isFinite(buffer.size) && bytes > buffer.size) {
    throw new Error(`RoPE QK ${label} buffer is smaller than requested range (${bytes} > ${buffer.size} bytes).`);
  }
}

export function canUseRoPEQK(qTensor, kTensor, options = {}) {
  if (options.reusesSharedKV === true || !qTensor || !kTensor) return false;
  // The HIP kernel rotates f32 activations; f16 q/k stay with the one-buffer op.
  return qTensor.buffer !== kTensor.buffer && qTensor.dtype === 'f32' && kTensor.dtype === 'f32';
}

function aliases(qTensor, kTensor) {
  return {
    q: createTensor(qTensor.buffer, qTensor.dtype, [...qTensor.shape], 'rope_q_output'),
    k: createTensor(kTensor.buffer, kTensor.dtype, [...kTensor.shape], 'rope_k_output'),
  };
}

async function ropeQK(recorder, qTensor, kTensor, freqsCos, freqsSin, seqLen, options = {}) {
  const { numQHeads, numKVHeads, headDim } = options;
  const rotaryDim = options.rotaryDim === undefined ? headDim : options.rotaryDim;
  const pairSpanDim = options.pairSpanDim === undefined ? rotaryDim : options.pairSpanDim;
  const startPos = options.startPos === undefined ? 0 : options.startPos;
  requireInteger(seqLen, 'seqLen', 0, 'non-negative');
  requireInteger(startPos, 'startPos', 0, 'non-negative');
  requireInteger(numQHeads, 'numQHeads', 1, 'positive');
  requireInteger(numKVHeads, 'numKVHeads', 1, 'positive');
  requireInteger(headDim, 'headDim', 1, 'positive');
  requireInteger(rotaryDim, 'rotaryDim', 1, 'positive');
  requireInteger(pairSpanDim, 'pairSpanDim', 1, 'positive');
  if (qTensor.dtype !== kTensor.dtype) {
    throw new Error(`RoPE QK requires matching Q/K dtypes, got ${qTensor.dtype} and ${kTensor.dtype}.`);
  }
  if (qTensor.dtype !== 'f32') {
    throw new Error(`RoPE QK on the HIP path takes f32 tensors, got ${qTensor.dtype}.`);
  }
  if (seqLen === 0) return aliases(qTensor, kTensor);
  const cos = bufferOf(freqsCos);
  const sin = bufferOf(freqsSin);
  const tableBytes = (startPos + seqLen) * Math.floor(rotaryDim / 2) * 4;
  requireRange(qTensor.buffer, seqLen * numQHeads * headDim * 4, 'Q input');
  requireRange(kTensor.buffer, seqLen * numKVHeads * headDim * 4, 'K input');
  requireRange(cos, tableBytes, 'cos frequencies');
  requireRange(sin, tableBytes, 'sin frequencies');
  // Geometry rules (even dims, rotaryDim <= pairSpanDim <= headDim) are checked by the library,
  // which words its errors as the reference does.
  getNative().ropeQK(qTensor.buffer.ptr, kTensor.buffer.ptr, cos.ptr, sin.ptr, seqLen, numQHeads, numKVHeads, headDim,
    rotaryDim, pairSpanDim, options.interleaved ? 1 : 0, startPos);
  noteDispatch(recorder, 'rope_qk');
  return aliases(qTensor, kTensor);
}

export async function runRoPEQK(qTensor, kTensor, freqsCos, freqsSin, seqLen, options = {}) {
  return ropeQK(null, qTensor, kTensor, freqsCos, freqsSin, seqLen, options);
}

export async function recordRoPEQK(recorder, qTensor, kTensor, freqsCos, freqsSin, seqLen, options = {}) {
  return ropeQK(recorder, qTensor, kTensor, freqsCos, freqsSin, seqLen, options);
}
