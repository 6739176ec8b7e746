// runRoPE / recordRoPE: reference src/gpu/kernels/rope.js:14-114.  In place; the returned
// Tensor aliases the input buffer.  f16 activations take the reference's own route for a device
// without an f16 rotary kernel (rope.js:44-63,89-107): widened into a temporary, rotated in f32,
// narrowed back into the input buffer (one rounding, as a kernel that computes in f32 and stores
// f16 would make).
import { getNative } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { bufferOf, noteDispatch } from './constants.js';

async function rope(recorder, input, freqsCos, freqsSin, seqLen, options = {}) {
  const {
    numHeads = 1,
    headDim = 64,
    rotaryDim = headDim,
    pairSpanDim = rotaryDim,
    interleaved = false,
    startPos = 0,
  } = options;
  if (!Number.isFinite(headDim) || headDim % 2 !== 0) {
    throw new Error(`RoPE headDim must be even, got ${headDim}`);
  }
  if (!Number.isFinite(rotaryDim) || rotaryDim % 2 !== 0) {
    throw new Error(`RoPE rotaryDim must be even, got ${rotaryDim}`);
  }
  if (rotaryDim <= 0 || rotaryDim > headDim) {
    throw new Error(`RoPE rotaryDim must be in (0, headDim]; got ${rotaryDim} for headDim ${headDim}`);
  }
  if (!Number.isFinite(pairSpanDim) || pairSpanDim % 2 !== 0) {
    throw new Error(`RoPE pairSpanDim must be even, got ${pairSpanDim}`);
  }
  if (pairSpanDim < rotaryDim || pairSpanDim > headDim) {
    throw new Error(
      `RoPE pairSpanDim must be in [rotaryDim, headDim]; got ${pairSpanDim} for rotaryDim ${rotaryDim} and headDim ${headDim}`
    );
  }
  if (input.dtype !== 'f32' && input.dtype !== 'f16') {
    throw new Error(`RoPE on the HIP path takes f32 or f16 activations, got ${input.dtype}`);
  }
  const cos = bufferOf(freqsCos);
  const sin = bufferOf(freqsSin);
  const need = (startPos + seqLen) * (rotaryDim / 2) * 4;
  if (cos.size < need || sin.size < need) {
    throw new Error(`RoPE frequency tables are smaller than ${need} bytes (startPos=${startPos}, seqLen=${seqLen})`);
  }
  const native = getNative();
  if (input.dtype === 'f16') {
    const n = seqLen * numHeads * headDim;
    if (input.buffer.size < n * 2) {
      throw new Error(`RoPE input buffer is smaller than [${seqLen}, ${numHeads}, ${headDim}] f16.`);
    }
    const wide = acquireBuffer(n * 4, undefined, 'rope_f32_temp');
    try {
      native.castF16ToF32(input.buffer.ptr, wide.ptr, n);
      native.rope(wide.ptr, cos.ptr, sin.ptr, seqLen, numHeads, headDim, rotaryDim, pairSpanDim,
        interleaved ? 1 : 0, startPos);
      native.castF32ToF16(wide.ptr, input.buffer.ptr, n);
    } catch (error) {
      releaseBuffer(wide);
      throw error;
    }
    if (recorder) recorder.trackTemporaryBuffer(wide); else releaseBuffer(wide);
  } else {
    native.rope(input.buffer.ptr, cos.ptr, sin.ptr, seqLen, numHeads, headDim, rotaryDim, pairSpanDim,
      interleaved ? 1 : 0, startPos);
  }
  noteDispatch(recorder, 'rope');
  return createTensor(input.buffer, input.dtype, [...input.shape], 'rope_output');
}

export async function runRoPE(input, freqsCos, freqsSin, seqLen, options = {}) {
  return rope(null, input, freqsCos, freqsSin, seqLen, options);
}

export async function recordRoPE(recorder, input, freqsCos, freqsSin, seqLen, options = {}) {
  return rope(recorder, input, freqsCos, freqsSin, seqLen, options);
}
