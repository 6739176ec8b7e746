// recordLmHeadArgmax / recordLmHeadArgmaxF16: reference src/gpu/kernels/lm-head-argmax.js:292-315.
// Final-logit GEMV over the f16 (tied) embedding fused with greedy argmax; returns the
// output buffer with the token id at `outputIndex`.  Beyond the reference's options: `normWeight` (f32
// tensor [hiddenSize]) with `rmsNormEps` and `rmsNormWeightOffset` applies the final RMSNorm of
// recordLogitsGPU (src/inference/pipelines/text/logits/gpu.js:1122-1157) to the row inside the same
// kernel (hiddenSize <= 4096; use lmHeadArgmaxNormFusable to ask).
import { getNative } from '../native.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { getBuffer, getWeightDtype } from '../weight-buffer.js';

function validateArgmaxOptions(options) {
  if (!Number.isInteger(options.vocabSize) || options.vocabSize <= 0) {
    throw new Error(`[LmHeadArgmax] vocabSize must be a positive integer, got ${options.vocabSize}.`);
  }
  if (!Number.isInteger(options.hiddenSize) || options.hiddenSize <= 0) {
    throw new Error(`[LmHeadArgmax] hiddenSize must be a positive integer, got ${options.hiddenSize}.`);
  }
  const idx = options.outputIndex === undefined ? 0 : options.outputIndex;
  if (!Number.isInteger(idx) || idx < 0) {
    throw new Error(`[LmHeadArgmax] outputIndex must be a non-negative integer, got ${idx}.`);
  }
  return idx;
}

export function lmHeadArgmaxNormFusable(hiddenSize) {
  return Number.isInteger(hiddenSize) && hiddenSize > 0 && hiddenSize <= 4096 && hiddenSize % 8 === 0;
}

export async function recordLmHeadArgmaxF16(recorder, inputTensor, lmHead, options = {}) {
  if (!recorder || !recorder.device) {
    throw new Error('[LmHeadArgmax] CommandRecorder is required.');
  }
  if (!inputTensor || inputTensor.dtype !== 'f32') {
    throw new Error(`[LmHeadArgmax] input tensor must be f32, got "${inputTensor && inputTensor.dtype ? inputTensor.dtype : 'unknown'}".`);
  }
  const outputIndex = validateArgmaxOptions(options);
  const dtype = getWeightDtype(lmHead);
  if (dtype !== 'f16') {
    throw new Error(`[LmHeadArgmax] LM head weight must be f16 on the HIP path, got "${dtype}".`);
  }
  const weight = getBuffer(lmHead);
  if (weight.size < options.vocabSize * options.hiddenSize * 2) {
    throw new Error(`[LmHeadArgmax] LM head buffer smaller than [${options.vocabSize}, ${options.hiddenSize}] f16.`);
  }
  const native = getNative();
  const minOutputBytes = Math.max(4, (outputIndex + 1) * 4);
  const output = options.outputBuffer || acquireBuffer(minOutputBytes, undefined, 'lm_head_argmax_output');
  if (output.size < minOutputBytes) {
    throw new Error(`[LmHeadArgmax] output buffer too small for outputIndex ${outputIndex}.`);
  }
  const workspace = acquireBuffer(native.lmheadArgmaxWorkspaceBytes(options.vocabSize), undefined, 'lm_head_argmax_temp');
  const pad = options.padTokenId === null || options.padTokenId === undefined ? -1 : options.padTokenId;
  const normWeight = options.normWeight || null;
  try {
    if (normWeight) {
      if (normWeight.dtype !== 'f32' || normWeight.buffer.size < options.hiddenSize * 4) {
        throw new Error(`[LmHeadArgmax] normWeight must be an f32 tensor of ${options.hiddenSize} values.`);
      }
      if (!(options.rmsNormEps >= 0)) {
        throw new Error('[LmHeadArgmax] rmsNormEps is required with normWeight.');
      }
      native.lmheadArgmaxF16RMSNorm(inputTensor.buffer.ptr, normWeight.buffer.ptr, options.rmsNormEps,
        options.rmsNormWeightOffset ? 1 : 0, weight.ptr, options.vocabSize, options.hiddenSize, pad,
        options.logitSoftcap || 0, workspace.ptr, output.ptr, outputIndex,
        options.logitsOutput ? options.logitsOutput.ptr : null);
    } else {
      native.lmheadArgmaxF16(inputTensor.buffer.ptr, weight.ptr, options.vocabSize, options.hiddenSize, pad,
        options.logitSoftcap || 0, workspace.ptr, output.ptr, outputIndex,
        options.logitsOutput ? options.logitsOutput.ptr : null);
    }
  } catch (error) {
    if (!options.outputBuffer) releaseBuffer(output);
    releaseBuffer(workspace);
    throw error;
  }
  recorder.trackTemporaryBuffer(workspace);
  if (typeof recorder.noteDispatch === 'function') recorder.noteDispatch('lm_head_argmax');
  return output;
}

export async function recordLmHeadArgmax(recorder, inputTensor, lmHead, options = {}) {
  return recordLmHeadArgmaxF16(recorder, inputTensor, lmHead, options);
}
