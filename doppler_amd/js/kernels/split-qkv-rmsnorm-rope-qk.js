// runSplitQKVRMSNormRoPEQK / recordSplitQKVRMSNormRoPEQK with the f16 KV-cache write:
// reference src/gpu/kernels/split-qkv-rmsnorm-rope-qk.js:101-250.
import { getNative } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { getBuffer } from '../weight-buffer.js';
import { padToQ4KBlock, bufferOf, noteDispatch } from './constants.js';

function assertPositiveInteger(value, label) {
  if (!Number.isInteger(value) || value <= 0) {
    throw new Error(`split_qkv_rmsnorm_rope_qk ${label} must be a positive integer, got ${value}.`);
  }
}

function assertBufferCapacity(buffer, bytes, label) {
  if (!buffer || !Number.isFinite(buffer.size) || buffer.size < bytes) {
    throw new Error(`split_qkv_rmsnorm_rope_qk ${label} buffer is smaller than ${bytes} bytes.`);
  }
}

async function splitQKV(recorder, qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, options = {}) {
  const {
    numTokens, numHeads, numKVHeads, headDim, qSize, kSize, vSize,
    startPos = 0, rotaryDim = headDim, interleaved = false, rmsNormWeightOffset = false, f16KVCacheWrite = null,
  } = options;
  assertPositiveInteger(numTokens, 'numTokens');
  assertPositiveInteger(numHeads, 'numHeads');
  assertPositiveInteger(numKVHeads, 'numKVHeads');
  assertPositiveInteger(headDim, 'headDim');
  assertPositiveInteger(qSize, 'qSize');
  assertPositiveInteger(kSize, 'kSize');
  assertPositiveInteger(vSize, 'vSize');
  if (!Number.isInteger(startPos) || startPos < 0) {
    throw new Error(`split_qkv_rmsnorm_rope_qk startPos must be a non-negative integer, got ${startPos}.`);
  }
  if (qSize !== numHeads * headDim || kSize !== numKVHeads * headDim || vSize !== kSize) {
    throw new Error(`split_qkv_rmsnorm_rope_qk sizes do not match heads*headDim (q=${qSize}, k=${kSize}, v=${vSize}).`);
  }
  if (qkvTensor.dtype !== 'f32') {
    throw new Error(`split_qkv_rmsnorm_rope_qk requires f32 QKV input, got ${qkvTensor.dtype}.`);
  }
  if (!f16KVCacheWrite) {
    throw new Error('split_qkv_rmsnorm_rope_qk: the HIP path always writes K/V into the f16 cache (f16KVCacheWrite).');
  }
  const cos = bufferOf(freqsCos);
  const sin = bufferOf(freqsSin);
  const freqBytes = (startPos + numTokens) * (rotaryDim / 2) * 4;
  assertBufferCapacity(qkvTensor.buffer, numTokens * (qSize + kSize + vSize) * 4, 'QKV input');
  assertBufferCapacity(cos, freqBytes, 'cos frequencies');
  assertBufferCapacity(sin, freqBytes, 'sin frequencies');
  const dst = f16KVCacheWrite.dstOffset;
  if (!Number.isInteger(dst) || dst < 0) {
    throw new Error(`split_qkv_rmsnorm_rope_qk f16KVCacheWrite.dstOffset must be a non-negative integer, got ${dst}.`);
  }
  const cacheBytes = (dst + numTokens * numKVHeads * headDim) * 2;
  assertBufferCapacity(f16KVCacheWrite.keysBuffer, cacheBytes, 'f16 KV keys cache');
  assertBufferCapacity(f16KVCacheWrite.valuesBuffer, cacheBytes, 'f16 KV values cache');
  const qRows = numTokens * numHeads;
  const qOutput = acquireBuffer(qRows * padToQ4KBlock(headDim) * 4, undefined, 'split_qkv_rmsnorm_rope_qk_q_output');
  try {
    getNative().qkvNormRopeKvwrite(qkvTensor.buffer.ptr, getBuffer(qWeight).ptr, getBuffer(kWeight).ptr, cos.ptr, sin.ptr,
      qOutput.ptr, f16KVCacheWrite.keysBuffer.ptr, f16KVCacheWrite.valuesBuffer.ptr, numTokens, numHeads, numKVHeads,
      headDim, startPos, rotaryDim, interleaved ? 1 : 0, eps, rmsNormWeightOffset ? 1 : 0, dst, 1);
  } catch (error) {
    releaseBuffer(qOutput);
    throw error;
  }
  noteDispatch(recorder, 'split_qkv_rmsnorm_rope_qk:f16kv_cache');
  return {
    Q: createTensor(qOutput, 'f32', [qRows, headDim], 'split_qkv_rmsnorm_rope_qk_q_output'),
    K: null,
    V: null,
    wroteF16KVCache: true,
  };
}

export async function runSplitQKVRMSNormRoPEQK(qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, options = {}) {
  return splitQKV(null, qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, options);
}

export async function recordSplitQKVRMSNormRoPEQK(recorder, qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, options = {}) {
  return splitQKV(recorder, qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, options);
}
