// The dependent products of a decoder layer as ONE launch (no counterpart among the reference's ops,
// which issue them one by one: o-projection + residual in attention/interpreter.js:1121-1160, RMSNorm,
// gate/up, activation and down + residual in ffn/standard.js, then the next layer's q/k/v projection),
// optionally with the merge of the decode attention's key splits in front.
// recordDecodeAttentionPartials is recordDecodeAttentionFromQKV without that merge: the splits' partial
// results stay in a workspace that recordLayerChain then reads.
import { getNative, ACT, KV_LAYOUT } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { getBuffer } from '../weight-buffer.js';
import { bufferOf, noteDispatch } from './constants.js';

const PHASE_BYTES = 72;      // struct dh_chain_phase
const SOURCE_BYTES = 48;     // struct dh_chain_attn_source
let sizesChecked = false;

function checkSizes() {
  if (sizesChecked) return;
  const [phase, source] = getNative().chainStructSizes();
  if (phase !== PHASE_BYTES || source !== SOURCE_BYTES) {
    throw new Error(`[GemvChain] struct sizes of the library (${phase}, ${source}) differ from this host's (${PHASE_BYTES}, ${SOURCE_BYTES}).`);
  }
  sizesChecked = true;
}

function ptr(x) {
  if (x === null || x === undefined) return 0n;
  const b = bufferOf(x);
  return b.ptr;
}

// phases: [{weight, weight2?, output, residual?, normWeight?, N, K, activation?, rmsNormWeightOffset?, alpha?,
//           swigluLimit?, rmsNormEps?}] with device buffers / tensors / weight buffers
export function packChainPhases(phases) {
  checkSizes();
  if (!Array.isArray(phases) || phases.length < 1 || phases.length > 4) {
    throw new Error(`[GemvChain] a chain holds 1..4 products, got ${phases && phases.length}.`);
  }
  const bytes = new ArrayBuffer(PHASE_BYTES * phases.length);
  const v = new DataView(bytes);
  phases.forEach((ph, i) => {
    const o = i * PHASE_BYTES;
    for (const [label, n] of [['N', ph.N], ['K', ph.K]]) {
      if (!Number.isInteger(n) || n <= 0) throw new Error(`[GemvChain] product ${i}: ${label} must be a positive integer, got ${n}.`);
    }
    const act = ph.activation || 'silu';
    if (ph.weight2 && !(act in ACT)) throw new Error(`[GemvChain] product ${i}: unknown activation "${act}".`);
    v.setBigUint64(o + 0, ptr(getBuffer(ph.weight)), true);
    v.setBigUint64(o + 8, ph.weight2 ? ptr(getBuffer(ph.weight2)) : 0n, true);
    v.setBigUint64(o + 16, ptr(ph.output), true);
    v.setBigUint64(o + 24, ptr(ph.residual), true);
    v.setBigUint64(o + 32, ptr(ph.normWeight), true);
    v.setInt32(o + 40, ph.N, true);
    v.setInt32(o + 44, ph.K, true);
    v.setInt32(o + 48, ACT[act], true);
    v.setInt32(o + 52, ph.rmsNormWeightOffset ? 1 : 0, true);
    v.setFloat32(o + 56, ph.alpha === undefined ? 1.0 : ph.alpha, true);
    v.setFloat32(o + 60, ph.swigluLimit || 0.0, true);
    v.setFloat32(o + 64, ph.rmsNormEps || 0.0, true);
  });
  return new Uint8Array(bytes);
}

// source: {workspace, numHeads, numKVHeads, headDim, nsplit | kvLenBuffer + maxKvLen, slidingWindow?, kvStart?}
export function packChainAttnSource(source) {
  checkSizes();
  const bytes = new ArrayBuffer(SOURCE_BYTES);
  const v = new DataView(bytes);
  v.setBigUint64(0, ptr(source.workspace), true);
  v.setInt32(8, source.numHeads, true);
  v.setInt32(12, source.numKVHeads, true);
  v.setInt32(16, source.headDim, true);
  v.setInt32(20, source.kvLenBuffer ? 0 : source.nsplit, true);
  v.setBigUint64(24, source.kvLenBuffer ? ptr(source.kvLenBuffer) : 0n, true);
  v.setInt32(32, source.kvLenBuffer ? source.maxKvLen : 0, true);
  v.setInt32(36, source.slidingWindow || 0, true);
  v.setInt32(40, source.kvStart || 0, true);
  return new Uint8Array(bytes);
}

export function layerChainSupported(hidden, inter, qSize) {
  return [hidden, inter, qSize].every((k) => k % 256 === 0 && k >= 2048 && k <= 32768);
}

export function layerChainMergesAttention(numHeads, numKVHeads, headDim, maxKvLen) {
  return getNative().q4kGemvChainAttnSupported(numHeads, numKVHeads, headDim, maxKvLen) === 1;
}

// The split kernel of the fused decode attention alone (see recordDecodeAttentionFromQKV for the options):
// returns {workspace, nsplit} for recordLayerChain's `attention` source; with kvLenBuffer the split count
// follows the device word (nsplit: 0).
export function recordDecodeAttentionPartials(recorder, qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, keys, values, options = {}) {
  const {
    numHeads, numKVHeads = numHeads, headDim, startPos, rotaryDim = headDim, interleaved = false,
    rmsNormWeightOffset = false, useNorm = true, scale = 1.0 / Math.sqrt(headDim), attnSoftcap = 0, slidingWindow = 0,
    kvStart = 0, kvLayout = 'contiguous', kvLenBuffer = null, maxKvLen = 0,
  } = options;
  if (!(kvLayout in KV_LAYOUT)) throw new Error(`[Attention] kvLayout "${kvLayout}" is not supported by the HIP path (contiguous, ring).`);
  if (kvLenBuffer) {
    if (!Number.isInteger(maxKvLen) || maxKvLen < 1) throw new Error(`[Attention] kvLenBuffer needs a positive maxKvLen, got ${maxKvLen}.`);
  } else if (!Number.isInteger(startPos) || startPos < 0) {
    throw new Error(`[Attention] fused decode startPos must be a non-negative integer, got ${startPos}.`);
  }
  const native = getNative();
  const lastPos = kvLenBuffer ? kvStart + maxKvLen - 1 : startPos;
  const workspace = acquireBuffer(native.attnDecodeWorkspaceBytes(numHeads, headDim, lastPos - kvStart + 1), undefined,
    'attention_splitk_workspace');
  let nsplit = 0;
  try {
    const head = [qkvTensor.buffer.ptr, useNorm ? getBuffer(qWeight).ptr : 0n, useNorm ? getBuffer(kWeight).ptr : 0n,
      bufferOf(freqsCos).ptr, bufferOf(freqsSin).ptr, keys.buffer.ptr, values.buffer.ptr, numHeads, numKVHeads, headDim];
    const tail = [rotaryDim, interleaved ? 1 : 0, eps, rmsNormWeightOffset ? 1 : 0, useNorm ? 1 : 0, scale, attnSoftcap,
      slidingWindow, kvStart, KV_LAYOUT[kvLayout], workspace.ptr];
    if (kvLenBuffer) native.attnDecodeQkvKvLenPartials(...head, kvLenBuffer.ptr, maxKvLen, ...tail);
    else nsplit = native.attnDecodeQkvPartials(...head, startPos, ...tail);
  } catch (error) {
    releaseBuffer(workspace);
    throw error;
  }
  noteDispatch(recorder, 'attention:partials');
  return { workspace, nsplit, numHeads, numKVHeads, headDim, kvLenBuffer, maxKvLen, slidingWindow, kvStart };
}

// One launch: [merge of `attention` partial results |] input -> phases.  Outputs are the phases' `output`
// buffers (caller-supplied).  input: tensor/buffer of the first product's activations, or null with `attention`.
export function recordLayerChain(recorder, input, phases, attention = null) {
  const native = getNative();
  const packed = packChainPhases(phases);
  if (attention) native.q4kGemvChainAttn(packChainAttnSource(attention), packed, phases.length);
  else native.q4kGemvChain(ptr(input), packed, phases.length);
  noteDispatch(recorder, attention ? 'gemv_chain:attn' : 'gemv_chain');
}

export function chainOutputTensor(buffer, n, label) {
  return createTensor(buffer, 'f32', [1, n], label);
}
