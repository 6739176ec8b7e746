// Op API of the HIP path: the subset of the reference's src/gpu/kernels/index.js that the
// text pipeline's quantized decode path calls (src/inference/pipelines/text/ops.js:3-30,
// attention/interpreter.js:6-23).  Same names, argument order and option names.
export { runMatmul, recordMatmul, runDequantQ4K } from './matmul.js';
export { runFusedFFN, recordFusedFFN, runFusedNormedFFN, recordFusedNormedFFN } from './fused_ffn.js';
export { runAttention, recordAttention } from './attention.js';
export { runDecodeAttentionFromQKV, recordDecodeAttentionFromQKV, decodeAttentionFromQKVSupported } from './attention-from-qkv.js';
export {
  recordLayerChain, recordDecodeAttentionPartials, layerChainSupported, layerChainMergesAttention, packChainPhases,
  packChainAttnSource,
} from './gemv-chain.js';
export { runRMSNorm, recordRMSNorm } from './rmsnorm.js';
export { runRMSNormQK, recordRMSNormQK, canUseRMSNormQK } from './rmsnorm-qk.js';
export {
  runSandwichRMSNormPair, recordSandwichRMSNormPair, runResidualNextRMSNormPair, recordResidualNextRMSNormPair,
} from './rmsnorm-pair.js';
export { runRoPE, recordRoPE } from './rope.js';
export { runRoPEQK, recordRoPEQK, canUseRoPEQK } from './rope-qk.js';
export { runKVCacheWriteF32ToF16, recordKVCacheWriteF32ToF16 } from './kv-cache-write.js';
export { runSplitQKVRMSNormRoPEQK, recordSplitQKVRMSNormRoPEQK } from './split-qkv-rmsnorm-rope-qk.js';
export { runSiLU, recordSiLU, runSiLURowSplit, recordSiLURowSplit } from './silu.js';
export { runGeLU, recordGeLU } from './gelu.js';
export { runResidualAdd, recordResidualAdd } from './residual.js';
export { runSplitQKV, recordSplitQKV } from './split_qkv.js';
export { runBiasAdd, recordBiasAdd, runScale, recordScale } from './bias-scale.js';
export { runGather, recordGather } from './gather.js';
export { runArgmax, recordArgmax, runGPUSample, recordGPUSample, seededRandom } from './sample.js';
export { recordLmHeadArgmax, recordLmHeadArgmaxF16, lmHeadArgmaxNormFusable } from './lm-head-argmax.js';
export { castF32ToF16, castF16ToF32, recordCastF32ToF16, recordCastF16ToF32 } from './cast.js';
export {
  runMatmulRMSNormFused, recordMatmulRMSNormFused, shouldUseFusedMatmulRMSNorm, selectMatmulRMSNormFusedVariant,
} from './fused_matmul_rmsnorm.js';
export {
  recordCheckFiniteness, createFinitenessStatusBuffer, parseFinitenessStatusWords, resolveFinitenessAbsThreshold,
  shouldTriggerFinitenessValue, DEFAULT_FINITENESS_ABS_THRESHOLD, FINITENESS_STATUS_BYTES,
} from './check-finiteness.js';
