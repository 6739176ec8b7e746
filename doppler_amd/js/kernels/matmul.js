// runMatmul / recordMatmul: reference src/gpu/kernels/matmul.js:280-666 for the weight
// dtypes the HIP path serves: 'q4k' (row layout) and 'f16' ([N, K] row-major).
import { getNative, DTYPE } from '../native.js';
import { createTensor } from '../tensor.js';
import { acquireBuffer, releaseBuffer } from '../buffer-pool.js';
import { getBuffer, getWeightDtype } from '../weight-buffer.js';
import { QK_K, Q4K_BLOCK_BYTES, ptrOf, noteDispatch } from './constants.js';

const STORAGE_ALIGNMENT = 256;

function requireOutputDtype(dtype, opLabel) {
  if (dtype === 'f16' || dtype === 'f32') return dtype;
  throw new Error(`[${opLabel}] options.outputDtype is required and must be "f16" or "f32", got ${String(dtype)}.`);
}

function validateDimensions(label, M, N, K) {
  if (!Number.isFinite(M) || !Number.isFinite(N) || !Number.isFinite(K)) {
    throw new Error(`[${label}] Invalid dimensions: M=${M}, N=${N}, K=${K}`);
  }
  if (M <= 0 || N <= 0 || K <= 0) {
    throw new Error(`[${label}] Dimensions must be positive: M=${M}, N=${N}, K=${K}`);
  }
}

function validateOffsets(label, aOffset, bOffset, cOffset) {
  if (!Number.isFinite(aOffset) || aOffset < 0 || !Number.isFinite(bOffset) || bOffset < 0 ||
      !Number.isFinite(cOffset) || cOffset < 0) {
    throw new Error(`[${label}] Invalid buffer offsets: aOffset=${aOffset}, bOffset=${bOffset}, cOffset=${cOffset}`);
  }
  if (aOffset % STORAGE_ALIGNMENT !== 0 || bOffset % STORAGE_ALIGNMENT !== 0 || cOffset % STORAGE_ALIGNMENT !== 0) {
    throw new Error(
      `[${label}] Buffer offsets must be ${STORAGE_ALIGNMENT}-byte aligned: ` +
      `aOffset=${aOffset}, bOffset=${bOffset}, cOffset=${cOffset}`
    );
  }
}

async function executeMatmul(recorder, A, B, M, N, K, options = {}) {
  const opLabel = recorder ? 'recordMatmul' : 'runMatmul';
  const {
    alpha = 1.0,
    outputBuffer = null,
    transposeB = true,
    aOffset = 0,
    bOffset = 0,
    cOffset = 0,
    residualTensor = null,
  } = options;
  validateDimensions(opLabel, M, N, K);
  const weightDtype = getWeightDtype(B) || options.bDtype;
  if (weightDtype === null || weightDtype === undefined || weightDtype === '') {
    const details = [
      options.role ? `role=${options.role}` : null,
      Number.isFinite(options.layerIdx) ? `layer=${options.layerIdx}` : null,
      B && B.label ? `label=${B.label}` : null,
    ].filter(Boolean);
    throw new Error(`[${opLabel}] B dtype is required for matmul dispatch${details.length ? ` (${details.join(', ')})` : ''}.`);
  }
  const outputDtype = requireOutputDtype(options.outputDtype, opLabel);
  validateOffsets(opLabel, aOffset, bOffset, cOffset);
  if (A.dtype !== 'f32' && A.dtype !== 'f16') {
    throw new Error(`[${opLabel}] the HIP path takes f32 or f16 activations, got ${A.dtype}.`);
  }
  const fusedNorm = weightDtype === 'q4k' && options.normWeight != null && options.useFusedRmsnormWideTile === true;
  if (A.dtype === 'f16' && (weightDtype !== 'q4k' || fusedNorm)) {
    // reference: the f16-activation Q4_K kernels (fused_matmul_q4_f16a.wgsl and its batched forms)
    throw new Error(`[${opLabel}] f16 activations are served for q4k weights without the fused RMSNorm only.`);
  }
  const aBuf = getBuffer(A);
  const bBuf = getBuffer(B);
  const aRequired = aOffset + M * K * (A.dtype === 'f16' ? 2 : 4);
  if (aBuf.size < aRequired) {
    throw new Error(`[${opLabel}] A buffer too small: ${aBuf.size} < ${aRequired} (M=${M}, K=${K}, aDtype=${A.dtype})`);
  }
  let bRequired;
  if (weightDtype === 'q4k') {
    bRequired = bOffset + N * Math.ceil(K / QK_K) * Q4K_BLOCK_BYTES;
  } else if (weightDtype === 'f16') {
    if (transposeB !== true && transposeB !== 'auto') {
      throw new Error(`[${opLabel}] f16 weights must be [N, K] row-major (transposeB=true) on the HIP path.`);
    }
    bRequired = bOffset + N * K * 2;
  } else {
    throw new Error(`[${opLabel}] weight dtype "${weightDtype}" is not supported by the HIP path (q4k, f16).`);
  }
  if (bBuf.size < bRequired) {
    throw new Error(
      `[${opLabel}] B buffer too small: ${bBuf.size} < ${bRequired} ` +
      `(N=${N}, K=${K}, bDtype=${weightDtype}, transposeB=${transposeB})`
    );
  }
  const elementSize = outputDtype === 'f16' ? 2 : 4;
  const outputSize = M * N * elementSize;
  const output = outputBuffer || acquireBuffer(outputSize, undefined, 'matmul_output');
  const owned = outputBuffer ? null : output;
  try {
    if (output.size < cOffset + outputSize) {
      throw new Error(`[${opLabel}] C buffer too small: ${output.size} < ${cOffset + outputSize}`);
    }
    const native = getNative();
    const aPtr = aBuf.ptr + BigInt(aOffset);
    const bPtr = bBuf.ptr + BigInt(bOffset);
    const cPtr = output.ptr + BigInt(cOffset);
    if (fusedNorm) {
      // RMSNorm of A inside the matmul (reference: matmul-selection.js:609-620)
      if (!Number.isFinite(options.rmsNormEps)) {
        throw new Error(`[${opLabel}] rmsNormEps is required with normWeight.`);
      }
      const normDtype = getWeightDtype(options.normWeight) || options.normWeight.dtype || 'f32';
      if (normDtype !== 'f32') {
        throw new Error(`[${opLabel}] the fused RMSNorm prologue takes an f32 norm weight, got ${normDtype}.`);
      }
      native.q4kMatmulRmsnorm(aPtr, ptrOf(options.normWeight), options.rmsNormEps, options.rmsNormOffset === true ? 1 : 0,
        bPtr, cPtr, DTYPE[outputDtype], M, N, K, alpha, ptrOf(residualTensor));
    } else if (weightDtype === 'q4k') {
      native.q4kMatmul(aPtr, DTYPE[A.dtype], bPtr, cPtr, DTYPE[outputDtype], M, N, K, alpha, ptrOf(residualTensor));
    } else {
      if (outputDtype !== 'f32' || residualTensor) {
        throw new Error(`[${opLabel}] f16-weight matmul produces f32 without a fused residual on the HIP path.`);
      }
      native.f16wMatmul(aPtr, bPtr, cPtr, M, N, K, alpha);
    }
    noteDispatch(recorder, options.role ? `matmul:${options.role}` : 'matmul');
    return createTensor(output, outputDtype, [M, N], 'matmul_output');
  } catch (error) {
    if (owned) releaseBuffer(owned);
    throw error;
  }
}

export async function runMatmul(A, B, M, N, K, options = {}) {
  return executeMatmul(null, A, B, M, N, K, options);
}

export async function recordMatmul(recorder, A, B, M, N, K, options = {}) {
  return executeMatmul(recorder, A, B, M, N, K, options);
}

// Bit-exact Q4_K -> f32 (reference: src/gpu/kernels/dequant.js, q4k variants).
export async function runDequantQ4K(weight, numBlocks, options = {}) {
  const buf = getBuffer(weight);
  if (buf.size < numBlocks * Q4K_BLOCK_BYTES) {
    throw new Error(`[Dequant] Q4_K buffer too small: ${buf.size} < ${numBlocks * Q4K_BLOCK_BYTES}`);
  }
  const output = options.outputBuffer || acquireBuffer(numBlocks * QK_K * 4, undefined, 'dequant_output');
  getNative().q4kDequant(buf.ptr, numBlocks, output.ptr);
  return createTensor(output, 'f32', [numBlocks * QK_K], 'dequant_output');
}
