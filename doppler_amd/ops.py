"""Python host mirror of the reference's op API for the quantized-inference hot path.

Names, argument meaning and error behaviour follow the reference's JavaScript wrappers
(src/gpu/kernels/index.js): `runMatmul`, `runAttention`, `runRMSNorm`, `runRoPE`,
`runKVCacheWriteF32ToF16`, `runSplitQKVRMSNormRoPEQK`, `runSiLU`, `runSiLURowSplit`, `runGeLU`,
`runResidualAdd`, `runBiasAdd`, `runScale`, `runSplitQKV`, `runRoPEQK`, `runGather`, `runFusedFFN`, `runArgmax`,
`recordLmHeadArgmaxF16`, `runMatmulRMSNormFused`, `recordCheckFiniteness`, plus the
handle helpers `createTensor` / `createWeightBuffer` and the pool calls `acquireBuffer` /
`uploadData` / `readBuffer`.  Options are keyword arguments with the reference's camelCase
names.  Every op goes through the C ABI of libdopplerhip.so; torch only provides device
memory (a buffer is a torch.uint8 CUDA tensor) -- there is no torch or CPU compute path.
"""
import math

import numpy as np
import torch

from . import capi
from .capi import DopplerHipError

QK_K = 256
Q4K_BLOCK_BYTES = 144


def padToQ4KBlock(size):
    """src/config/schema/quantization.schema.js:26-28"""
    return (size + QK_K - 1) // QK_K * QK_K


class Tensor:
    """src/gpu/tensor.js:7-19 createTensor: {buffer, dtype, shape, label}."""
    __slots__ = ("buffer", "dtype", "shape", "label")

    def __init__(self, buffer, dtype, shape, label=None):
        self.buffer, self.dtype, self.shape, self.label = buffer, dtype, tuple(shape), label


class WeightBuffer:
    """src/gpu/weight-buffer.js:78-115 createWeightBuffer."""
    __slots__ = ("buffer", "dtype", "layout", "shape", "label")

    def __init__(self, buffer, dtype, layout, shape, label=None):
        self.buffer, self.dtype, self.layout, self.shape, self.label = buffer, dtype, layout, tuple(shape), label


def createTensor(buffer, dtype, shape, label=None):
    return Tensor(buffer, dtype, shape, label)


def createWeightBuffer(buffer, dtype, layout, shape, label=None):
    return WeightBuffer(buffer, dtype, layout, shape, label)


def _lib():
    if not torch.cuda.is_available():
        raise DopplerHipError("no GPU visible: the HIP path cannot run (there is no CPU fallback)")
    return capi.init(torch.cuda.current_device())


def _dev():
    return torch.device("cuda", torch.cuda.current_device())


# ------------------------------------------------------------------ buffer pool mirror

def acquireBuffer(size, usage=None, label=None):
    """src/memory/buffer-pool.js:815 acquireBuffer(size, usage, label): zero-filled device bytes."""
    _lib()
    return torch.zeros(int(size), dtype=torch.uint8, device=_dev())


def releaseBuffer(buffer):
    return None   # torch's caching allocator owns the memory


def uploadData(buffer, data, offset=0):
    """src/memory/buffer-pool.js:863 uploadData(buffer, data, offset)."""
    src = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
    if offset + src.size > buffer.numel():
        raise DopplerHipError("uploadData: %d bytes at offset %d exceed buffer of %d" % (src.size, offset, buffer.numel()))
    capi.check(_lib().dh_upload(buffer.data_ptr(), offset, src.ctypes.data, src.size))
    return buffer


def readBuffer(buffer, size=None, dtype=np.uint8):
    """src/memory/buffer-pool.js:866 readBuffer(buffer, size): waits for queued work."""
    size = buffer.numel() * buffer.element_size() if size is None else int(size)
    out = np.empty(size, np.uint8)
    capi.check(_lib().dh_download(out.ctypes.data, buffer.data_ptr(), 0, size))
    return out.view(dtype)


def tensorFromNumpy(arr, dtype=None, label=None):
    """Upload a numpy array as a Tensor (f32 stays f32; uint16 is taken as f16 bits)."""
    arr = np.ascontiguousarray(arr)
    if dtype is None:
        dtype = "f16" if arr.dtype in (np.uint16, np.float16) else "f32"
    buf = acquireBuffer(max(arr.nbytes, 4))
    uploadData(buf, arr)
    return Tensor(buf, dtype, arr.shape, label)


def readTensor(t, count=None):
    n = int(np.prod(t.shape)) if count is None else count
    if t.dtype == "f16":
        return readBuffer(t.buffer, n * 2, np.uint16)
    return readBuffer(t.buffer, n * 4, np.float32)


def _buf(x):
    return x.buffer if isinstance(x, (Tensor, WeightBuffer)) else x


def _ptr(x):
    return None if x is None else _buf(x).data_ptr()


def _nbytes(x):
    b = _buf(x)
    return b.numel() * b.element_size()


def _out(outputBuffer, nbytes):
    if outputBuffer is not None:
        if _nbytes(outputBuffer) < nbytes:
            raise DopplerHipError("output buffer too small: %d < %d" % (_nbytes(outputBuffer), nbytes))
        return _buf(outputBuffer)
    return acquireBuffer(nbytes)


def _act_code(activation, op):
    if activation == "silu":
        return capi.ACT_SILU
    if activation in ("gelu", "gelu_tanh", "geglu"):
        return capi.ACT_GELU
    raise DopplerHipError("[%s] unsupported activation %r" % (op, activation))


# ------------------------------------------------------------------ matmul

def runMatmul(A, B, M, N, K, alpha=1.0, outputBuffer=None, transposeB=True, outputDtype=None, role=None,
              layerIdx=None, residualTensor=None, normWeight=None, rmsNormEps=None, rmsNormOffset=False,
              useFusedRmsnormWideTile=False, **_ignored):
    """src/gpu/kernels/matmul.js:659 runMatmul(A, B, M, N, K, options) for q4k ('row') and f16
    weights ([N, K] row-major, transposeB true).  With `normWeight` and
    `useFusedRmsnormWideTile` the RMSNorm of A runs inside the matmul
    (src/gpu/kernels/matmul-selection.js:609-620)."""
    op = "runMatmul"
    for v in (M, N, K):
        if not isinstance(v, (int, np.integer)):
            raise DopplerHipError("[%s] Invalid dimensions: M=%s, N=%s, K=%s" % (op, M, N, K))
    if M <= 0 or N <= 0 or K <= 0:
        raise DopplerHipError("[%s] Dimensions must be positive: M=%s, N=%s, K=%s" % (op, M, N, K))
    if outputDtype not in ("f16", "f32"):
        raise DopplerHipError('[%s] options.outputDtype is required and must be "f16" or "f32", got %s.' % (op, outputDtype))
    bdtype = B.dtype if isinstance(B, (Tensor, WeightBuffer)) else None
    if not bdtype:
        raise DopplerHipError("[%s] B dtype is required for matmul dispatch%s." % (op, " (role=%s)" % role if role else ""))
    if A.dtype not in ("f32", "f16"):
        raise DopplerHipError("[%s] f32 or f16 activations required, got %s" % (op, A.dtype))
    a_elem = 2 if A.dtype == "f16" else 4
    if _nbytes(A) < M * K * a_elem:
        raise DopplerHipError("[%s] A buffer too small: %d < %d (M=%d, K=%d, aDtype=%s)"
                              % (op, _nbytes(A), M * K * a_elem, M, K, A.dtype))
    if A.dtype == "f16" and (bdtype != "q4k" or (normWeight is not None and useFusedRmsnormWideTile)):
        raise DopplerHipError("[%s] f16 activations are served for q4k weights without the fused RMSNorm only" % op)
    L = _lib()
    if bdtype == "q4k":
        need = N * ((K + QK_K - 1) // QK_K) * Q4K_BLOCK_BYTES
        if _nbytes(B) < need:
            raise DopplerHipError("[%s] B buffer too small: %d < %d (N=%d, K=%d, bDtype=q4k, transposeB=%s)"
                                  % (op, _nbytes(B), need, N, K, transposeB))
        out = _out(outputBuffer, M * N * (2 if outputDtype == "f16" else 4))
        cdt = capi.F16 if outputDtype == "f16" else capi.F32
        if normWeight is not None and useFusedRmsnormWideTile:
            if rmsNormEps is None:
                raise DopplerHipError("[%s] rmsNormEps is required with normWeight" % op)
            if getattr(normWeight, "dtype", "f32") != "f32":
                raise DopplerHipError("[%s] fused RMSNorm requires an f32 norm weight" % op)
            capi.check(L.dh_q4k_matmul_rmsnorm(_ptr(A), _ptr(normWeight), float(rmsNormEps),
                                               1 if rmsNormOffset else 0, _ptr(B), out.data_ptr(), cdt,
                                               M, N, K, alpha, _ptr(residualTensor)))
        else:
            capi.check(L.dh_q4k_matmul(_ptr(A), capi.F16 if A.dtype == "f16" else capi.F32, _ptr(B),
                                       out.data_ptr(), cdt, M, N, K, alpha, _ptr(residualTensor)))
        return Tensor(out, outputDtype, (M, N), "matmul_output")
    if bdtype == "f16":
        if transposeB not in (True, "auto"):
            raise DopplerHipError("[%s] f16 weights must be row-major [N, K] (transposeB=true)" % op)
        if outputDtype != "f32" or residualTensor is not None:
            raise DopplerHipError("[%s] f16-weight matmul supports f32 output without residual only" % op)
        if _nbytes(B) < N * K * 2:
            raise DopplerHipError("[%s] B buffer too small: %d < %d (N=%d, K=%d, bDtype=f16, transposeB=true)"
                                  % (op, _nbytes(B), N * K * 2, N, K))
        out = _out(outputBuffer, M * N * 4)
        capi.check(L.dh_f16w_matmul(_ptr(A), _ptr(B), out.data_ptr(), M, N, K, alpha))
        return Tensor(out, "f32", (M, N), "matmul_output")
    raise DopplerHipError("[%s] weight dtype %r is not supported by the HIP path" % (op, bdtype))


# Limits of the fused dense matmul + RMSNorm (src/config/schema/kernel-thresholds.schema.js:87-88).
FUSED_MATMUL_MAX_MEDIUM_N = 4096
FUSED_MATMUL_MAX_MEDIUM_K = 8192
_WORKGROUP_SIZE_DEFAULT = 256


def selectMatmulRMSNormFusedVariant(N, dtype):
    """src/gpu/kernels/fused_matmul_rmsnorm.js:30-37 with the rule table of
    src/rules/kernels/fused-matmul-rmsnorm.rules.json.  The name is informational here: one pair
    of kernels serves every N."""
    if not dtype:
        raise DopplerHipError("[MatmulRMSNormFused] dtype is required for variant selection.")
    small = N <= _WORKGROUP_SIZE_DEFAULT
    f16 = dtype == "f16"
    return ("small" if small else "medium") + ("_f16" if f16 else "")


def shouldUseFusedMatmulRMSNorm(M, N, K=None):
    """src/gpu/kernels/fused_matmul_rmsnorm.js:295-312."""
    if M != 1 or N > FUSED_MATMUL_MAX_MEDIUM_N:
        return False
    if isinstance(K, (int, float, np.integer)) and not isinstance(K, bool) and K > FUSED_MATMUL_MAX_MEDIUM_K:
        return False
    return True


def runMatmulRMSNormFused(input, weight, normWeight, options=None, **kw):
    """src/gpu/kernels/fused_matmul_rmsnorm.js:50 runMatmulRMSNormFused(input, weight, normWeight,
    {N, K, eps, residual, outputBuffer, transposeB, rmsNormWeightOffset, label}): one activation
    row through a dense weight ([N, K] with transposeB, else [K, N]), RMSNorm over the N outputs,
    residual added after the norm; all f32, or all f16 with f32 sums (the output dtype is the
    input's, as in the reference)."""
    o = dict(options or {})
    o.update(kw)
    if o.get("transposeB") is None:
        raise DopplerHipError("[MatmulRMSNormFused] transposeB is required.")
    if o.get("rmsNormWeightOffset") is None:
        raise DopplerHipError("[MatmulRMSNormFused] rmsNormWeightOffset is required.")
    if o.get("eps") is None:
        raise DopplerHipError("[MatmulRMSNormFused] eps is required.")
    N, K = o.get("N"), o.get("K")
    for v in (N, K):
        if not isinstance(v, (int, np.integer)) or v <= 0:
            raise DopplerHipError("[MatmulRMSNormFused] N and K must be positive integers: N=%s, K=%s" % (N, K))
    if N > FUSED_MATMUL_MAX_MEDIUM_N:
        raise DopplerHipError("[MatmulRMSNormFused] N=%d exceeds maxMediumN=%d; kernel only supports "
                              "single-workgroup RMSNorm." % (N, FUSED_MATMUL_MAX_MEDIUM_N))
    if not getattr(input, "dtype", None):
        raise DopplerHipError("[MatmulRMSNormFused] input dtype is required.")
    selectMatmulRMSNormFusedVariant(N, input.dtype)
    dtype = input.dtype
    if dtype not in ("f32", "f16"):
        raise DopplerHipError("[MatmulRMSNormFused] f32 or f16 activations required, got %s" % dtype)
    elem = 2 if dtype == "f16" else 4
    # the f16 variants take f16 weights, residual and output as well (fused_matmul_rmsnorm_f16.wgsl:41-45)
    wdtype = weight.dtype if isinstance(weight, (Tensor, WeightBuffer)) else dtype
    if wdtype != dtype:
        raise DopplerHipError("[MatmulRMSNormFused] dense %s weights required for %s activations, got %s"
                              % (dtype, dtype, wdtype))
    if _nbytes(input) < K * elem or _nbytes(weight) < N * K * elem:
        raise DopplerHipError("[MatmulRMSNormFused] input or weight buffer too small for N=%d, K=%d" % (N, K))
    # the reference tells an f16 norm weight from an f32 one by the buffer's size (:14-28)
    nw_bytes = _nbytes(normWeight)
    if nw_bytes >= N * 4:
        nw = capi.F32
    elif nw_bytes >= N * 2:
        nw = capi.F16
    else:
        raise DopplerHipError("[MatmulRMSNormFused] norm weight size (%d bytes) does not match hiddenSize=%d "
                              "(expected %d or %d bytes)." % (nw_bytes, N, N * 2, N * 4))
    residual = o.get("residual")
    if residual is not None and _nbytes(residual) < N * elem:
        raise DopplerHipError("[MatmulRMSNormFused] residual buffer smaller than N=%d elements" % N)
    if residual is not None and getattr(residual, "dtype", dtype) != dtype:
        raise DopplerHipError("[MatmulRMSNormFused] residual dtype must match the input's (%s)" % dtype)
    out = _out(o.get("outputBuffer"), N * elem)
    fn = _lib().dh_matmul_rmsnorm_f16 if dtype == "f16" else _lib().dh_matmul_rmsnorm_f32
    capi.check(fn(_ptr(input), _ptr(weight), 1 if o["transposeB"] else 0, _ptr(normWeight), nw, float(o["eps"]),
                  1 if o["rmsNormWeightOffset"] else 0, _ptr(residual), out.data_ptr(), int(N), int(K)))
    return Tensor(out, dtype, (1, N), "matmul_rmsnorm_fused_output")


def recordMatmulRMSNormFused(recorder, input, weight, normWeight, options=None, **kw):
    """src/gpu/kernels/fused_matmul_rmsnorm.js:173 recordMatmulRMSNormFused.  `recorder` is accepted
    for signature parity: every op already enqueues in order on one stream."""
    return runMatmulRMSNormFused(input, weight, normWeight, options, **kw)


# ------------------------------------------------------------------ finiteness guard

DEFAULT_FINITENESS_ABS_THRESHOLD = 65500
FINITENESS_STATUS_BYTES = 16


def resolveFinitenessAbsThreshold(value):
    """src/gpu/kernels/check-finiteness.js:7-12."""
    if isinstance(value, (int, float, np.integer, np.floating)) and not isinstance(value, bool) \
            and math.isfinite(value) and value > 0:
        return value
    return DEFAULT_FINITENESS_ABS_THRESHOLD


def shouldTriggerFinitenessValue(value, absThreshold=DEFAULT_FINITENESS_ABS_THRESHOLD):
    """src/gpu/kernels/check-finiteness.js:14-19."""
    if not math.isfinite(value):
        return True
    return abs(value) > resolveFinitenessAbsThreshold(absThreshold)


def parseFinitenessStatusWords(words, offset=0):
    """src/inference/pipelines/text/finiteness-guard-status.js:1-21."""
    status = int(words[offset]) if offset < len(words) else 0
    if status <= 0:
        return {"triggered": False, "layer": 0, "step": 0, "metadata": ""}
    layer = int(words[offset + 1]) if offset + 1 < len(words) else 0
    step = int(words[offset + 2]) if offset + 2 < len(words) else 0
    return {"triggered": True, "layer": layer, "step": step, "metadata": " (layer %d, step %d)" % (layer, step)}


def createFinitenessStatusBuffer():
    """Four zeroed u32 words: [status, layer, step, pad], the layout the reference copies beside
    the sampled token (src/inference/pipelines/text/generator-steps.js:786-798)."""
    buf = acquireBuffer(FINITENESS_STATUS_BYTES)
    buf.zero_()
    return buf


def recordCheckFiniteness(target, inputBuffer, size, statusBuffer, layerIdx=0, step=0,
                          absThreshold=DEFAULT_FINITENESS_ABS_THRESHOLD, inputDtype=None):
    """src/gpu/kernels/check-finiteness.js:98 recordCheckFiniteness(target, inputBuffer, size,
    statusBuffer, layerIdx, step, absThreshold).  The reference's shader reads f16; here the
    element type is the tensor's (or `inputDtype` for a bare buffer, default f16 as there)."""
    dtype = inputDtype or getattr(inputBuffer, "dtype", None)
    if not isinstance(dtype, str):
        dtype = "f16"
    if dtype not in ("f16", "f32"):
        raise DopplerHipError("[check_finiteness] input dtype must be f16 or f32, got %s" % dtype)
    elem = 2 if dtype == "f16" else 4
    if _nbytes(inputBuffer) < size * elem:
        raise DopplerHipError("[check_finiteness] input buffer smaller than size=%d" % size)
    if _nbytes(statusBuffer) < FINITENESS_STATUS_BYTES:
        raise DopplerHipError("[check_finiteness] status buffer must hold 4 u32 words")
    capi.check(_lib().dh_check_finiteness(_ptr(inputBuffer), capi.F16 if dtype == "f16" else capi.F32, int(size),
                                          _ptr(statusBuffer), int(layerIdx), int(step),
                                          float(resolveFinitenessAbsThreshold(absThreshold))))


def runDequantQ4K(W, numBlocks, outputBuffer=None):
    """Dequantize Q4_K super-blocks to f32 (src/gpu/kernels/dequant.js dequantize, q4k -> f32)."""
    if _nbytes(W) < numBlocks * Q4K_BLOCK_BYTES:
        raise DopplerHipError("[runDequantQ4K] weight buffer too small")
    out = _out(outputBuffer, numBlocks * QK_K * 4)
    capi.check(_lib().dh_q4k_dequant(_ptr(W), numBlocks, out.data_ptr()))
    return Tensor(out, "f32", (numBlocks * QK_K,), "dequant_output")


def runFusedFFN(input, W_gate, W_up, hiddenSize, intermediateSize, batchSize=1, activation="silu",
                alpha=1.0, outputBuffer=None, swigluLimit=None, **_ignored):
    """src/gpu/kernels/fused_ffn.js:501 runFusedFFN."""
    gd = W_gate.dtype if isinstance(W_gate, (Tensor, WeightBuffer)) else None
    ud = W_up.dtype if isinstance(W_up, (Tensor, WeightBuffer)) else None
    if not gd or not ud:
        raise DopplerHipError("Fused FFN requires explicit gate/up weight dtypes")
    if gd != ud:
        raise DopplerHipError("Fused FFN requires matching gate/up dtypes (gate=%s, up=%s)" % (gd, ud))
    if gd != "q4k":
        raise DopplerHipError("Fused FFN does not support %s weights" % gd)
    if input.dtype != "f32":
        raise DopplerHipError("Fused FFN requires f32 activations")
    out = _out(outputBuffer, batchSize * intermediateSize * 4)
    capi.check(_lib().dh_q4k_ffn_gate_up(_ptr(input), _ptr(W_gate), _ptr(W_up), out.data_ptr(), batchSize,
                                         hiddenSize, intermediateSize, _act_code(activation, "FusedFFN"),
                                         alpha, float(swigluLimit or 0.0) if activation == "silu" else 0.0))
    return Tensor(out, "f32", (batchSize, intermediateSize), "fused_ffn_output")


def runFusedNormedFFN(input, normWeight, eps, W_gate, W_up, hiddenSize, intermediateSize, batchSize=1,
                      activation="silu", alpha=1.0, outputBuffer=None, swigluLimit=None,
                      rmsNormWeightOffset=False, **_ignored):
    """Gate/up projection + gated activation over RMSNorm(input) in one launch.  Stands in for
    src/gpu/kernels/fused_ffn.js:770 runFusedFFNFromRMSNormStats; the inverse RMS that the
    reference takes as a buffer from its rmsnorm-stats pass is computed in the kernel prologue."""
    gd = W_gate.dtype if isinstance(W_gate, (Tensor, WeightBuffer)) else None
    ud = W_up.dtype if isinstance(W_up, (Tensor, WeightBuffer)) else None
    if gd != "q4k" or ud != "q4k":
        raise DopplerHipError("Fused normed FFN requires Q4_K gate/up weights; got gate=%s, up=%s." % (gd, ud))
    if input.dtype != "f32":
        raise DopplerHipError("Fused normed FFN requires f32 prenorm input; got %s." % input.dtype)
    if normWeight is None:
        raise DopplerHipError("Fused normed FFN requires a norm weight buffer.")
    out = _out(outputBuffer, batchSize * intermediateSize * 4)
    capi.check(_lib().dh_q4k_ffn_gate_up_rmsnorm(
        _ptr(input), _ptr(normWeight), float(eps), 1 if rmsNormWeightOffset else 0, _ptr(W_gate), _ptr(W_up),
        out.data_ptr(), batchSize, hiddenSize, intermediateSize, _act_code(activation, "FusedNormedFFN"), alpha,
        float(swigluLimit or 0.0) if activation == "silu" else 0.0))
    return Tensor(out, "f32", (batchSize, intermediateSize), "fused_normed_ffn_output")


# ------------------------------------------------------------------ attention

def attentionWorkspaceBytes(numHeads, headDim, kvLen):
    return int(capi.load().dh_attn_decode_workspace_bytes(numHeads, headDim, kvLen))


def runAttention(Q, K, V, mask, numHeads, headDim, seqLen=1, kvLen=None, numKVHeads=None, scale=None,
                 causal=True, startPos=0, outputBuffer=None, attnSoftcap=0, slidingWindow=0, kvStart=0,
                 kvLayout="contiguous", workspace=None, kvLenBuffer=None, **_ignored):
    """src/gpu/kernels/attention.js:2007 runAttention over an f16 KV cache: decode (seqLen == 1,
    split-K kernel) or prefill (seqLen > 1, matrix-core flash kernel).  kvLenBuffer (decode only): a
    device u32 holding the key count, read by the kernels (attention.js:1071,1224-1232); kvLen then
    bounds it, and startPos < 0 places the query at the last key."""
    kvLen = seqLen if kvLen is None else kvLen
    numKVHeads = numHeads if numKVHeads is None else numKVHeads
    scale = 1.0 / math.sqrt(headDim) if scale is None else scale
    if seqLen < 1:
        raise DopplerHipError("[Attention] seqLen must be positive, got %d" % seqLen)
    if mask is not None:
        raise DopplerHipError("[Attention] explicit masks are not supported on the HIP path")
    if Q.dtype not in ("f32", "f16") or K.dtype != "f16" or V.dtype != "f16":
        raise DopplerHipError("[Attention] the HIP path needs f32 or f16 Q and f16 K/V (got %s/%s/%s)" % (Q.dtype, K.dtype, V.dtype))
    if Q.dtype == "f16":
        # the reference's f16-activation plan (variants *_f16, outputDtype f16): Q widened (exact), the f32-Q
        # kernels, the output narrowed once
        n = seqLen * numHeads * headDim
        if _nbytes(Q) < n * 2:
            raise DopplerHipError("[Attention] Q buffer smaller than [%d, %d, %d] f16" % (seqLen, numHeads, headDim))
        wide = acquireBuffer(n * 4)
        capi.check(_lib().dh_cast_f16_to_f32(_ptr(Q), _ptr(wide), n))
        r = runAttention(Tensor(wide, "f32", Q.shape, "attention_q_f32"), K, V, mask, numHeads, headDim, seqLen=seqLen,
                         kvLen=kvLen, numKVHeads=numKVHeads, scale=scale, causal=causal, startPos=startPos,
                         attnSoftcap=attnSoftcap, slidingWindow=slidingWindow, kvStart=kvStart, kvLayout=kvLayout,
                         workspace=workspace, kvLenBuffer=kvLenBuffer)
        out = _out(outputBuffer, n * 2)
        capi.check(_lib().dh_cast_f32_to_f16(_ptr(r), _ptr(out), n))
        return Tensor(out, "f16", (seqLen, numHeads, headDim), "attention_output")
    layouts = {"contiguous": capi.KV_CONTIGUOUS, "ring": capi.KV_RING}
    if kvLayout not in layouts:
        raise DopplerHipError("[Attention] kvLayout %r is not supported by the HIP path" % (kvLayout,))
    if kvLenBuffer is not None and seqLen > 1:
        raise DopplerHipError("[Attention] kvLenBuffer is served for decode (seqLen 1) only, got seqLen=%d" % seqLen)
    if kvLenBuffer is not None and _nbytes(kvLenBuffer) < 4:
        raise DopplerHipError("[Attention] kvLenBuffer must hold one u32")
    if seqLen > 1:
        if kvLayout != "contiguous" or kvStart != 0:
            raise DopplerHipError("[Attention] prefill (seqLen=%d) needs a contiguous cache with kvStart=0" % seqLen)
        if min(_nbytes(K), _nbytes(V)) < kvLen * numKVHeads * headDim * 2:
            raise DopplerHipError("[Attention] KV buffer smaller than kvLen=%d rows" % kvLen)
        out = _out(outputBuffer, seqLen * numHeads * headDim * 4)
        capi.check(_lib().dh_attn_prefill(_ptr(Q), _ptr(K), _ptr(V), out.data_ptr(), seqLen, numHeads, numKVHeads,
                                          headDim, kvLen, scale, int(bool(causal)), startPos, float(attnSoftcap),
                                          slidingWindow))
        return Tensor(out, "f32", (seqLen, numHeads, headDim), "attention_output")
    rows = slidingWindow if kvLayout == "ring" else kvStart + kvLen
    if kvLen > 0 and min(_nbytes(K), _nbytes(V)) < rows * numKVHeads * headDim * 2:
        raise DopplerHipError("[Attention] KV buffer smaller than kvLen=%d rows" % kvLen)
    padded = padToQ4KBlock(numHeads * headDim)
    out = _out(outputBuffer, seqLen * padded * 4)
    L = _lib()
    if workspace is None:
        workspace = acquireBuffer(attentionWorkspaceBytes(numHeads, headDim, max(kvLen, 1)))
    if kvLenBuffer is not None:
        capi.check(L.dh_attn_decode_kvlen(_ptr(Q), _ptr(K), _ptr(V), out.data_ptr(), numHeads, numKVHeads, headDim,
                                          _ptr(kvLenBuffer), max(kvLen, 1), scale, int(bool(causal)), startPos,
                                          float(attnSoftcap), slidingWindow, kvStart, layouts[kvLayout], _ptr(workspace)))
    else:
        capi.check(L.dh_attn_decode(_ptr(Q), _ptr(K), _ptr(V), out.data_ptr(), numHeads, numKVHeads, headDim, kvLen,
                                    scale, int(bool(causal)), startPos, float(attnSoftcap), slidingWindow, kvStart,
                                    layouts[kvLayout], _ptr(workspace)))
    return Tensor(out, "f32", (seqLen, numHeads, headDim), "attention_output")


# ------------------------------------------------------------------ norm / rope / kv

def runRMSNorm(input, weight, eps, batchSize=1, hiddenSize=None, residual=None, outputBuffer=None,
               rmsNormWeightOffset=False, preResidual=None, residualSumOutput=None, outputScale=None, **_ignored):
    """src/gpu/kernels/rmsnorm.js:146 runRMSNorm."""
    if input.dtype != "f32":
        raise DopplerHipError("[RMSNorm] f32 input required, got %s" % input.dtype)
    hidden = hiddenSize if hiddenSize else input.shape[-1]
    scale = 1.0 if outputScale is None else float(outputScale)
    if not math.isfinite(scale):
        raise DopplerHipError('[RMSNorm] outputScale must be finite; got "%s".' % outputScale)
    wdt = capi.F32
    if weight is not None:
        wd = weight.dtype if isinstance(weight, (Tensor, WeightBuffer)) else "f32"
        wdt = capi.F16 if wd == "f16" else capi.F32
        if _nbytes(weight) < hidden * (2 if wdt == capi.F16 else 4):
            raise DopplerHipError("[RMSNorm] weight buffer smaller than hiddenSize=%d" % hidden)
    out = _out(outputBuffer, batchSize * padToQ4KBlock(hidden) * 4)
    capi.check(_lib().dh_rmsnorm(_ptr(input), _ptr(weight), wdt, out.data_ptr(), batchSize, hidden, eps,
                                 int(bool(rmsNormWeightOffset)), _ptr(preResidual), _ptr(residual),
                                 _ptr(residualSumOutput) if preResidual is not None else None, scale))
    return Tensor(out, "f32", (batchSize, hidden), "rmsnorm_output")


def _norm_weight_dtype(weight, hidden, what):
    wd = weight.dtype if isinstance(weight, (Tensor, WeightBuffer)) else "f32"
    dt = capi.F16 if wd == "f16" else capi.F32
    if _nbytes(weight) < hidden * (2 if dt == capi.F16 else 4):
        raise DopplerHipError("%s weight buffer smaller than hiddenSize=%d" % (what, hidden))
    return dt


def _pair_inputs(tag, input, residual, hiddenSize):
    if input.dtype != "f32":
        raise DopplerHipError('[%s] input dtype must be f32; got "%s".' % (tag, input.dtype))
    if residual is not None and isinstance(residual, Tensor) and residual.dtype != "f32":
        raise DopplerHipError('[%s] residual dtype must be f32; got "%s".' % (tag, residual.dtype))
    hidden = hiddenSize if hiddenSize else input.shape[-1]
    if not isinstance(hidden, (int, np.integer)) or hidden <= 0:
        raise DopplerHipError("[%s] hiddenSize must be a positive integer." % tag)
    return int(hidden)


def runSandwichRMSNormPair(input, residual, postWeight, preWeight, eps, batchSize=1, hiddenSize=None,
                           rmsNormWeightOffset=False, postOutputBuffer=None, preOutputBuffer=None, **_ignored):
    """src/gpu/kernels/rmsnorm-pair.js:147 runSandwichRMSNormPair: postAttn = residual + rmsnorm(input, postWeight),
    ffnInput = rmsnorm(postAttn, preWeight), one launch."""
    hidden = _pair_inputs("rmsnorm_pair", input, residual, hiddenSize)
    pdt = _norm_weight_dtype(postWeight, hidden, "[rmsnorm_pair] post")
    qdt = _norm_weight_dtype(preWeight, hidden, "[rmsnorm_pair] pre")
    nbytes = batchSize * padToQ4KBlock(hidden) * 4
    post, pre = _out(postOutputBuffer, nbytes), _out(preOutputBuffer, nbytes)
    capi.check(_lib().dh_rmsnorm_sandwich_pair(_ptr(input), _ptr(residual), _ptr(postWeight), pdt, _ptr(preWeight), qdt,
                                               post.data_ptr(), pre.data_ptr(), batchSize, hidden, eps,
                                               int(bool(rmsNormWeightOffset))))
    return {"postAttn": Tensor(post, "f32", (batchSize, hidden), "rmsnorm_pair_post_output"),
            "ffnInput": Tensor(pre, "f32", (batchSize, hidden), "rmsnorm_pair_pre_output")}


def runResidualNextRMSNormPair(input, residual, normWeight, eps, batchSize=1, hiddenSize=None, rmsNormWeightOffset=False,
                               residualOutputBuffer=None, normOutputBuffer=None, outputScale=1, **_ignored):
    """src/gpu/kernels/rmsnorm-pair.js:246 runResidualNextRMSNormPair: residual = (input + residual) * outputScale,
    nextInput = rmsnorm(residual, normWeight), one launch."""
    hidden = _pair_inputs("rmsnorm_pair", input, residual, hiddenSize)
    if residual is None:
        raise DopplerHipError("[residual_rmsnorm_pair] a residual tensor is required.")
    scale = float(outputScale)
    if not math.isfinite(scale):
        raise DopplerHipError('[residual_rmsnorm_pair] outputScale must be finite; got "%s".' % outputScale)
    wdt = _norm_weight_dtype(normWeight, hidden, "[residual_rmsnorm_pair] norm")
    nbytes = batchSize * padToQ4KBlock(hidden) * 4
    res, nrm = _out(residualOutputBuffer, nbytes), _out(normOutputBuffer, nbytes)
    capi.check(_lib().dh_residual_rmsnorm_pair(_ptr(input), _ptr(residual), _ptr(normWeight), wdt, res.data_ptr(),
                                               nrm.data_ptr(), batchSize, hidden, eps, int(bool(rmsNormWeightOffset)), scale))
    return {"residual": Tensor(res, "f32", (batchSize, hidden), "residual_rmsnorm_pair_residual_output"),
            "nextInput": Tensor(nrm, "f32", (batchSize, hidden), "residual_rmsnorm_pair_norm_output")}


def canUseRMSNormQK(qTensor, kTensor, skipKNorm=False):
    """src/gpu/kernels/rmsnorm-qk.js:29 canUseRMSNormQK (f32 tensors on this path)."""
    if skipKNorm or qTensor is None or kTensor is None or qTensor.buffer is kTensor.buffer:
        return False
    return qTensor.dtype == kTensor.dtype == "f32"


def runRMSNormQK(qTensor, kTensor, qWeight, kWeight, eps, numTokens=None, numHeads=None, numKVHeads=None,
                 headDim=None, rmsNormWeightOffset=False, **_ignored):
    """src/gpu/kernels/rmsnorm-qk.js:122 runRMSNormQK: per-head RMSNorm of q and k in one launch; returns
    {"q": Tensor [numTokens*numHeads, headDim], "k": Tensor [numTokens*numKVHeads, headDim]}."""
    for name, v in (("numTokens", numTokens), ("numHeads", numHeads), ("numKVHeads", numKVHeads), ("headDim", headDim)):
        if not isinstance(v, (int, np.integer)) or v <= 0:
            raise DopplerHipError("RMSNorm QK requires a positive integer %s, got %r." % (name, v))
    if qTensor.dtype != kTensor.dtype:
        raise DopplerHipError("RMSNorm QK requires matching Q/K dtypes, got %s and %s." % (qTensor.dtype, kTensor.dtype))
    if qTensor.dtype != "f32":
        raise DopplerHipError("RMSNorm QK: the HIP path takes f32 tensors, got %s." % qTensor.dtype)
    q_rows, k_rows = numTokens * numHeads, numTokens * numKVHeads
    if _nbytes(qTensor) < q_rows * headDim * 4:
        raise DopplerHipError("RMSNorm QK: Q input buffer smaller than %d bytes" % (q_rows * headDim * 4))
    if _nbytes(kTensor) < k_rows * headDim * 4:
        raise DopplerHipError("RMSNorm QK: K input buffer smaller than %d bytes" % (k_rows * headDim * 4))
    dts = []
    for name, w in (("q", qWeight), ("k", kWeight)):
        wd = w.dtype if isinstance(w, (Tensor, WeightBuffer)) else "f32"
        dt = capi.F16 if wd == "f16" else capi.F32
        if _nbytes(w) < headDim * (2 if dt == capi.F16 else 4):
            raise DopplerHipError("RMSNorm QK: %s weight buffer smaller than headDim=%d" % (name, headDim))
        dts.append(dt)
    q_out = _out(None, q_rows * padToQ4KBlock(headDim) * 4)
    k_out = _out(None, k_rows * padToQ4KBlock(headDim) * 4)
    capi.check(_lib().dh_rmsnorm_qk(_ptr(qTensor), _ptr(kTensor), _ptr(qWeight), dts[0], _ptr(kWeight), dts[1],
                                    q_out.data_ptr(), k_out.data_ptr(), q_rows, k_rows, headDim, eps,
                                    int(bool(rmsNormWeightOffset))))
    return {"q": Tensor(q_out, "f32", (q_rows, headDim), "rmsnorm_qk_q_output"),
            "k": Tensor(k_out, "f32", (k_rows, headDim), "rmsnorm_qk_k_output")}


def runRoPE(input, freqsCos, freqsSin, seqLen, numHeads=1, headDim=64, rotaryDim=None, pairSpanDim=None,
            interleaved=False, startPos=0, **_ignored):
    """src/gpu/kernels/rope.js:108 runRoPE: in place, returns a Tensor aliasing the input."""
    rotaryDim = headDim if rotaryDim is None else rotaryDim
    pairSpanDim = rotaryDim if pairSpanDim is None else pairSpanDim
    if input.dtype not in ("f32", "f16"):
        raise DopplerHipError("[RoPE] f32 or f16 input required, got %s" % input.dtype)
    need = (startPos + seqLen) * (rotaryDim // 2) * 4
    if min(_nbytes(freqsCos), _nbytes(freqsSin)) < need:
        raise DopplerHipError("[RoPE] cos/sin tables smaller than %d bytes" % need)
    L = _lib()
    target = input
    if input.dtype == "f16":
        # the reference's route for a device without the f16 kernel (rope.js:44-63,89-107): widen, rotate in
        # f32, narrow back into the input buffer
        n = seqLen * numHeads * headDim
        if _nbytes(input) < n * 2:
            raise DopplerHipError("[RoPE] input buffer smaller than [%d, %d, %d] f16" % (seqLen, numHeads, headDim))
        target = acquireBuffer(n * 4)
        capi.check(L.dh_cast_f16_to_f32(_ptr(input), _ptr(target), n))
    capi.check(L.dh_rope(_ptr(target), _ptr(freqsCos), _ptr(freqsSin), seqLen, numHeads, headDim, rotaryDim,
                         pairSpanDim, int(bool(interleaved)), startPos))
    if input.dtype == "f16":
        capi.check(L.dh_cast_f32_to_f16(_ptr(target), _ptr(input), seqLen * numHeads * headDim))
    return Tensor(input.buffer, input.dtype, input.shape, "rope_output")


def canUseRoPEQK(qTensor, kTensor, reusesSharedKV=False, **_ignored):
    """src/gpu/kernels/rope-qk.js:56-64 canUseRoPEQK (the HIP kernel rotates f32 activations only)."""
    if reusesSharedKV or qTensor is None or kTensor is None or qTensor.buffer is kTensor.buffer:
        return False
    return qTensor.dtype == "f32" and kTensor.dtype == "f32"


def runRoPEQK(qTensor, kTensor, freqsCos, freqsSin, seqLen, numQHeads=None, numKVHeads=None, headDim=None,
              rotaryDim=None, pairSpanDim=None, interleaved=False, startPos=0, **_ignored):
    """src/gpu/kernels/rope-qk.js:136 runRoPEQK: q and k rotated in place by one launch; returns Tensors
    aliasing the inputs."""
    rotaryDim = headDim if rotaryDim is None else rotaryDim
    pairSpanDim = rotaryDim if pairSpanDim is None else pairSpanDim
    for label, v, low, kind in (("seqLen", seqLen, 0, "non-negative"), ("startPos", startPos, 0, "non-negative"),
                                ("numQHeads", numQHeads, 1, "positive"), ("numKVHeads", numKVHeads, 1, "positive"),
                                ("headDim", headDim, 1, "positive"), ("rotaryDim", rotaryDim, 1, "positive"),
                                ("pairSpanDim", pairSpanDim, 1, "positive")):
        if not isinstance(v, (int, np.integer)) or isinstance(v, bool) or v < low:
            raise DopplerHipError("RoPE QK requires %s to be a %s integer." % (label, kind))
    if qTensor.dtype != kTensor.dtype:
        raise DopplerHipError("RoPE QK requires matching Q/K dtypes, got %s and %s." % (qTensor.dtype, kTensor.dtype))
    if qTensor.dtype != "f32":
        raise DopplerHipError("RoPE QK on the HIP path takes f32 tensors, got %s." % qTensor.dtype)
    result = {"q": Tensor(qTensor.buffer, qTensor.dtype, qTensor.shape, "rope_q_output"),
              "k": Tensor(kTensor.buffer, kTensor.dtype, kTensor.shape, "rope_k_output")}
    if seqLen == 0:
        return result
    table = (startPos + seqLen) * (rotaryDim // 2) * 4
    for buf, need, label in ((qTensor, seqLen * numQHeads * headDim * 4, "Q input"),
                             (kTensor, seqLen * numKVHeads * headDim * 4, "K input"),
                             (freqsCos, table, "cos frequencies"), (freqsSin, table, "sin frequencies")):
        if need > _nbytes(buf):
            raise DopplerHipError("RoPE QK %s buffer is smaller than requested range (%d > %d bytes)."
                                  % (label, need, _nbytes(buf)))
    capi.check(_lib().dh_rope_qk(_ptr(qTensor), _ptr(kTensor), _ptr(freqsCos), _ptr(freqsSin), seqLen, numQHeads,
                                 numKVHeads, headDim, rotaryDim, pairSpanDim, int(bool(interleaved)), startPos))
    return result


def runKVCacheWriteF32ToF16(keys, values, outputKeys, outputValues, srcOffset=0, dstOffset=0, elementCount=None):
    """src/gpu/kernels/kv-cache-write.js:107 runKVCacheWriteF32ToF16."""
    for name, v in (("srcOffset", srcOffset), ("dstOffset", dstOffset), ("elementCount", elementCount)):
        if not isinstance(v, (int, np.integer)) or v < 0:
            raise DopplerHipError("KV cache write %s must be a non-negative integer, got %s." % (name, v))
    if elementCount == 0:
        return
    for buf, off, bpe, label in ((keys, srcOffset, 4, "keys input"), (values, srcOffset, 4, "values input"),
                                 (outputKeys, dstOffset, 2, "keys output"), (outputValues, dstOffset, 2, "values output")):
        if (off + elementCount) * bpe > _nbytes(buf):
            raise DopplerHipError("KV cache write %s buffer is smaller than requested range (%d > %d bytes)."
                                  % (label, (off + elementCount) * bpe, _nbytes(buf)))
    capi.check(_lib().dh_kv_write_f16(_ptr(keys), _ptr(values), _ptr(outputKeys), _ptr(outputValues), srcOffset,
                                      dstOffset, elementCount))


def runSplitQKVRMSNormRoPEQK(qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, numTokens=None, numHeads=None,
                             numKVHeads=None, headDim=None, qSize=None, kSize=None, vSize=None, startPos=0,
                             rotaryDim=None, interleaved=False, rmsNormWeightOffset=False, f16KVCacheWrite=None,
                             **_ignored):
    """src/gpu/kernels/split-qkv-rmsnorm-rope-qk.js:244 with f16KVCacheWrite = {keysBuffer,
    valuesBuffer, dstOffset}: returns {Q, K: None, V: None, wroteF16KVCache: True}."""
    rotaryDim = headDim if rotaryDim is None else rotaryDim
    for name, v in (("numTokens", numTokens), ("numHeads", numHeads), ("numKVHeads", numKVHeads), ("headDim", headDim),
                    ("qSize", qSize), ("kSize", kSize), ("vSize", vSize)):
        if not isinstance(v, (int, np.integer)) or v <= 0:
            raise DopplerHipError("split_qkv_rmsnorm_rope_qk %s must be a positive integer, got %s." % (name, v))
    if qSize != numHeads * headDim or kSize != numKVHeads * headDim or vSize != kSize:
        raise DopplerHipError("split_qkv_rmsnorm_rope_qk sizes do not match heads*headDim")
    if qkvTensor.dtype != "f32":
        raise DopplerHipError("split_qkv_rmsnorm_rope_qk requires f32 QKV input, got %s." % qkvTensor.dtype)
    if f16KVCacheWrite is None:
        raise DopplerHipError("split_qkv_rmsnorm_rope_qk: the HIP path writes K/V to the f16 cache (f16KVCacheWrite is required)")
    dst = f16KVCacheWrite["dstOffset"]
    need = (dst + numTokens * numKVHeads * headDim) * 2
    if _nbytes(f16KVCacheWrite["keysBuffer"]) < need or _nbytes(f16KVCacheWrite["valuesBuffer"]) < need:
        raise DopplerHipError("split_qkv_rmsnorm_rope_qk f16 KV cache is smaller than %d bytes" % need)
    qRows = numTokens * numHeads
    q_out = acquireBuffer(qRows * padToQ4KBlock(headDim) * 4)
    capi.check(_lib().dh_qkv_norm_rope_kvwrite(_ptr(qkvTensor), _ptr(qWeight), _ptr(kWeight), _ptr(freqsCos),
                                               _ptr(freqsSin), q_out.data_ptr(), _ptr(f16KVCacheWrite["keysBuffer"]),
                                               _ptr(f16KVCacheWrite["valuesBuffer"]), numTokens, numHeads, numKVHeads,
                                               headDim, startPos, rotaryDim, int(bool(interleaved)), eps,
                                               int(bool(rmsNormWeightOffset)), dst, 1))
    return dict(Q=Tensor(q_out, "f32", (qRows, headDim), "split_qkv_rmsnorm_rope_qk_q_output"), K=None, V=None,
                wroteF16KVCache=True)


def decodeAttentionFromQKVSupported(numHeads, numKVHeads, headDim, rotaryDim=None, interleaved=False):
    rotaryDim = headDim if rotaryDim is None else rotaryDim
    return bool(_lib().dh_attn_decode_qkv_supported(numHeads, numKVHeads, headDim, rotaryDim, int(bool(interleaved))))


def runDecodeAttentionFromQKV(qkvTensor, qWeight, kWeight, freqsCos, freqsSin, eps, keysBuffer, valuesBuffer, numHeads,
                              numKVHeads, headDim, startPos, rotaryDim=None, interleaved=False,
                              rmsNormWeightOffset=False, useNorm=True, scale=None, attnSoftcap=0, slidingWindow=0,
                              kvStart=0, kvLayout="contiguous", outputBuffer=None, workspace=None, **_ignored):
    """One decode step of runSplitQKVRMSNormRoPEQK (f16KVCacheWrite at the row of startPos,
    src/gpu/kernels/split-qkv-rmsnorm-rope-qk.js:244) followed by runAttention with seqLen == 1
    (src/gpu/kernels/attention.js:2007) in one launch: the new key/value are appended to the cache
    and the token attends to rows up to and including its own."""
    rotaryDim = headDim if rotaryDim is None else rotaryDim
    scale = 1.0 / math.sqrt(headDim) if scale is None else scale
    if qkvTensor.dtype != "f32":
        raise DopplerHipError("[Attention] fused decode requires f32 QKV input, got %s." % qkvTensor.dtype)
    layouts = {"contiguous": capi.KV_CONTIGUOUS, "ring": capi.KV_RING}
    if kvLayout not in layouts:
        raise DopplerHipError("[Attention] kvLayout %r is not supported by the HIP path" % (kvLayout,))
    if _nbytes(qkvTensor) < (numHeads + 2 * numKVHeads) * headDim * 4:
        raise DopplerHipError("[Attention] fused decode: qkv tensor smaller than (H + 2 Hkv) * headDim floats")
    rows = slidingWindow if kvLayout == "ring" else startPos + 1
    if min(_nbytes(keysBuffer), _nbytes(valuesBuffer)) < rows * numKVHeads * headDim * 2:
        raise DopplerHipError("[Attention] KV buffer smaller than %d rows" % rows)
    if min(_nbytes(freqsCos), _nbytes(freqsSin)) < (startPos + 1) * (rotaryDim // 2) * 4:
        raise DopplerHipError("[Attention] rotary tables end before position %d" % startPos)
    out = _out(outputBuffer, padToQ4KBlock(numHeads * headDim) * 4)
    if workspace is None:
        workspace = acquireBuffer(attentionWorkspaceBytes(numHeads, headDim, max(startPos - kvStart + 1, 1)))
    capi.check(_lib().dh_attn_decode_qkv(_ptr(qkvTensor), _ptr(qWeight) if useNorm else None,
                                         _ptr(kWeight) if useNorm else None, _ptr(freqsCos), _ptr(freqsSin),
                                         _ptr(keysBuffer), _ptr(valuesBuffer), out.data_ptr(), numHeads, numKVHeads,
                                         headDim, startPos, rotaryDim, int(bool(interleaved)), eps,
                                         int(bool(rmsNormWeightOffset)), int(bool(useNorm)), scale,
                                         float(attnSoftcap), slidingWindow, kvStart, layouts[kvLayout],
                                         _ptr(workspace)))
    return Tensor(out, "f32", (1, numHeads, headDim), "attention_output")


# ------------------------------------------------------------------ elementwise

def runResidualAdd(a, b, size, outputBuffer=None, outputScale=None, **_ignored):
    """src/gpu/kernels/residual.js:210 runResidualAdd: (a + b) * outputScale."""
    scale = 1.0 if outputScale is None else float(outputScale)
    if not math.isfinite(scale):
        raise DopplerHipError('[Residual] outputScale must be finite; got "%s".' % outputScale)
    out = _out(outputBuffer, size * 4)
    capi.check(_lib().dh_residual_add(_ptr(a), _ptr(b), out.data_ptr(), size, scale))
    return Tensor(out, "f32", (size,), "residual_output")


def runSplitQKV(qkvTensor, numTokens=None, qSize=None, kSize=None, vSize=None, qTensor=None, kTensor=None,
                vTensor=None, **_ignored):
    """src/gpu/kernels/split_qkv.js:40 runSplitQKV: the stacked projection copied apart into Q, K, V (new buffers
    unless the caller passes tensors to fill)."""
    if qkvTensor.dtype != "f32":
        raise DopplerHipError("[SplitQKV] the HIP path takes f32 tensors, got %s." % qkvTensor.dtype)
    if numTokens * (qSize + kSize + vSize) * 4 > _nbytes(qkvTensor):
        raise DopplerHipError("[SplitQKV] qkv buffer is smaller than numTokens=%d x %d elements."
                              % (numTokens, qSize + kSize + vSize))
    outs = []
    for given, size, name in ((qTensor, qSize, "Q"), (kTensor, kSize, "K"), (vTensor, vSize, "V")):
        if given is not None and _nbytes(given) < numTokens * size * 4:
            raise DopplerHipError("[SplitQKV] %s tensor is smaller than numTokens=%d x %d elements." % (name, numTokens, size))
        outs.append(given if given is not None else Tensor(_out(None, numTokens * size * 4), "f32", (numTokens, size), name))
    capi.check(_lib().dh_split_qkv(_ptr(qkvTensor), _ptr(outs[0]), _ptr(outs[1]), _ptr(outs[2]), numTokens, qSize,
                                   kSize, vSize))
    return {"Q": outs[0], "K": outs[1], "V": outs[2]}


def runBiasAdd(data, bias, numTokens, dim, dataOffset=0, biasOffset=0, **_ignored):
    """src/gpu/kernels/residual.js:218 runBiasAdd: data[t, :] += bias in place (offsets in bytes); the returned
    Tensor aliases data.  The bias may be f32 or f16 and is widened on the fly."""
    if data.dtype != "f32":
        raise DopplerHipError("[BiasAdd] the HIP path takes f32 data, got %s." % data.dtype)
    bias_dtype = getattr(bias, "dtype", "f32")
    if bias_dtype not in ("f32", "f16"):
        raise DopplerHipError("[BiasAdd] bias dtype must be f32 or f16, got %s." % bias_dtype)
    if dataOffset + numTokens * dim * 4 > _nbytes(data):
        raise DopplerHipError("[BiasAdd] data buffer is smaller than numTokens=%d x dim=%d at offset %d."
                              % (numTokens, dim, dataOffset))
    if biasOffset + dim * (2 if bias_dtype == "f16" else 4) > _nbytes(bias):
        raise DopplerHipError("[BiasAdd] bias buffer is smaller than dim=%d at offset %d." % (dim, biasOffset))
    capi.check(_lib().dh_bias_add(_ptr(data), _ptr(bias), capi.F16 if bias_dtype == "f16" else capi.F32, numTokens, dim, dataOffset, biasOffset))
    return Tensor(data.buffer, data.dtype, (numTokens, dim), "bias_add_output")


def runScale(input, scale, count=None, outputBuffer=None, inplace=False, **_ignored):
    """src/gpu/kernels/scale.js:44 runScale: out = input * scale, into a new buffer, outputBuffer or in place."""
    if input.dtype != "f32":
        raise DopplerHipError("[Scale] the HIP path takes f32 tensors, got %s." % input.dtype)
    n = _nbytes(input) // 4 if count is None else count
    if n * 4 > _nbytes(input):
        raise DopplerHipError("[Scale] count=%d exceeds the input buffer." % n)
    out = input.buffer if inplace else _out(outputBuffer, n * 4)
    capi.check(_lib().dh_scale(_ptr(input), _ptr(out), n, float(scale)))
    return Tensor(out, input.dtype, input.shape, "scale_output")


def runGather(indices, embeddings, numTokens, hiddenSize, vocabSize, outputBuffer=None, embeddingDtype=None,
              outputDtype=None, transpose=False, indexOffset=0, **_ignored):
    """src/gpu/kernels/gather.js:370 runGather for f16 tables -> f32 rows, or (outputDtype 'f16', the
    reference's f16-activation plan) the stored bits of the rows."""
    if embeddingDtype is None:
        raise DopplerHipError("[Gather] embeddingDtype is required.")
    if outputDtype is None:
        raise DopplerHipError("[Gather] outputDtype is required.")
    if embeddingDtype != "f16" or outputDtype not in ("f32", "f16") or transpose:
        raise DopplerHipError('[Gather] unsupported embeddingDtype="%s" / outputDtype="%s" on the HIP path.' % (embeddingDtype, outputDtype))
    narrow = outputDtype == "f16"
    out = _out(outputBuffer, numTokens * padToQ4KBlock(hiddenSize) * (2 if narrow else 4))
    wide = acquireBuffer(numTokens * hiddenSize * 4) if narrow else out
    capi.check(_lib().dh_gather_f16(_ptr(indices), _ptr(embeddings), wide.data_ptr(), numTokens, hiddenSize, vocabSize,
                                    indexOffset))
    if narrow:
        capi.check(_lib().dh_cast_f32_to_f16(wide.data_ptr(), out.data_ptr(), numTokens * hiddenSize))   # exact
    return Tensor(out, outputDtype, (numTokens, hiddenSize), "gather_output")


def runSiLU(input, size=None, gate=None, outputBuffer=None, swigluLimit=None, **_ignored):
    """src/gpu/kernels/silu.js:95 runSiLU with `gate`: silu(gate) * input."""
    if gate is None:
        raise DopplerHipError("[SiLU] the HIP path implements the gated form only (options.gate)")
    n = size or _nbytes(input) // 4
    out = _out(outputBuffer, n * 4)
    capi.check(_lib().dh_act_gate(_ptr(gate), _ptr(input), out.data_ptr(), n, capi.ACT_SILU, float(swigluLimit or 0.0)))
    return Tensor(out, "f32", (n,), "silu_output")


def runGeLU(input, size=None, gate=None, outputBuffer=None, **_ignored):
    """src/gpu/kernels/gelu.js:49 runGeLU with `gate`: gelu_tanh(gate) * input."""
    if gate is None:
        raise DopplerHipError("[GeLU] the HIP path implements the gated form only (options.gate)")
    n = size or _nbytes(input) // 4
    out = _out(outputBuffer, n * 4)
    capi.check(_lib().dh_act_gate(_ptr(gate), _ptr(input), out.data_ptr(), n, capi.ACT_GELU, 0.0))
    return Tensor(out, "f32", (n,), "gelu_output")


def runSiLURowSplit(input, numTokens=None, dim=None, activation="silu", outputBuffer=None, swigluLimit=None):
    """src/gpu/kernels/silu.js:230 runSiLURowSplit: [T, 2*dim] -> act(gate) * up."""
    out = _out(outputBuffer, numTokens * dim * 4)
    code = _act_code(activation, "SiLU row-split")
    capi.check(_lib().dh_act_gate_rowsplit(_ptr(input), out.data_ptr(), numTokens, dim, code,
                                           float(swigluLimit or 0.0) if activation == "silu" else 0.0))
    return Tensor(out, "f32", (numTokens, dim), "silu_rowsplit_output")


def runArgmax(logits, vocabSize, padTokenId=None, logitSoftcap=0.0, logitsDtype="f32", outputBuffer=None,
              outputIndex=0, readback=True):
    """src/gpu/kernels/sample.js:334 runArgmax: returns the token id (reads it back)."""
    if logitsDtype != "f32":
        raise DopplerHipError("[Argmax] logitsDtype %r is not supported on the HIP path" % (logitsDtype,))
    L = _lib()
    ws = acquireBuffer(int(L.dh_argmax_workspace_bytes()))
    out = _out(outputBuffer, max(4, (outputIndex + 1) * 4))
    capi.check(L.dh_argmax(_ptr(logits), vocabSize, -1 if padTokenId is None else padTokenId, logitSoftcap,
                           ws.data_ptr(), out.data_ptr(), outputIndex))
    if not readback:
        return out
    return int(readBuffer(out, (outputIndex + 1) * 4, np.uint32)[outputIndex])


def seededRandom(seed):
    """src/gpu/kernels/sample.js:569-572: the reference's Math.sin based uniform number."""
    x = math.sin(seed) * 10000.0
    return x - math.floor(x)


def runGPUSample(logits, vocabSize, temperature=1.0, topK=40, randomSeed=None, randomValue=None, padTokenId=None,
                 logitSoftcap=0.0, greedyThreshold=0.01, logitsDtype="f32", outputBuffer=None, outputIndex=0,
                 readback=True):
    """src/gpu/kernels/sample.js:343 runGPUSample: top-k temperature sampling; below the greedy
    threshold or with topK <= 1 it is runArgmax.  randomValue overrides the seeded draw."""
    if logitsDtype != "f32":
        raise DopplerHipError("[Sample] logitsDtype %r is not supported on the HIP path" % (logitsDtype,))
    if temperature < greedyThreshold or topK <= 1:
        return runArgmax(logits, vocabSize, padTokenId=padTokenId, logitSoftcap=logitSoftcap, outputBuffer=outputBuffer,
                         outputIndex=outputIndex, readback=readback)
    if randomValue is None:
        if randomSeed is None:
            raise DopplerHipError("[Sample] randomSeed (or randomValue) is required on the HIP path")
        randomValue = seededRandom(randomSeed)
    L = _lib()
    ws = acquireBuffer(int(L.dh_sample_topk_workspace_bytes(vocabSize, topK)))
    out = _out(outputBuffer, max(4, (outputIndex + 1) * 4))
    capi.check(L.dh_sample_topk(_ptr(logits), vocabSize, float(temperature), int(topK), float(randomValue),
                                -1 if padTokenId is None else padTokenId, logitSoftcap, ws.data_ptr(), out.data_ptr(),
                                outputIndex))
    if not readback:
        return out
    return int(readBuffer(out, (outputIndex + 1) * 4, np.uint32)[outputIndex])


def lmHeadArgmaxNormFusable(hiddenSize):
    """Whether recordLmHeadArgmaxF16 takes `normWeight` for this hidden size (the row must fit the registers
    of the LM head kernel)."""
    return 0 < hiddenSize <= 4096 and hiddenSize % 8 == 0


def recordLmHeadArgmaxF16(recorder, inputTensor, lmHead, vocabSize=None, hiddenSize=None, padTokenId=None,
                          logitSoftcap=0.0, outputBuffer=None, outputIndex=0, logitsOutput=None, normWeight=None,
                          rmsNormEps=None, rmsNormWeightOffset=False):
    """src/gpu/kernels/lm-head-argmax.js:304 recordLmHeadArgmaxF16: returns the output buffer
    (token at outputIndex).  `recorder` is accepted for signature parity and unused: every op
    already enqueues in order on one stream.  Beyond the reference's options: `normWeight` (f32 tensor
    [hiddenSize]) with `rmsNormEps` applies the final RMSNorm of recordLogitsGPU
    (src/inference/pipelines/text/logits/gpu.js:1122-1157) to the row inside the same kernel."""
    if inputTensor.dtype != "f32":
        raise DopplerHipError('[LmHeadArgmax] input tensor must be f32, got "%s".' % inputTensor.dtype)
    L = _lib()
    ws = acquireBuffer(int(L.dh_lmhead_argmax_workspace_bytes(vocabSize)))
    out = _out(outputBuffer, max(4, (outputIndex + 1) * 4))
    pad = -1 if padTokenId is None else padTokenId
    if normWeight is not None:
        if rmsNormEps is None:
            raise DopplerHipError("[LmHeadArgmax] rmsNormEps is required with normWeight.")
        if getattr(normWeight, "dtype", "f32") != "f32" or _nbytes(normWeight) < hiddenSize * 4:
            raise DopplerHipError("[LmHeadArgmax] normWeight must be an f32 tensor of %d values." % hiddenSize)
        capi.check(L.dh_lmhead_argmax_f16_rmsnorm(_ptr(inputTensor), _ptr(normWeight), float(rmsNormEps),
                                                  1 if rmsNormWeightOffset else 0, _ptr(lmHead), vocabSize, hiddenSize,
                                                  pad, logitSoftcap, ws.data_ptr(), out.data_ptr(), outputIndex,
                                                  _ptr(logitsOutput)))
        return out
    capi.check(L.dh_lmhead_argmax_f16(_ptr(inputTensor), _ptr(lmHead), vocabSize, hiddenSize, pad, logitSoftcap,
                                      ws.data_ptr(), out.data_ptr(), outputIndex, _ptr(logitsOutput)))
    return out


def sync():
    capi.check(_lib().dh_sync())
