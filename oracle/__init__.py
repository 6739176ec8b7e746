"""numpy front end of the CPU oracle (oracle/doppler_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py.  Product code (doppler_amd/) never imports this package.

Every function takes and returns numpy arrays; shapes and dtypes are checked here so a
wrong call fails in Python rather than inside C.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libdoppler_oracle.so")

QK_K = 256
Q4K_BLOCK_BYTES = 144


def build(force=False):
    """Compile the C restatement with the Makefile next to it."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "--no-print-directory"], check=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _declare(_lib)
        _lib.dor_init_tables()
    return _lib


_P = ctypes.c_void_p
_I64 = ctypes.c_int64
_F = ctypes.c_float
_D = ctypes.c_double
_I = ctypes.c_int


class ModelCfg(ctypes.Structure):
    _fields_ = [(n, _I64) for n in ("layers", "hidden", "inter", "heads", "kv_heads",
                                    "head_dim", "vocab", "max_seq")] + [("eps", _F), ("qk_norm", _I)]


class Layer(ctypes.Structure):
    _fields_ = [(n, _P) for n in ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown",
                                  "input_norm", "post_attn_norm", "q_norm", "k_norm",
                                  "cache_k", "cache_v")]


def _declare(L):
    L.dor_f16_to_f32.restype = _F
    L.dor_f16_to_f32.argtypes = [ctypes.c_uint16]
    for name in ("dor_f32_to_f16_rne", "dor_f32_to_f16_half_up", "dor_f32_to_f16_trunc"):
        getattr(L, name).restype = ctypes.c_uint16
        getattr(L, name).argtypes = [_F]
    L.dor_f16_to_f32_array.argtypes = [_P, _P, _I64]
    L.dor_f32_to_f16_rne_array.argtypes = [_P, _P, _I64]
    L.dor_q4k_unpack_scale_bits.argtypes = [_P, _P, _P]
    L.dor_q4k_dequant_blocks.argtypes = [_P, _I64, _P]
    L.dor_q4k_dequant_blocks_fast.argtypes = [_P, _I64, _P]
    L.dor_q4k_decoded_scales.argtypes = [_P, _I64, _P, _P]
    L.dor_q4k_dequant_rows.argtypes = [_P, _I64, _I64, _P]
    L.dor_q4k_matmul.argtypes = [_P, _P, _I64, _I64, _I64, _F, _P]
    L.dor_f16w_matmul.argtypes = [_P, _P, _I64, _I64, _I64, _F, _P]
    L.dor_q4k_ffn_gate_up.argtypes = [_P, _P, _P, _I64, _I64, _I64, _F, _I, _F, _P]
    L.dor_act_gate.argtypes = [_P, _P, _I64, _I, _F, _P]
    L.dor_act_gate_rowsplit.argtypes = [_P, _I64, _I64, _I, _F, _P]
    L.dor_residual_add.argtypes = [_P, _P, _I64, _F, _P]
    L.dor_rmsnorm.argtypes = [_P, _P, _I64, _I64, _F, _I, _P, _P, _P, _F, _P]
    L.dor_rope_tables.argtypes = [_I64, _I64, _D, _I, _D, _P, _P]
    L.dor_rope_apply.argtypes = [_P, _P, _P, _I64, _I64, _I64, _I64, _I64, _I64, _I, _P]
    L.dor_attention_ref.argtypes = [_P, _P, _P, _I64, _I64, _I64, _I64, _I64, _P, _F, _P]
    L.dor_attention_decode_f16kv.argtypes = [_P, _P, _P, _I64, _I64, _I64, _I64, _F, _I, _I64,
                                             _F, _I64, _I64, _I, _P]
    L.dor_kv_write_f16.argtypes = [_P, _P, _I64, _I64, _I64, _P, _P]
    L.dor_qkv_norm_rope_kvwrite.argtypes = [_P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64,
                                            _I64, _I, _F, _I, _I64, _P, _P, _P]
    L.dor_gather_f16.argtypes = [_P, _P, _I64, _I64, _I64, _P]
    L.dor_argmax.restype = _I64
    L.dor_argmax.argtypes = [_P, _I64, _I64, _F]
    L.dor_sample_topk.restype = _I64
    L.dor_sample_topk.argtypes = [_P, _I64, ctypes.c_double, _I64, ctypes.c_double, _I64, _F]
    L.dor_seeded_random.restype = ctypes.c_double
    L.dor_seeded_random.argtypes = [ctypes.c_double]
    L.dor_decode_step.restype = _I64
    L.dor_decode_step.argtypes = [_P, _P, _P, _P, _P, _P, ctypes.c_uint32, _I64, _P]


def _c(a, dtype):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _ptr(a):
    return a.ctypes.data_as(_P) if a is not None else None


# --------------------------------------------------------------------------- f16

def f16_bits_to_f32(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, np.float32)
    lib().dor_f16_to_f32_array(_ptr(bits), _ptr(out), bits.size)
    return out


def f32_to_f16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().dor_f32_to_f16_rne_array(_ptr(x), _ptr(out), x.size)
    return out


# --------------------------------------------------------------------------- Q4_K

def q4k_row_blocks(K):
    return (K + QK_K - 1) // QK_K


def q4k_bytes(N, K):
    return N * q4k_row_blocks(K) * Q4K_BLOCK_BYTES


def q4k_unpack_scale_bits(block):
    block = _c(block, np.uint8)
    assert block.size >= 16
    sc = np.empty(8, np.uint8)
    mn = np.empty(8, np.uint8)
    lib().dor_q4k_unpack_scale_bits(_ptr(block), _ptr(sc), _ptr(mn))
    return sc, mn


def q4k_dequant_blocks(packed):
    packed = _c(packed, np.uint8).reshape(-1)
    assert packed.size % Q4K_BLOCK_BYTES == 0
    nb = packed.size // Q4K_BLOCK_BYTES
    out = np.empty(nb * QK_K, np.float32)
    lib().dor_q4k_dequant_blocks(_ptr(packed), nb, _ptr(out))
    return out


def q4k_dequant_blocks_fast(packed):
    """f32-arithmetic twin used inside the matmul loops; must equal q4k_dequant_blocks bit for bit."""
    packed = _c(packed, np.uint8).reshape(-1)
    nb = packed.size // Q4K_BLOCK_BYTES
    out = np.empty(nb * QK_K, np.float32)
    lib().dor_q4k_dequant_blocks_fast(_ptr(packed), nb, _ptr(out))
    return out


def q4k_decoded_scales(packed):
    packed = _c(packed, np.uint8).reshape(-1)
    nb = packed.size // Q4K_BLOCK_BYTES
    sc = np.empty(nb * 8, np.float32)
    mn = np.empty(nb * 8, np.float32)
    lib().dor_q4k_decoded_scales(_ptr(packed), nb, _ptr(sc), _ptr(mn))
    return sc, mn


def q4k_dequant_rows(packed, N, K):
    packed = _c(packed, np.uint8).reshape(-1)
    assert packed.size == q4k_bytes(N, K), (packed.size, N, K)
    out = np.empty((N, K), np.float32)
    lib().dor_q4k_dequant_rows(_ptr(packed), N, K, _ptr(out))
    return out


def q4k_matmul(A, W, M, N, K, alpha=1.0):
    A = _c(A, np.float32).reshape(M, K)
    W = _c(W, np.uint8).reshape(-1)
    assert W.size == q4k_bytes(N, K), (W.size, N, K)
    C = np.empty((M, N), np.float32)
    lib().dor_q4k_matmul(_ptr(A), _ptr(W), M, N, K, alpha, _ptr(C))
    return C


def f16w_matmul(A, W_bits, M, N, K, alpha=1.0):
    A = _c(A, np.float32).reshape(M, K)
    W = _c(W_bits, np.uint16).reshape(N, K)
    C = np.empty((M, N), np.float32)
    lib().dor_f16w_matmul(_ptr(A), _ptr(W), M, N, K, alpha, _ptr(C))
    return C


def q4k_ffn_gate_up(X, Wg, Wu, M, hidden, inter, alpha=1.0, activation="silu", swiglu_limit=0.0):
    X = _c(X, np.float32).reshape(M, hidden)
    Wg = _c(Wg, np.uint8).reshape(-1)
    Wu = _c(Wu, np.uint8).reshape(-1)
    assert Wg.size == q4k_bytes(inter, hidden) and Wu.size == Wg.size
    out = np.empty((M, inter), np.float32)
    lib().dor_q4k_ffn_gate_up(_ptr(X), _ptr(Wg), _ptr(Wu), M, hidden, inter, alpha,
                              0 if activation == "silu" else 1, swiglu_limit or 0.0, _ptr(out))
    return out


# --------------------------------------------------------------------------- elementwise

def act_gate(gate, up, activation="silu", swiglu_limit=0.0):
    gate = _c(gate, np.float32)
    up = _c(up, np.float32)
    assert gate.shape == up.shape
    out = np.empty(gate.shape, np.float32)
    lib().dor_act_gate(_ptr(gate), _ptr(up), gate.size, 0 if activation == "silu" else 1,
                       swiglu_limit or 0.0, _ptr(out))
    return out


def act_gate_rowsplit(x, T, dim, activation="silu", swiglu_limit=0.0):
    x = _c(x, np.float32).reshape(T, 2 * dim)
    out = np.empty((T, dim), np.float32)
    lib().dor_act_gate_rowsplit(_ptr(x), T, dim, 0 if activation == "silu" else 1,
                                swiglu_limit or 0.0, _ptr(out))
    return out


def residual_add(a, b, scale=1.0):
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    assert a.shape == b.shape
    out = np.empty(a.shape, np.float32)
    lib().dor_residual_add(_ptr(a), _ptr(b), a.size, scale, _ptr(out))
    return out


def rmsnorm(x, weight, eps, batch=None, hidden=None, weight_offset=False, pre_residual=None,
            post_residual=None, want_prenorm=False, output_scale=1.0):
    x = _c(x, np.float32)
    hidden = hidden or x.shape[-1]
    batch = batch or x.size // hidden
    x = x.reshape(batch, hidden)
    w = _c(weight, np.float32).reshape(hidden) if weight is not None else None
    pre = _c(pre_residual, np.float32).reshape(batch, hidden) if pre_residual is not None else None
    post = _c(post_residual, np.float32).reshape(batch, hidden) if post_residual is not None else None
    prenorm = np.empty((batch, hidden), np.float32) if want_prenorm else None
    out = np.empty((batch, hidden), np.float32)
    lib().dor_rmsnorm(_ptr(x), _ptr(w), batch, hidden, eps, int(bool(weight_offset)), _ptr(pre),
                      _ptr(post), _ptr(prenorm), output_scale, _ptr(out))
    return (out, prenorm) if want_prenorm else out


# --------------------------------------------------------------------------- RoPE

def rope_tables(rotary_dim, max_seq, theta, recipe="production", rope_scale=1.0):
    """recipe 'test' = tests/kernels/reference/rope.js, 'production' = init-rope.js."""
    half = rotary_dim // 2
    cos = np.empty((max_seq, half), np.float32)
    sin = np.empty((max_seq, half), np.float32)
    lib().dor_rope_tables(rotary_dim, max_seq, float(theta), 1 if recipe == "production" else 0,
                          float(rope_scale), _ptr(cos), _ptr(sin))
    return cos, sin


def rope_apply(x, cos, sin, seq, heads, head_dim, start_pos=0, rotary_dim=None,
               pair_span_dim=None, interleaved=False):
    rotary_dim = rotary_dim or head_dim
    pair_span_dim = pair_span_dim or rotary_dim
    x = _c(x, np.float32).reshape(seq, heads, head_dim)
    cos = _c(cos, np.float32)
    sin = _c(sin, np.float32)
    assert cos.shape[-1] == rotary_dim // 2 and cos.shape[0] >= start_pos + seq
    out = np.empty_like(x)
    lib().dor_rope_apply(_ptr(x), _ptr(cos), _ptr(sin), seq, heads, head_dim, start_pos,
                         rotary_dim, pair_span_dim, int(bool(interleaved)), _ptr(out))
    return out


# --------------------------------------------------------------------------- attention

def attention_ref(Q, K, V, seq, kv_len, H, Hkv, D, mask=None, scale=0.0):
    Q = _c(Q, np.float32).reshape(seq, H, D)
    K = _c(K, np.float32).reshape(kv_len, Hkv, D)
    V = _c(V, np.float32).reshape(kv_len, Hkv, D)
    m = _c(mask, np.float32).reshape(seq, kv_len) if mask is not None else None
    out = np.empty((seq, H, D), np.float32)
    lib().dor_attention_ref(_ptr(Q), _ptr(K), _ptr(V), seq, kv_len, H, Hkv, D, _ptr(m), scale,
                            _ptr(out))
    return out


def causal_mask(seq, kv_len=None):
    """tests/kernels/reference/attention.js:129-144 createCausalMask."""
    kv_len = kv_len or seq
    i = np.arange(seq)[:, None]
    j = np.arange(kv_len)[None, :]
    return np.where(j <= i + (kv_len - seq), 0.0, -np.inf).astype(np.float32)


def attention_decode_f16kv(Q, K_bits, V_bits, H, Hkv, D, kv_len, scale=None, causal=True,
                           start_pos=None, softcap=0.0, sliding_window=0, kv_start=0,
                           kv_layout=0):
    Q = _c(Q, np.float32).reshape(H, D)
    K = _c(K_bits, np.uint16).reshape(-1, Hkv, D)
    V = _c(V_bits, np.uint16).reshape(-1, Hkv, D)
    if scale is None:
        scale = 1.0 / np.sqrt(D)
    if start_pos is None:
        start_pos = kv_start + kv_len - 1
    rows_needed = sliding_window if (kv_layout == 1 and sliding_window > 0) else kv_start + kv_len
    assert K.shape[0] >= rows_needed and V.shape[0] >= rows_needed
    out = np.empty((H, D), np.float32)
    lib().dor_attention_decode_f16kv(_ptr(Q), _ptr(K), _ptr(V), H, Hkv, D, kv_len, scale,
                                     int(bool(causal)), start_pos, softcap, sliding_window,
                                     kv_start, kv_layout, _ptr(out))
    return out


# --------------------------------------------------------------------------- KV / gather / argmax

def kv_write_f16(k, v, cache_k, cache_v, src_off, dst_off, count):
    k = _c(k, np.float32).reshape(-1)
    v = _c(v, np.float32).reshape(-1)
    assert cache_k.dtype == np.uint16 and cache_v.dtype == np.uint16
    assert src_off + count <= k.size and dst_off + count <= cache_k.size
    lib().dor_kv_write_f16(_ptr(k), _ptr(v), src_off, dst_off, count, _ptr(cache_k), _ptr(cache_v))


def qkv_norm_rope_kvwrite(qkv, q_weight, k_weight, cos, sin, T, H, Hkv, D, start_pos, cache_k,
                          cache_v, kv_dst_offset, eps=1e-6, rotary_dim=None, interleaved=False,
                          weight_offset=False):
    rotary_dim = rotary_dim or D
    qkv = _c(qkv, np.float32).reshape(T, (H + 2 * Hkv) * D)
    qw = _c(q_weight, np.float32).reshape(D)
    kw = _c(k_weight, np.float32).reshape(D)
    cos = _c(cos, np.float32)
    sin = _c(sin, np.float32)
    assert cache_k.dtype == np.uint16 and cache_k.flags.c_contiguous
    assert kv_dst_offset + T * Hkv * D <= cache_k.size
    q_out = np.empty((T * H, D), np.float32)
    lib().dor_qkv_norm_rope_kvwrite(_ptr(qkv), _ptr(qw), _ptr(kw), _ptr(cos), _ptr(sin), T, H, Hkv,
                                    D, start_pos, rotary_dim, int(bool(interleaved)), eps,
                                    int(bool(weight_offset)), kv_dst_offset, _ptr(q_out),
                                    _ptr(cache_k), _ptr(cache_v))
    return q_out


def gather_f16(ids, table_bits, hidden, vocab):
    ids = _c(ids, np.uint32).reshape(-1)
    table = _c(table_bits, np.uint16).reshape(vocab, hidden)
    out = np.empty((ids.size, hidden), np.float32)
    lib().dor_gather_f16(_ptr(ids), _ptr(table), ids.size, hidden, vocab, _ptr(out))
    return out


def argmax(logits, pad_id=None, softcap=0.0):
    logits = _c(logits, np.float32).reshape(-1)
    return int(lib().dor_argmax(_ptr(logits), logits.size, -1 if pad_id is None else pad_id,
                                softcap))


def sample_topk(logits, temperature, top_k, random_value, pad_id=None, softcap=0.0):
    logits = _c(logits, np.float32).reshape(-1)
    return int(lib().dor_sample_topk(_ptr(logits), logits.size, float(temperature), int(top_k), float(random_value),
                                     -1 if pad_id is None else pad_id, softcap))


def seeded_random(seed):
    return float(lib().dor_seeded_random(float(seed)))


# --------------------------------------------------------------------------- dense matmul + RMSNorm

def matmul_rmsnorm_fused(x, W, norm_weight, N, K, eps, transpose_b=True, weight_offset=False, residual=None):
    """src/gpu/kernels/fused_matmul_rmsnorm.wgsl:215-272 (gemv_rmsnorm_medium; :166-213 is the same
    arithmetic for N <= 256): y[n] = sum_k x[k] * W(n, k) with W stored [N, K] (transpose_b) or
    [K, N]; out[n] = y[n] / sqrt(sum(y^2) / N + eps) * (w[n] | 1 + w[n]) + residual[n].  Sums run
    in float64 and each stage is rounded to f32 where the shader stores one."""
    x = _c(x, np.float32).reshape(K).astype(np.float64)
    W = _c(W, np.float32).reshape((N, K) if transpose_b else (K, N)).astype(np.float64)
    y = ((W @ x) if transpose_b else (x @ W)).astype(np.float32).astype(np.float64)
    inv_rms = 1.0 / np.sqrt(np.sum(y * y) / N + float(eps))
    w = _c(norm_weight, np.float32).reshape(N).astype(np.float64)
    if weight_offset:
        w = 1.0 + w
    out = y * inv_rms * w
    if residual is not None:
        out = out.astype(np.float32).astype(np.float64) + _c(residual, np.float32).reshape(N)
    return out.astype(np.float32)


# --------------------------------------------------------------------------- finiteness guard

def finiteness_should_trigger(value, abs_threshold=65500):
    """src/gpu/kernels/check-finiteness.js:7-19: a threshold that is not a positive finite number
    falls back to 65500; NaN and +-inf always trigger."""
    thr = abs_threshold if (abs_threshold is not None and np.isfinite(abs_threshold) and abs_threshold > 0) else 65500
    v = float(value)
    return (not np.isfinite(v)) or abs(v) > thr


def check_finiteness(values, status, layer=0, step=0, abs_threshold=65500):
    """src/gpu/kernels/check-finiteness.js:25-62: `status` is 4 u32 words, updated in place; the
    first triggering call turns word 0 from 0 to 1 and records its layer and step in words 1
    and 2, later calls leave a set status alone.  The f32 compare is the shader's: the value
    (f16 widened, or f32) against the threshold rounded to f32."""
    v = np.asarray(values)
    assert v.dtype in (np.float16, np.float32)
    v = v.astype(np.float32).ravel()
    thr = np.float32(abs_threshold if (np.isfinite(abs_threshold) and abs_threshold > 0) else 65500)
    bits = v.view(np.uint32)
    bad = ((bits & 0x7F800000) == 0x7F800000) | (np.abs(v) > thr)
    if bad.any() and status[0] == 0:
        status[0], status[1], status[2] = 1, layer, step
    return status


def finiteness_parse_status(words, offset=0):
    """src/inference/pipelines/text/finiteness-guard-status.js:1-21."""
    words = list(words)
    get = lambda i: int(words[i]) if i < len(words) else 0
    if get(offset) <= 0:
        return {"triggered": False, "layer": 0, "step": 0, "metadata": ""}
    layer, step = get(offset + 1), get(offset + 2)
    return {"triggered": True, "layer": layer, "step": step, "metadata": " (layer %d, step %d)" % (layer, step)}


# --------------------------------------------------------------------------- decode step

class DecoderOracle:
    """Holds numpy weights of a Q4_K decoder and steps it one token at a time."""

    def __init__(self, cfg, layers, embed_bits, final_norm, cos, sin):
        self.cfg = ModelCfg(cfg["layers"], cfg["hidden"], cfg["inter"], cfg["heads"],
                            cfg["kv_heads"], cfg["head_dim"], cfg["vocab"], cfg["max_seq"],
                            cfg["eps"], int(cfg.get("qk_norm", 1)))
        self._keep = (layers, embed_bits, final_norm, cos, sin)
        arr = (Layer * len(layers))()
        for i, L in enumerate(layers):
            for name, _ in Layer._fields_:
                a = L[name]
                assert a.flags.c_contiguous
                setattr(arr[i], name, a.ctypes.data)
        self._layers = arr
        self.embed, self.final_norm, self.cos, self.sin = embed_bits, final_norm, cos, sin
        self.vocab = cfg["vocab"]

    def step(self, token, pos, want_logits=False):
        logits = np.empty(self.vocab, np.float32) if want_logits else None
        tok = lib().dor_decode_step(ctypes.byref(self.cfg), self._layers, _ptr(self.embed),
                                    _ptr(self.final_norm), _ptr(self.cos), _ptr(self.sin),
                                    int(token), int(pos), _ptr(logits))
        return (int(tok), logits) if want_logits else int(tok)
