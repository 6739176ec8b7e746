"""ctypes binding of libdopplerhip.so (the C ABI declared in include/doppler_hip.h).

There is no fallback: if the shared library is missing or a call fails, a DopplerHipError is
raised with the library's own message.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libdopplerhip.so")

F32, F16 = 0, 1
ACT_SILU, ACT_GELU = 0, 1
KV_CONTIGUOUS, KV_RING = 0, 1
PLAN_GEMV_I8, PLAN_GEMV_ROWS, PLAN_GEMV_RING, PLAN_GEMM, PLAN_GEMV_LDS = 1, 2, 3, 4, 5


class DopplerHipError(RuntimeError):
    pass


_P = ctypes.c_void_p
_I = ctypes.c_int
_I64 = ctypes.c_int64
_F = ctypes.c_float
_SZ = ctypes.c_size_t

class ChainPhase(ctypes.Structure):
    """struct dh_chain_phase: one product of dh_q4k_gemv_chain."""
    _fields_ = [("d_W", _P), ("d_W2", _P), ("d_C", _P), ("d_residual", _P), ("d_norm_weight", _P),
                ("N", _I), ("K", _I), ("activation", _I), ("norm_weight_offset", _I),
                ("alpha", _F), ("swiglu_limit", _F), ("norm_eps", _F)]


class ChainAttnSource(ctypes.Structure):
    """struct dh_chain_attn_source: the attention partial results a chain's first product merges."""
    _fields_ = [("d_workspace", _P), ("H", _I), ("Hkv", _I), ("D", _I), ("nsplit", _I), ("d_kv_len", _P),
                ("max_kv_len", _I), ("sliding_window", _I), ("kv_start", _I)]


def chain_phases(phases):
    """list of dicts (W, W2, C, residual, norm_weight: device addresses or None; N, K; activation,
    norm_weight_offset, alpha, swiglu_limit, norm_eps) -> ctypes array of dh_chain_phase."""
    arr = (ChainPhase * len(phases))()
    for i, ph in enumerate(phases):
        arr[i] = ChainPhase(ph["W"], ph.get("W2"), ph["C"], ph.get("residual"), ph.get("norm_weight"), ph["N"], ph["K"],
                            ph.get("activation", 0), ph.get("norm_weight_offset", 0), ph.get("alpha", 1.0),
                            ph.get("swiglu_limit", 0.0), ph.get("norm_eps", 0.0))
    return arr


# name -> (restype, argtypes); every symbol include/doppler_hip.h declares
SIGNATURES = {
    "dh_init": (_I, [_I]),
    "dh_shutdown": (_I, []),
    "dh_last_error": (ctypes.c_char_p, []),
    "dh_set_stream": (_I, [_P]),
    "dh_get_stream": (_P, []),
    "dh_malloc": (_I, [_SZ, ctypes.POINTER(_P)]),
    "dh_free": (_I, [_P]),
    "dh_upload": (_I, [_P, _SZ, _P, _SZ]),
    "dh_download": (_I, [_P, _P, _SZ, _SZ]),
    "dh_copy": (_I, [_P, _SZ, _P, _SZ, _SZ]),
    "dh_fill_zero": (_I, [_P, _SZ, _SZ]),
    "dh_sync": (_I, []),
    "dh_host_alloc": (_I, [_SZ, ctypes.POINTER(_P)]),
    "dh_host_free": (_I, [_P]),
    "dh_download_async": (_I, [_P, _P, _SZ, _SZ]),
    "dh_event_synchronize": (_I, [_P]),
    "dh_event_create": (_I, [ctypes.POINTER(_P)]),
    "dh_event_record": (_I, [_P]),
    "dh_event_elapsed_ms": (_I, [_P, _P, ctypes.POINTER(_F)]),
    "dh_event_destroy": (_I, [_P]),
    "dh_graph_begin": (_I, []),
    "dh_graph_end": (_I, [_I, ctypes.POINTER(_P)]),
    "dh_graph_launch": (_I, [_P, _I]),
    "dh_graph_set_max_position": (_I, [_P, _I]),
    "dh_graph_prepare": (_I, [_P, _I]),
    "dh_graph_destroy": (_I, [_P]),
    "dh_q4k_dequant": (_I, [_P, _I64, _P]),
    "dh_q4k_matmul": (_I, [_P, _I, _P, _P, _I, _I, _I, _I, _F, _P]),
    "dh_q4k_matmul_rmsnorm": (_I, [_P, _P, _F, _I, _P, _P, _I, _I, _I, _I, _F, _P]),
    "dh_q4k_matmul_plan": (_I, [_I, _I, _I, _I, _I, _I]),
    "dh_q4k_gemv_layout": (_I, [_I, _I, _I, _I, _I, _I, ctypes.POINTER(ctypes.c_int64)]),
    "dh_q4k_ffn_gate_up": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _F, _F]),
    "dh_q4k_ffn_gate_up_rmsnorm": (_I, [_P, _P, _F, _I, _P, _P, _P, _I, _I, _I, _I, _F, _F]),
    "dh_q4k_gemv_chain": (_I, [_P, ctypes.POINTER(ChainPhase), _I]),
    "dh_q4k_gemv_chain_limited": (_I, [_P, ctypes.POINTER(ChainPhase), _I, _I, _I]),
    "dh_q4k_gemv_chain_attn_supported": (_I, [_I, _I, _I, _I]),
    "dh_q4k_gemv_chain_attn": (_I, [ctypes.POINTER(ChainAttnSource), ctypes.POINTER(ChainPhase), _I]),
    "dh_f16w_matmul": (_I, [_P, _P, _P, _I, _I, _I, _F]),
    "dh_lmhead_argmax_workspace_bytes": (_SZ, [_I]),
    "dh_lmhead_argmax_f16": (_I, [_P, _P, _I, _I, _I64, _F, _P, _P, _I, _P]),
    "dh_lmhead_argmax_f16_rmsnorm": (_I, [_P, _P, _F, _I, _P, _I, _I, _I64, _F, _P, _P, _I, _P]),
    "dh_attn_decode_workspace_bytes": (_SZ, [_I, _I, _I]),
    "dh_attn_prefill": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _F, _I]),
    "dh_attn_decode": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _F, _I, _I, _F, _I, _I, _I, _P]),
    "dh_attn_decode_static_max_bytes": (_SZ, []),
    "dh_attn_decode_static": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _F, _I, _I, _F, _I, _I, _I]),
    "dh_attn_decode_qkv_supported": (_I, [_I, _I, _I, _I, _I]),
    "dh_attn_decode_qkv": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _F, _F, _I, _I,
                                _I, _P]),
    "dh_attn_decode_kvlen": (_I, [_P, _P, _P, _P, _I, _I, _I, _P, _I, _F, _I, _I, _F, _I, _I, _I, _P]),
    "dh_attn_decode_qkv_kvlen": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P, _I, _I, _I, _F, _I, _I, _F, _F, _I,
                                      _I, _I, _P]),
    "dh_attn_decode_qkv_partials": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _I, _F, _F, _I, _I,
                                         _I, _P, ctypes.POINTER(_I)]),
    "dh_attn_decode_qkv_kvlen_partials": (_I, [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _P, _I, _I, _I, _F, _I, _I, _F, _F,
                                               _I, _I, _I, _P]),
    "dh_rmsnorm": (_I, [_P, _P, _I, _P, _I, _I, _F, _I, _P, _P, _P, _F]),
    "dh_rmsnorm_sandwich_pair": (_I, [_P, _P, _P, _I, _P, _I, _P, _P, _I, _I, _F, _I]),
    "dh_residual_rmsnorm_pair": (_I, [_P, _P, _P, _I, _P, _P, _I, _I, _F, _I, _F]),
    "dh_rmsnorm_qk": (_I, [_P, _P, _P, _I, _P, _I, _P, _P, _I, _I, _I, _F, _I]),
    "dh_rope": (_I, [_P, _P, _P, _I, _I, _I, _I, _I, _I, _I]),
    "dh_rope_qk": (_I, [_P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I]),
    "dh_qkv_norm_rope_kvwrite": (_I, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F,
                                      _I, _I64, _I]),
    "dh_kv_write_f16": (_I, [_P, _P, _P, _P, _I64, _I64, _I64]),
    "dh_residual_add": (_I, [_P, _P, _P, _I64, _F]),
    "dh_bias_add": (_I, [_P, _P, _I, _I64, _I, _I64, _I64]),
    "dh_scale": (_I, [_P, _P, _I64, _F]),
    "dh_split_qkv": (_I, [_P, _P, _P, _P, _I, _I, _I, _I]),
    "dh_gather_f16": (_I, [_P, _P, _P, _I, _I, _I, _I]),
    "dh_act_gate": (_I, [_P, _P, _P, _I64, _I, _F]),
    "dh_act_gate_rowsplit": (_I, [_P, _P, _I, _I, _I, _F]),
    "dh_argmax_workspace_bytes": (_SZ, []),
    "dh_argmax": (_I, [_P, _I, _I64, _F, _P, _P, _I]),
    "dh_sample_topk_workspace_bytes": (_SZ, [_I, _I]),
    "dh_sample_topk": (_I, [_P, _I, ctypes.c_double, _I, ctypes.c_double, _I64, _F, _P, _P, _I]),
    "dh_cast_f32_to_f16": (_I, [_P, _P, _I64]),
    "dh_cast_f16_to_f32": (_I, [_P, _P, _I64]),
    "dh_matmul_rmsnorm_f32": (_I, [_P, _P, _I, _P, _I, _F, _I, _P, _P, _I, _I]),
    "dh_matmul_rmsnorm_f16": (_I, [_P, _P, _I, _P, _I, _F, _I, _P, _P, _I, _I]),
    "dh_check_finiteness": (_I, [_P, _I, _I64, _P, ctypes.c_uint32, ctypes.c_uint32, _F]),
}



_lib = None


def load():
    """Loads the shared library (no GPU needed for loading) and types every symbol."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise DopplerHipError(
                "libdopplerhip.so is not built (expected %s); run `python -m doppler_amd.build`" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(rc):
    if rc != 0:
        raise DopplerHipError(load().dh_last_error().decode("utf-8", "replace"))


_initialised = False


def init(device=0):
    global _initialised
    check(load().dh_init(device))
    _initialised = True
    return _lib
