"""No-GPU checks of the C ABI: the library loads and exports exactly what the header declares,
and calls fail loudly (not silently) when no device has been initialised."""
import os
import re

import pytest

from doppler_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "doppler_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dh_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_python_binds():
    assert header_symbols() == sorted(capi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    for name in header_symbols():
        assert hasattr(lib, name), name


def test_ops_fail_loudly_without_init():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present: covered by the GPU error tests")
    lib = capi.load()
    assert lib.dh_sync() != 0
    assert b"dh_init" in lib.dh_last_error()
    assert lib.dh_q4k_matmul(None, 0, None, None, 0, 1, 1, 256, 1.0, None) != 0
    from doppler_amd import ops
    with pytest.raises(capi.DopplerHipError):
        ops.acquireBuffer(16)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "doppler_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".js", ".mjs", ".hip", ".h", ".c")):
                src = open(os.path.join(dirpath, f), errors="replace").read()
                assert "import oracle" not in src and "from oracle" not in src and "doppler_oracle" not in src, f


def test_finiteness_host_helpers_follow_the_reference_tests():
    from doppler_amd import ops
    # tests/inference/finiteness-overflow-gate.test.js
    assert ops.resolveFinitenessAbsThreshold(None) == ops.DEFAULT_FINITENESS_ABS_THRESHOLD == 65500
    assert ops.resolveFinitenessAbsThreshold(50000) == 50000
    assert ops.resolveFinitenessAbsThreshold(-1) == 65500
    assert ops.shouldTriggerFinitenessValue(100) is False
    assert ops.shouldTriggerFinitenessValue(65501, 65500) is True
    assert ops.shouldTriggerFinitenessValue(-70000, 65500) is True
    for v in (float("inf"), float("-inf"), float("nan")):
        assert ops.shouldTriggerFinitenessValue(v, 65500) is True
    # tests/inference/finiteness-guard-status.test.js
    assert ops.parseFinitenessStatusWords([0, 7, 9], 0) == {"triggered": False, "layer": 0, "step": 0, "metadata": ""}
    assert ops.parseFinitenessStatusWords([1, 8, 12], 0) == {"triggered": True, "layer": 8, "step": 12,
                                                             "metadata": " (layer 8, step 12)"}
    assert ops.parseFinitenessStatusWords([42, 1, 3, 15, 0], 1)["metadata"] == " (layer 3, step 15)"


def test_fused_matmul_rmsnorm_selection_follows_the_reference_rules():
    from doppler_amd import ops
    # src/rules/kernels/fused-matmul-rmsnorm.rules.json; small means N <= 256
    assert ops.selectMatmulRMSNormFusedVariant(256, "f32") == "small"
    assert ops.selectMatmulRMSNormFusedVariant(256, "f16") == "small_f16"
    assert ops.selectMatmulRMSNormFusedVariant(257, "f32") == "medium"
    assert ops.selectMatmulRMSNormFusedVariant(1152, "f16") == "medium_f16"
    with pytest.raises(capi.DopplerHipError, match="dtype is required"):
        ops.selectMatmulRMSNormFusedVariant(8, None)
    # src/gpu/kernels/fused_matmul_rmsnorm.js:295-312
    assert ops.shouldUseFusedMatmulRMSNorm(1, 4096, 8192) is True
    assert ops.shouldUseFusedMatmulRMSNorm(2, 1152, 6912) is False
    assert ops.shouldUseFusedMatmulRMSNorm(1, 4097, 1024) is False
    assert ops.shouldUseFusedMatmulRMSNorm(1, 1152, 8193) is False
    assert ops.shouldUseFusedMatmulRMSNorm(1, 1152) is True


def test_matmul_plan_pins_the_kernel_family_of_every_benchmark_shape():
    """dh_q4k_matmul_plan needs no device: the family each BASELINE shape (and the shapes on either
    side of every dispatch boundary) is served by, so that a regression onto a slower family shows
    up here and not only as a number in a benchmark."""
    L = capi.load()
    I8, ROWS, RING, GEMM, LDS = (capi.PLAN_GEMV_I8, capi.PLAN_GEMV_ROWS, capi.PLAN_GEMV_RING, capi.PLAN_GEMM,
                                 capi.PLAN_GEMV_LDS)

    def plan(M, N, K, normed=0, dual=0, cus=256):
        return L.dh_q4k_matmul_plan(M, N, K, normed, dual, cus)

    # config 0: one 640 -> 2048 product
    assert plan(1, 2048, 640) == I8
    # config 1: the linear layers of a hidden-1024 block at M = 1, 2, 4, 8
    for N, K in ((2048, 1024), (1024, 1024), (1024, 2048), (3072, 1024)):
        assert [plan(M, N, K) for M in (1, 2, 4, 8)] == [I8, I8, RING, RING], (N, K)
    assert [plan(M, 3072, 1024, 1, 1) for M in (1, 2, 4, 8)] == [I8, I8, RING, RING]
    assert [plan(M, 1024, 3072) for M in (1, 2, 4, 8)] == [I8, I8, ROWS, ROWS]
    # config 2: prefill FFN at M = 512
    assert plan(512, 6912, 1152, 0, 1) == GEMM and plan(512, 1152, 6912) == GEMM
    # config 4: the decoder's products (normed q/k/v, o, normed gate/up pair, down), M across every boundary
    for N, K, normed, dual in ((6144, 4096, 1, 0), (4096, 4096, 0, 0), (12288, 4096, 1, 1), (4096, 12288, 0, 0)):
        got = [plan(M, N, K, normed, dual) for M in (1, 2, 3, 8, 9, 15, 16, 2048)]
        assert got == [I8, I8, ROWS, ROWS, ROWS, ROWS, GEMM, GEMM], (N, K, got)
    # rows longer than the int8 kernel's LDS holds with the RMSNorm prologue go to the few-row kernel
    assert [plan(M, 4096, 32768, 1, 0) for M in (1, 2, 3)] == [ROWS, ROWS, ROWS]
    assert plan(1, 4096, 25088, 1, 0) == I8 and plan(1, 4096, 25344, 1, 0) == ROWS
    # K off the vector path, tiny shapes
    assert plan(1, 512, 1023) == I8 and plan(4, 512, 1023) == RING and plan(16, 512, 1023) == GEMM
    assert plan(1, 8, 256) == RING and plan(5, 8, 256) == RING      # one column per tile: too many tile slots for the int8 kernel
    # a device with a quarter of the compute units: more tiles per workgroup; the few-row kernel's
    # per-tile accumulators then no longer fit the LDS for the gate/up pair
    assert plan(1, 12288, 4096, 1, 1, cus=64) == I8 and plan(8, 12288, 4096, 1, 1, cus=64) == RING
    assert plan(8, 4096, 4096, 0, 0, cus=64) == ROWS
    # what nothing serves fails with a message instead of a family
    assert plan(16, 4096, 40000, 1, 0) == 0 and b"K <= 16384" in L.dh_last_error()
    assert plan(0, 8, 256) == 0 and b"Dimensions must be positive" in L.dh_last_error()
