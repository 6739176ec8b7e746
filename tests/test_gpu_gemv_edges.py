"""Edge behaviour of the decode GEMV kernels through the C ABI (dh_q4k_matmul, dh_q4k_ffn_gate_up) at
M = 1, 2 (int8 matrix-core kernel) and M = 4, 8 (few-row f16 matrix-core kernel), against the CPU
oracle: activation outliers judged PER ELEMENT (a relative L2 over a row hides what an outlier does
to its neighbours), tiny and subnormal activations, and non-finite activations, which the
reference's f32 kernels propagate (src/gpu/kernels/fused_matmul_q4.wgsl:122-258) and its guard
then catches (src/gpu/kernels/check-finiteness.js:25-62).
"""
import numpy as np
import pytest

import oracle
from doppler_amd import ops, synth

pytestmark = pytest.mark.gpu

N, K = 1024, 4096            # 16 super-block columns; served by the int8 kernel (M <= 2) and the few-row kernel (M 3..15)
PER_ELEMENT = 1e-5           # of the row's sum of |w x|: what an f32 accumulation itself may lose


def _weight(n, k, seed):
    W = synth.q4k_tensor(n, k, seed)
    buf = ops.acquireBuffer(W.size)
    ops.uploadData(buf, W)
    return W, ops.createWeightBuffer(buf, "q4k", "row", (n, k), "w%d" % seed)


def _abs_product(W, A, n, k):
    """sum over k of |w[n,k] x[m,k]| in f64: the scale an error of the product is judged against."""
    Wd = np.abs(oracle.q4k_dequant_rows(W, n, k).astype(np.float64))
    return np.abs(A.astype(np.float64)) @ Wd.T


def _with_outliers(M, seed):
    A = synth.normal_f32((M, K), seed)
    r = synth.rng(seed + 1)
    for m in range(M):
        for c in range(K // 256):
            i, j = r.choice(256, 2, replace=False)
            A[m, c * 256 + i] = 1e3 * (1 if r.random() < 0.5 else -1)
            A[m, c * 256 + j] = 1e6 * (1 if r.random() < 0.5 else -1)
    return A


@pytest.mark.parametrize("M", [1, 2, 4, 8])
def test_matmul_outliers_per_element(M):
    W, wb = _weight(N, K, 4100)
    A = _with_outliers(M, 4110 + M)
    got = ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(A), wb, M, N, K, outputDtype="f32")).astype(np.float64)
    want = oracle.q4k_matmul(A, W, M, N, K).astype(np.float64)
    bound = PER_ELEMENT * _abs_product(W, A, N, K)
    worst = float(np.max(np.abs(got.reshape(M, N) - want.reshape(M, N)) / bound))
    assert worst <= 1.0, worst


@pytest.mark.parametrize("M", [1, 2, 4, 8])
def test_outlier_does_not_cost_the_other_sub_blocks_their_bits(M):
    """A 1e6 outlier in every 256-column, placed in a sub-block whose weights are all zero (scale and
    min 0): it contributes exactly nothing, so the product is that of the other seven sub-blocks, whose
    N(0,1) activations must keep their own precision.  With one exponent per column they would be
    quantised in steps of about 1 and the result would be noise."""
    W = synth.q4k_tensor(N, K, 4120).reshape(N, K // 256, 144).copy()
    W[:, :, 4] &= 0xC0            # 6-bit scale of sub-block 0
    W[:, :, 8] &= 0xC0            # 6-bit min of sub-block 0
    W = W.reshape(-1)
    buf = ops.acquireBuffer(W.size)
    ops.uploadData(buf, W)
    wb = ops.createWeightBuffer(buf, "q4k", "row", (N, K), "wz0")
    A = synth.normal_f32((M, K), 4121 + M)
    A[:, 7::256] = 1e6
    got = ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(A), wb, M, N, K, outputDtype="f32")).astype(np.float64).reshape(M, N)
    want = oracle.q4k_matmul(A, W, M, N, K).astype(np.float64).reshape(M, N)
    clean = A.copy()
    clean[:, 7::256] = 0
    assert np.array_equal(want, oracle.q4k_matmul(clean, W, M, N, K).astype(np.float64).reshape(M, N))
    assert float(np.linalg.norm(got - want) / np.linalg.norm(want)) <= 1e-5
    assert float(np.max(np.abs(got - want) / (PER_ELEMENT * _abs_product(W, clean, N, K)))) <= 1.0


@pytest.mark.parametrize("M", [1, 2, 4, 8])
@pytest.mark.parametrize("activation", ["silu", "gelu"])
def test_ffn_outliers_per_element(M, activation):
    hidden, inter = K, N
    Wg, wg = _weight(inter, hidden, 4130)
    Wu, wu = _weight(inter, hidden, 4131)
    X = _with_outliers(M, 4140 + M) * np.float32(1e-3)      # outliers 1 and 1e3 among N(0, 1e-3): the gate stays in the activation's curved range
    got = ops.readTensor(ops.runFusedFFN(ops.tensorFromNumpy(X), wg, wu, hidden, inter, batchSize=M,
                                         activation=activation)).astype(np.float64).reshape(M, inter)
    want = oracle.q4k_ffn_gate_up(X, Wg, Wu, M, hidden, inter, activation=activation).astype(np.float64).reshape(M, inter)
    g = oracle.q4k_matmul(X, Wg, M, inter, hidden).astype(np.float64).reshape(M, inter)
    u = oracle.q4k_matmul(X, Wu, M, inter, hidden).astype(np.float64).reshape(M, inter)
    sg, su = _abs_product(Wg, X, inter, hidden), _abs_product(Wu, X, inter, hidden)
    # |d act| <= 1.13 |dg| for both activations; act(g) <= |g|
    bound = PER_ELEMENT * (1.13 * sg * np.abs(u) + np.abs(g) * su) + 1e-30
    assert float(np.max(np.abs(got - want) / bound)) <= 1.0


@pytest.mark.parametrize("M", [1, 2, 4, 8])
def test_matmul_tiny_and_subnormal_activations(M):
    W, wb = _weight(N, K, 4150)
    base = synth.normal_f32((M, K), 4151 + M)
    # all activations around 1e-30: every element keeps its bits
    A = (base * np.float32(1e-30)).astype(np.float32)
    got = ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(A), wb, M, N, K, outputDtype="f32")).astype(np.float64).reshape(M, N)
    want = oracle.q4k_matmul(A, W, M, N, K).astype(np.float64).reshape(M, N)
    assert float(np.max(np.abs(got - want) / (PER_ELEMENT * _abs_product(W, A, N, K)))) <= 1.0
    # subnormal activations among ordinary ones: they are below what the row's sum can resolve
    A = base.copy()
    A[:, 3::16] = np.float32(1e-40)
    assert A[0, 3] != 0 and abs(A[0, 3]) < np.finfo(np.float32).tiny
    got = ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(A), wb, M, N, K, outputDtype="f32")).astype(np.float64).reshape(M, N)
    want = oracle.q4k_matmul(A, W, M, N, K).astype(np.float64).reshape(M, N)
    assert float(np.max(np.abs(got - want) / (PER_ELEMENT * _abs_product(W, A, N, K)))) <= 1.0
    # nothing but subnormals: magnitudes below 2^-127 count as zero (flush-to-zero, as f32 GPU arithmetic does)
    A = (base * np.float32(1e-40)).astype(np.float32)
    got = ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(A), wb, M, N, K, outputDtype="f32")).astype(np.float64).reshape(M, N)
    want = oracle.q4k_matmul(A, W, M, N, K).astype(np.float64).reshape(M, N)
    Wabs = np.abs(oracle.q4k_dequant_rows(W, N, K).astype(np.float64)).sum(axis=1)
    assert np.all(np.isfinite(got))
    assert float(np.max(np.abs(got - want) / (2.0 ** -126 * Wabs[None, :]))) <= 1.0


def _finite_pattern_case(M, bad, via_ffn):
    """Row 0 gets one bad activation; the other rows stay clean and must stay accurate."""
    W, wb = _weight(N, K, 4160)
    A = synth.normal_f32((M, K), 4161 + M)
    A[0, 1234] = bad
    with np.errstate(invalid="ignore", over="ignore"):
        if via_ffn:
            W2, wb2 = _weight(N, K, 4162)
            got = ops.readTensor(ops.runFusedFFN(ops.tensorFromNumpy(A), wb, wb2, K, N, batchSize=M)).reshape(M, N)
            want = oracle.q4k_ffn_gate_up(A, W, W2, M, K, N).reshape(M, N)
        else:
            got = ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(A), wb, M, N, K, outputDtype="f32")).reshape(M, N)
            want = oracle.q4k_matmul(A, W, M, N, K).reshape(M, N)
    return got, want


@pytest.mark.parametrize("M", [1, 2, 4, 8])
@pytest.mark.parametrize("via_ffn", [False, True])
@pytest.mark.parametrize("bad", [np.nan, np.inf, -np.inf])
def test_non_finite_activation_reaches_the_outputs(M, via_ffn, bad):
    got, want = _finite_pattern_case(M, np.float32(bad), via_ffn)
    # non-finite exactly where the oracle's outputs are: all of row 0, nothing else
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    assert not np.isfinite(want[0]).any()
    if M > 1:
        ok = np.isfinite(want)
        rel = np.linalg.norm(got[ok].astype(np.float64) - want[ok]) / np.linalg.norm(want[ok])
        assert rel <= 1e-3
    if np.isnan(bad):
        assert np.isnan(got[0]).all()
    elif M <= 2 and not via_ffn:
        # the int8 kernel finishes the infinite sub-block in f32 before the factor is applied:
        # +-Inf with the sign of the weight it met, as in the oracle (NaN where that weight is zero)
        assert np.array_equal(np.isnan(got[0]), np.isnan(want[0]))
        inf = np.isinf(want[0])
        assert np.array_equal(got[0][inf], want[0][inf])


def test_infinity_meets_a_zero_weight():
    """Inf x 0 is NaN: a super-block with d = dmin = 0 (all weights zero) turns an infinite activation
    into NaN, not into 0 or Inf."""
    W = synth.q4k_tensor(N, K, 4170).reshape(N, K // 256, 144).copy()
    W[5, 2, 0:4] = 0               # row 5, column 2: d = dmin = +0
    W = W.reshape(-1)
    buf = ops.acquireBuffer(W.size)
    ops.uploadData(buf, W)
    wb = ops.createWeightBuffer(buf, "q4k", "row", (N, K), "wz")
    A = synth.normal_f32((1, K), 4171)
    A[0, 2 * 256 + 40] = np.inf
    got = ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(A), wb, 1, N, K, outputDtype="f32")).reshape(N)
    with np.errstate(invalid="ignore", over="ignore"):
        want = oracle.q4k_matmul(A, W, 1, N, K).reshape(N)
    assert np.isnan(want[5]) and np.isnan(got[5])
    assert np.array_equal(np.isnan(got), np.isnan(want))
    inf = np.isinf(want)
    assert np.array_equal(got[inf], want[inf])
