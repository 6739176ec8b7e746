"""GPU parity tests: every op goes through the C ABI (doppler_amd.ops -> libdopplerhip.so)
and is compared with the CPU oracle on the same seeded inputs.

Bars (BASELINE north star): bit-exact for Q4_K unpacking / dequantized weights, integer
results (argmax, gather, f16 narrowing); relative L2 <= 1e-3 for f32-accumulate matmul,
attention and logits.
"""
import numpy as np
import pytest

import oracle
from doppler_amd import capi, ops, synth
from doppler_amd.capi import DopplerHipError

pytestmark = pytest.mark.gpu

REL_L2_F32 = 1e-3
REL_L2_F16_MFMA = 5e-3      # prefill GEMM: weights and activations rounded to f16 for the matrix cores


def matmul_bar(M):
    """M >= 16 takes the f16 matrix-core GEMM, smaller batches the f32-accurate GEMV."""
    return REL_L2_F16_MFMA if M >= 16 else REL_L2_F32


def rel_l2(got, want):
    got = np.asarray(got, np.float64).reshape(-1)
    want = np.asarray(want, np.float64).reshape(-1)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))


def q4k_weight(N, K, seed):
    W = synth.q4k_tensor(N, K, seed)
    buf = ops.acquireBuffer(W.size)
    ops.uploadData(buf, W)
    return W, ops.createWeightBuffer(buf, "q4k", "row", (N, K), "w%d" % seed)


# ----------------------------------------------------------------------------- dequant (bit-exact)

def test_dequant_bit_exact_synthetic_cfg0():
    N, K = synth.CFG0["N"], synth.CFG0["K"]
    W, wb = q4k_weight(N, K, seed=1000)
    nblk = W.size // 144
    got = ops.readTensor(ops.runDequantQ4K(wb, nblk))
    want = oracle.q4k_dequant_blocks(W)
    assert got.tobytes() == want.tobytes()


def test_dequant_bit_exact_real_scales_and_edge_d(receipt):
    nb = 20000
    q = synth.rng(5).integers(0, 16, size=(nb, 256), dtype=np.uint8)
    d_bits = receipt["d_bits"][:nb].copy()
    dmin_bits = receipt["dmin_bits"][:nb].copy()
    # edge cases for the f16 multipliers: zero, smallest/largest subnormal, smallest normal, max finite
    d_bits[:6] = [0, 1, 0x3FF, 0x400, 0x7BFF, 0x3C00]
    dmin_bits[:6] = [0x7BFF, 0x400, 1, 0, 0x3FF, 0x3C00]
    blocks = synth.q4k_pack_block_fields(d_bits, dmin_bits, receipt["scale_bits"][:nb * 8].reshape(nb, 8),
                                         receipt["min_bits"][:nb * 8].reshape(nb, 8), q).reshape(-1)
    buf = ops.acquireBuffer(blocks.size)
    ops.uploadData(buf, blocks)
    got = ops.readTensor(ops.runDequantQ4K(buf, nb))
    with np.errstate(over="ignore", invalid="ignore"):
        want = oracle.q4k_dequant_blocks(blocks)
    assert got.tobytes() == want.tobytes()


# ----------------------------------------------------------------------------- Q4_K matmul

def _matmul_case(M, N, K, seed, alpha=1.0, outputDtype="f32", residual=False):
    W, wb = q4k_weight(N, K, seed)
    A = synth.normal_f32((M, K), seed + 1)
    a = ops.tensorFromNumpy(A)
    res = synth.normal_f32((M, N), seed + 2) if residual else None
    r = ops.tensorFromNumpy(res) if residual else None
    out = ops.runMatmul(a, wb, M, N, K, alpha=alpha, outputDtype=outputDtype, role="test", residualTensor=r)
    assert out.shape == (M, N) and out.dtype == outputDtype
    got = ops.readTensor(out)
    if outputDtype == "f16":
        got = got.view(np.float16).astype(np.float32)
    want = oracle.q4k_matmul(A, W, M, N, K, alpha)
    if residual:
        want = want + res
    # the weight buffer must come back untouched (the reference's parity test asserts the same)
    assert ops.readBuffer(wb.buffer, W.size).tobytes() == W.tobytes()
    return rel_l2(got, want)


@pytest.mark.parametrize("M,N,K,outputDtype,residual", [
    (4, 6144, 1536, "f16", False),      # the shape of the reference's f16-activation parity test
    (1, 1024, 4096, "f16", False), (1, 4096, 4096, "f32", True), (8, 512, 1152, "f32", False),
    (12, 96, 300, "f16", True), (33, 257, 2048, "f32", True),
    # rows loaded as f16 by the decode kernels themselves: one and two rows (int8 kernel, K with a partial last
    # column too), three to eight and two passes of them (rows kernel)
    (2, 4096, 4096, "f16", True), (2, 1024, 1156, "f32", False), (1, 12288, 4096, "f32", False),
    (5, 4096, 3204, "f32", True), (8, 4096, 4096, "f16", False), (13, 4096, 3072, "f32", True)])
def test_matmul_f16_activations(M, N, K, outputDtype, residual):
    """f16 activations (tests/kernels/fused-matmul-q4-widetile-f16a-parity.test.js runs M=4, K=1536,
    N=6144): the product of the exactly widened rows, accumulated in f32."""
    W, wb = q4k_weight(N, K, 1150 + M)
    A16 = synth.normal_f32((M, K), 1151 + M).astype(np.float16)
    a = ops.tensorFromNumpy(A16.view(np.uint16))
    assert a.dtype == "f16"
    res = synth.normal_f32((M, N), 1152 + M) if residual else None
    out = ops.runMatmul(a, wb, M, N, K, outputDtype=outputDtype, role="test",
                        residualTensor=ops.tensorFromNumpy(res) if residual else None)
    got = ops.readTensor(out)
    if outputDtype == "f16":
        got = got.view(np.float16).astype(np.float32)
    want = oracle.q4k_matmul(A16.astype(np.float32), W, M, N, K)
    if residual:
        want = want + res
    assert rel_l2(got, want) <= matmul_bar(M) + (5e-4 if outputDtype == "f16" else 0)
    # same rows handed over as f32 take the same kernels: identical bits
    same = ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(A16.astype(np.float32)), wb, M, N, K, outputDtype=outputDtype,
                                        role="test", residualTensor=ops.tensorFromNumpy(res) if residual else None))
    assert same.tobytes() == ops.readTensor(out).tobytes()


@pytest.mark.parametrize("M", [1, 4])
def test_matmul_f16_activations_at_an_odd_address(M):
    """Rows that start 2 bytes past an 8-byte boundary cannot be loaded four elements at a time: the
    library widens them first, and the product is the same."""
    import torch
    N, K = 4096, 4096
    W, wb = q4k_weight(N, K, 1170 + M)
    A16 = synth.normal_f32((M, K), 1171 + M).astype(np.float16)
    buf = torch.zeros(M * K + 8, dtype=torch.float16, device="cuda")
    buf[1:1 + M * K] = torch.from_numpy(A16.reshape(-1)).cuda()
    out = torch.zeros(M * N, dtype=torch.float32, device="cuda")
    capi.check(capi.init(0).dh_q4k_matmul(buf.data_ptr() + 2, capi.F16, wb.buffer.data_ptr(), out.data_ptr(), capi.F32,
                                          M, N, K, 1.0, None))
    capi.check(capi.init(0).dh_sync())
    want = oracle.q4k_matmul(A16.astype(np.float32), W, M, N, K)
    assert rel_l2(out.cpu().numpy().reshape(M, N), want) <= matmul_bar(M)


def test_matmul_f16_activations_errors():
    W, wb = q4k_weight(8, 256, 1160)
    a = ops.tensorFromNumpy(np.zeros((1, 256), np.float16).view(np.uint16))
    with pytest.raises(DopplerHipError, match="A buffer too small"):
        ops.runMatmul(a, wb, 2, 8, 256, outputDtype="f32")
    nw = ops.tensorFromNumpy(np.ones(256, np.float32))
    with pytest.raises(DopplerHipError, match="f16 activations"):
        ops.runMatmul(a, wb, 1, 8, 256, outputDtype="f32", normWeight=nw, rmsNormEps=1e-6, useFusedRmsnormWideTile=True)
    with pytest.raises(DopplerHipError, match="activations must be f32 or f16|a_dtype"):
        capi.check(capi.init(0).dh_q4k_matmul(a.buffer.data_ptr(), 7, wb.buffer.data_ptr(), a.buffer.data_ptr(), capi.F32,
                                              1, 8, 256, 1.0, None))


def test_matmul_cfg0_gemv():
    assert _matmul_case(1, synth.CFG0["N"], synth.CFG0["K"], seed=1100) <= REL_L2_F32


@pytest.mark.parametrize("name", sorted(synth.CFG1_SHAPES))
@pytest.mark.parametrize("M", [1, 2, 4, 8])
def test_matmul_cfg1_block_sweep(name, M):
    N, K = synth.CFG1_SHAPES[name]
    assert _matmul_case(M, N, K, seed=1200 + 10 * M + len(name)) <= REL_L2_F32


@pytest.mark.parametrize("M,N,K", [(1, 4096, 4096), (1, 1024, 4096), (1, 12288, 4096), (1, 4096, 12288),
                                   (3, 4096, 4096), (8, 1024, 12288),
                                   # four and eight activation rows per pass, and the LDS limits around them
                                   (4, 6144, 4096), (8, 4096, 4096), (2, 4096, 12288), (4, 2048, 12288),
                                   (6, 1024, 3072), (7, 512, 6144), (8, 1000, 2048), (5, 4096, 1024)])
def test_matmul_cfg4_shapes(M, N, K):
    assert _matmul_case(M, N, K, seed=1300 + M) <= REL_L2_F32


@pytest.mark.parametrize("M,N,K", [(1, 33, 256), (5, 7, 512), (3, 64, 1152), (2, 1000, 300), (1, 1, 256),
                                   (7, 129, 5120), (12, 96, 1152), (17, 40, 768)])
def test_matmul_ragged_shapes(M, N, K):
    assert _matmul_case(M, N, K, seed=1400 + M + N) <= matmul_bar(M)


def test_matmul_random_shape_sweep():
    """Seeded sweep over the dispatch boundaries: M across the 1/2/4/8-row GEMV passes and the GEMM
    threshold, K with and without a 256 tail and across the LDS limits of the passes, N off the
    tile sizes, with and without residual / alpha / f16 output."""
    g = synth.rng(1700)
    ks = [256, 300, 640, 1024, 1152, 2048, 2304, 3072, 4096, 4352, 6144, 6400, 8192, 12288]
    for t in range(48):
        M = int(g.choice([1, 2, 3, 4, 5, 6, 7, 8, 9, 15, 16, 17, 33, 64, 100]))
        K = int(g.choice(ks))
        N = int(g.choice([1, 7, 31, 32, 33, 64, 100, 129, 257, 500, 1000]))
        kw = {}
        if g.random() < 0.4:
            kw["residual"] = True
        if g.random() < 0.3:
            kw["alpha"] = 0.5
        if g.random() < 0.2:
            kw["outputDtype"] = "f16"
        bar = 2e-3 if kw.get("outputDtype") == "f16" else matmul_bar(M)
        assert _matmul_case(M, N, K, seed=1701 + t, **kw) <= max(bar, matmul_bar(M)), (M, N, K, kw)


@pytest.mark.parametrize("M,N,K,kw", [(512, 6912, 1152, {}), (512, 1152, 6912, dict(residual=True)),
                                      (130, 200, 640, dict(alpha=0.5)), (16, 128, 256, dict(outputDtype="f16")),
                                      (77, 129, 1000, {}), (300, 96, 300, {}),
                                      # long K, few tiles: the split-K path with its ordered reduction
                                      (64, 64, 4096, dict(alpha=0.5, outputDtype="f16", residual=True)),
                                      (100, 70, 8192, dict(residual=True))])
def test_matmul_prefill_gemm(M, N, K, kw):
    """Config-2 shapes (X[512,1152] against [6912,1152] and [1152,6912]) and ragged tiles."""
    assert _matmul_case(M, N, K, seed=1500 + M, **kw) <= REL_L2_F16_MFMA


@pytest.mark.parametrize("M,N,K,kw", [(1000, 8200, 320, dict(residual=True)), (1024, 8192, 256, dict(outputDtype="f16")),
                                      (2048, 4224, 192, dict(alpha=0.5))])
def test_matmul_prefill_gemm_tall_tiles(M, N, K, kw):
    """Enough 256 x 128 tiles to fill 256 compute units: the eight-wave tall-tile kernel, with ragged edges in M
    and N, an odd number of K steps and a K that ends inside a super-block."""
    assert -(-M // 256) * -(-N // 128) >= 256
    assert _matmul_case(M, N, K, seed=1560 + K, **kw) <= REL_L2_F16_MFMA


@pytest.mark.parametrize("M,hidden,inter,activation", [(1000, 320, 8200, "silu"), (1024, 256, 8192, "gelu")])
def test_fused_ffn_prefill_tall_tiles(M, hidden, inter, activation):
    """The fused gate/up pair on 256 x 128 x 2 tiles."""
    Wg, wg = q4k_weight(inter, hidden, seed=2410)
    Wu, wu = q4k_weight(inter, hidden, seed=2411)
    X = synth.normal_f32((M, hidden), seed=2412, scale=0.05)
    out = ops.runFusedFFN(ops.tensorFromNumpy(X), wg, wu, hidden, inter, batchSize=M, activation=activation)
    want = oracle.q4k_ffn_gate_up(X, Wg, Wu, M, hidden, inter, alpha=1.0, activation=activation)
    assert rel_l2(ops.readTensor(out), want) <= REL_L2_F16_MFMA


def test_matmul_prefill_gemm_activation_range():
    """Rows far outside the f16 range (and far below it) go through the f16 matrix-core path: each
    row is scaled by its own power of two before rounding."""
    M, N, K = 64, 192, 1024
    W, wb = q4k_weight(N, K, seed=1600)
    A = synth.normal_f32((M, K), seed=1601)
    A[::3] *= 1e7
    A[1::3] *= 1e-9
    A[5] = 0.0
    out = ops.runMatmul(ops.tensorFromNumpy(A), wb, M, N, K, outputDtype="f32", role="test")
    got = ops.readTensor(out).reshape(M, N)
    want = oracle.q4k_matmul(A, W, M, N, K).reshape(M, N)
    assert np.isfinite(got).all()
    for m in range(M):
        assert rel_l2(got[m], want[m]) <= REL_L2_F16_MFMA or not want[m].any(), m
    assert not got[5].any()


@pytest.mark.parametrize("M,activation", [(512, "gelu"), (48, "silu")])
def test_fused_ffn_prefill_cfg2(M, activation):
    hidden, inter = synth.CFG2["hidden"], synth.CFG2["inter"]
    Wg, wg = q4k_weight(inter, hidden, seed=2400)
    Wu, wu = q4k_weight(inter, hidden, seed=2401)
    X = synth.normal_f32((M, hidden), seed=2402, scale=0.05)
    out = ops.runFusedFFN(ops.tensorFromNumpy(X), wg, wu, hidden, inter, batchSize=M, activation=activation)
    want = oracle.q4k_ffn_gate_up(X, Wg, Wu, M, hidden, inter, alpha=1.0, activation=activation)
    assert rel_l2(ops.readTensor(out), want) <= REL_L2_F16_MFMA


def test_prefill_ffn_chain_cfg2():
    """Config 2 as ONE chain: X[512,1152] -> fused gate/up with the GELU gate -> down projection, the
    intermediate H staying on the device in f32, against the oracle's chain
    (tests/kernels/reference/fused-ffn-q4k.js:42-73 then the row-major product)."""
    M, hidden, inter = 512, synth.CFG2["hidden"], synth.CFG2["inter"]
    Wg, wg = q4k_weight(inter, hidden, seed=2420)
    Wu, wu = q4k_weight(inter, hidden, seed=2421)
    Wd, wd = q4k_weight(hidden, inter, seed=2422)
    X = synth.normal_f32((M, hidden), seed=2423, scale=0.05)
    H = ops.runFusedFFN(ops.tensorFromNumpy(X), wg, wu, hidden, inter, batchSize=M, activation="gelu")
    Y = ops.runMatmul(H, wd, M, hidden, inter, outputDtype="f32", role="ffn_down")
    want_h = oracle.q4k_ffn_gate_up(X, Wg, Wu, M, hidden, inter, alpha=1.0, activation="gelu")
    want_y = oracle.q4k_matmul(want_h.reshape(M, inter), Wd, M, hidden, inter)
    assert rel_l2(ops.readTensor(H), want_h) <= REL_L2_F16_MFMA
    assert rel_l2(ops.readTensor(Y), want_y) <= REL_L2_F16_MFMA
    # row by row as well: no row may hide behind the others
    got = ops.readTensor(Y).reshape(M, hidden)
    want = want_y.reshape(M, hidden)
    assert max(rel_l2(got[m], want[m]) for m in range(M)) <= 2 * REL_L2_F16_MFMA


def test_matmul_alpha_residual_f16_output():
    assert _matmul_case(2, 512, 1024, seed=1500, alpha=0.125, residual=True) <= REL_L2_F32
    assert _matmul_case(4, 512, 1024, seed=1510, alpha=2.0 ** -8, outputDtype="f16") <= 1e-3


def test_matmul_one_hot_returns_dequantized_column():
    N, K = 256, 1152
    W, wb = q4k_weight(N, K, seed=1600)
    Wd = oracle.q4k_dequant_rows(W, N, K)
    for k in (0, 31, 32, 255, 256, 1151):
        e = np.zeros((1, K), np.float32)
        e[0, k] = 1.0
        got = ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(e), wb, 1, N, K, outputDtype="f32"))
        assert np.array_equal(got, Wd[:, k]), k


def test_matmul_padded_tail_is_ignored():
    M, N, K = 2, 64, 640
    W = synth.q4k_tensor(N, K, seed=1700)
    A = synth.normal_f32((M, K), seed=1701)
    W2 = W.reshape(N, 3, 144).copy()
    W2[:, 2, 16 + 64:] ^= 0xFF        # k 640..767 of every row
    outs = []
    for w in (W, W2.reshape(-1)):
        buf = ops.acquireBuffer(w.size)
        ops.uploadData(buf, w)
        outs.append(ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(A), ops.createWeightBuffer(buf, "q4k", "row", (N, K)),
                                                 M, N, K, outputDtype="f32")))
    assert np.array_equal(outs[0], outs[1])


def test_matmul_errors_match_reference_behaviour():
    W, wb = q4k_weight(8, 256, seed=1800)
    a = ops.tensorFromNumpy(np.zeros((1, 256), np.float32))
    with pytest.raises(DopplerHipError, match="outputDtype is required"):
        ops.runMatmul(a, wb, 1, 8, 256)
    with pytest.raises(DopplerHipError, match="Dimensions must be positive"):
        ops.runMatmul(a, wb, 0, 8, 256, outputDtype="f32")
    with pytest.raises(DopplerHipError, match="B buffer too small"):
        ops.runMatmul(a, wb, 1, 9, 256, outputDtype="f32")
    with pytest.raises(DopplerHipError, match="A buffer too small"):
        ops.runMatmul(a, wb, 2, 8, 256, outputDtype="f32")
    with pytest.raises(DopplerHipError, match="B dtype is required"):
        ops.runMatmul(a, wb.buffer, 1, 8, 256, outputDtype="f32")


# ----------------------------------------------------------------------------- fused FFN gate/up

@pytest.mark.parametrize("M,activation,limit", [(1, "silu", None), (4, "silu", 7.0), (1, "gelu", None), (3, "gelu", None),
                                                (8, "silu", None), (6, "gelu", 3.0)])
def test_fused_ffn_q4k(M, activation, limit):
    hidden, inter = 1536, 6144          # the shape of the reference's fused-ffn-q4k parity test
    Wg, wg = q4k_weight(inter, hidden, seed=2000)
    Wu, wu = q4k_weight(inter, hidden, seed=2001)
    X = synth.normal_f32((M, hidden), seed=2002, scale=0.02)
    out = ops.runFusedFFN(ops.tensorFromNumpy(X), wg, wu, hidden, inter, batchSize=M, activation=activation,
                          alpha=0.5, swigluLimit=limit)
    want = oracle.q4k_ffn_gate_up(X, Wg, Wu, M, hidden, inter, alpha=0.5, activation=activation, swiglu_limit=limit or 0.0)
    assert rel_l2(ops.readTensor(out), want) <= REL_L2_F32


def test_fused_ffn_random_shape_sweep():
    """Seeded sweep of the fused gate/up product (plain and with the RMSNorm prologue) over batch
    sizes on both sides of every GEMV pass size and of the GEMM threshold, hidden sizes with and
    without a 256 tail, odd intermediate sizes, both activations."""
    g = synth.rng(2600)
    for t in range(24):
        M = int(g.choice([1, 2, 3, 4, 5, 8, 9, 16, 17, 40]))
        hidden = int(g.choice([256, 640, 1024, 1152, 2048, 4096, 4352]))
        inter = int(g.choice([64, 100, 257, 1000, 1536]))
        act = str(g.choice(["silu", "gelu"]))
        normed = g.random() < 0.5
        Wg, wg = q4k_weight(inter, hidden, seed=2601 + 3 * t)
        Wu, wu = q4k_weight(inter, hidden, seed=2602 + 3 * t)
        X = synth.normal_f32((M, hidden), seed=2603 + 3 * t, scale=0.05)
        if normed:
            nw = 1.0 + synth.normal_f32((hidden,), seed=2604 + t, scale=0.1)
            out = ops.runFusedNormedFFN(ops.tensorFromNumpy(X), ops.tensorFromNumpy(nw), 1e-6, wg, wu, hidden, inter,
                                        batchSize=M, activation=act)
            xin = oracle.rmsnorm(X, nw, 1e-6)
        else:
            out = ops.runFusedFFN(ops.tensorFromNumpy(X), wg, wu, hidden, inter, batchSize=M, activation=act)
            xin = X
        want = oracle.q4k_ffn_gate_up(xin, Wg, Wu, M, hidden, inter, alpha=1.0, activation=act)
        assert rel_l2(ops.readTensor(out), want) <= matmul_bar(M), (M, hidden, inter, act, normed)


@pytest.mark.parametrize("M,N,K,offset", [(1, 6144, 4096, False), (2, 1024, 1024, True), (1, 2048, 640, False),
                                          (3, 96, 1152, False), (1, 4096, 12288, False), (5, 130, 2048, True),
                                          (4, 1024, 4096, False), (8, 512, 2048, True), (7, 256, 4096, False),
                                          (2, 300, 12288, False), (2, 40, 20480, True), (1, 33, 28672, False)])
def test_matmul_with_rmsnorm_prologue(M, N, K, offset):
    """runMatmul with normWeight + useFusedRmsnormWideTile == runRMSNorm followed by runMatmul
    (reference: src/gpu/kernels/matmul-selection.js:609-620)."""
    W, wb = q4k_weight(N, K, seed=2100 + M)
    A = synth.normal_f32((M, K), seed=2101 + N, scale=3.0)
    nw = (0.0 if offset else 1.0) + synth.normal_f32((K,), seed=2102, scale=0.1)
    res = synth.normal_f32((M, N), seed=2103)
    out = ops.runMatmul(ops.tensorFromNumpy(A), wb, M, N, K, alpha=0.75, outputDtype="f32",
                        residualTensor=ops.tensorFromNumpy(res), normWeight=ops.tensorFromNumpy(nw),
                        rmsNormEps=1e-6, rmsNormOffset=offset, useFusedRmsnormWideTile=True)
    normed = oracle.rmsnorm(A, nw, 1e-6, weight_offset=offset)
    want = oracle.q4k_matmul(normed, W, M, N, K, 0.75) + res
    assert rel_l2(ops.readTensor(out), want) <= REL_L2_F32


@pytest.mark.parametrize("M,activation", [(1, "silu"), (2, "gelu"), (4, "silu"), (8, "gelu"), (5, "silu")])
def test_fused_normed_ffn_q4k(M, activation):
    hidden, inter = 1536, 6144
    Wg, wg = q4k_weight(inter, hidden, seed=2200)
    Wu, wu = q4k_weight(inter, hidden, seed=2201)
    X = synth.normal_f32((M, hidden), seed=2202, scale=5.0)
    nw = 1.0 + synth.normal_f32((hidden,), seed=2203, scale=0.1)
    out = ops.runFusedNormedFFN(ops.tensorFromNumpy(X), ops.tensorFromNumpy(nw), 1e-6, wg, wu, hidden, inter,
                                batchSize=M, activation=activation)
    normed = oracle.rmsnorm(X, nw, 1e-6)
    want = oracle.q4k_ffn_gate_up(normed, Wg, Wu, M, hidden, inter, alpha=1.0, activation=activation)
    assert rel_l2(ops.readTensor(out), want) <= REL_L2_F32


def test_rmsnorm_prologue_fails_closed_for_rows_too_long_for_the_gemm():
    K = 32768                                   # from 16 rows on the product is the GEMM's, whose prologue stops at 16384
    W, wb = q4k_weight(32, K, seed=2300)
    A = ops.tensorFromNumpy(synth.normal_f32((16, K), seed=2301))
    nw = ops.tensorFromNumpy(np.ones(K, np.float32))
    with pytest.raises(DopplerHipError, match="RMSNorm prologue"):
        ops.runMatmul(A, wb, 16, 32, K, outputDtype="f32", normWeight=nw, rmsNormEps=1e-6,
                      useFusedRmsnormWideTile=True)


@pytest.mark.parametrize("M,N,K", [(2, 32, 32768), (7, 40, 32768), (12, 33, 20480)])
def test_rmsnorm_prologue_long_rows_below_the_gemm_batch(M, N, K):
    """Up to 15 rows the few-row kernel converts the activations column by column: no limit on K."""
    W, wb = q4k_weight(N, K, seed=2310 + M)
    A = synth.normal_f32((M, K), seed=2311 + M, scale=2.0)
    nw = 1.0 + synth.normal_f32((K,), seed=2312 + M, scale=0.1)
    out = ops.runMatmul(ops.tensorFromNumpy(A), wb, M, N, K, outputDtype="f32", normWeight=ops.tensorFromNumpy(nw),
                        rmsNormEps=1e-6, useFusedRmsnormWideTile=True)
    want = oracle.q4k_matmul(oracle.rmsnorm(A, nw, 1e-6), W, M, N, K, 1.0)
    assert rel_l2(ops.readTensor(out), want) <= REL_L2_F32


@pytest.mark.parametrize("M", [9, 12, 15])
def test_rmsnorm_prologue_between_gemv_and_gemm_batches(M):
    """9..15 rows: two passes of the streaming GEMV."""
    N, K = 200, 1024
    W, wb = q4k_weight(N, K, seed=2305 + M)
    X = synth.normal_f32((M, K), seed=2306 + M, scale=2.0)
    nw = 1.0 + synth.normal_f32((K,), seed=2307 + M, scale=0.1)
    res = synth.normal_f32((M, N), seed=2308 + M)
    out = ops.runMatmul(ops.tensorFromNumpy(X), wb, M, N, K, outputDtype="f32", normWeight=ops.tensorFromNumpy(nw),
                        rmsNormEps=1e-6, useFusedRmsnormWideTile=True, residualTensor=ops.tensorFromNumpy(res))
    assert rel_l2(ops.readTensor(out), oracle.q4k_matmul(oracle.rmsnorm(X, nw, 1e-6), W, M, N, K) + res) <= REL_L2_F32
    out = ops.runMatmul(ops.tensorFromNumpy(X), wb, M, N, K, outputDtype="f32")
    assert rel_l2(ops.readTensor(out), oracle.q4k_matmul(X, W, M, N, K)) <= REL_L2_F32


def test_prefill_gemm_rejects_a_weight_tensor_its_descriptor_cannot_address():
    """From 16 rows on the kernel reaches a weight row through a 32-bit offset: 2 GB or more fails before any launch
    (so the small buffers handed over here are never touched)."""
    lib = capi.load()
    A = ops.tensorFromNumpy(np.zeros((16, 1024), np.float32))
    small = ops.tensorFromNumpy(np.zeros(1024, np.float32))
    N = 4_000_000                               # 4e6 rows x 4 blocks x 144 bytes = 2.3 GB
    rc = lib.dh_q4k_matmul(A.buffer.data_ptr(), 0, small.buffer.data_ptr(), small.buffer.data_ptr(), 0, 16, N, 1024, 1.0, None)
    assert rc != 0 and b"2 GB" in lib.dh_last_error()


@pytest.mark.parametrize("M,N,K", [(16, 300, 1024), (40, 512, 1152), (512, 1024, 4096), (130, 200, 12288), (33, 96, 640)])
def test_matmul_rmsnorm_prologue_on_the_gemm_path(M, N, K):
    """M >= 16: the rows are normalised while the GEMM's activations are packed."""
    W, wb = q4k_weight(N, K, seed=2310 + M)
    X = synth.normal_f32((M, K), seed=2311 + M, scale=3.0)
    nw = 1.0 + synth.normal_f32((K,), seed=2312 + M, scale=0.1)
    res = synth.normal_f32((M, N), seed=2313 + M)
    out = ops.runMatmul(ops.tensorFromNumpy(X), wb, M, N, K, outputDtype="f32", normWeight=ops.tensorFromNumpy(nw),
                        rmsNormEps=1e-6, useFusedRmsnormWideTile=True, residualTensor=ops.tensorFromNumpy(res))
    want = oracle.q4k_matmul(oracle.rmsnorm(X, nw, 1e-6), W, M, N, K) + res
    assert rel_l2(ops.readTensor(out), want) <= matmul_bar(M)
    # weights given as offsets from one, as Gemma-style checkpoints store them
    out = ops.runMatmul(ops.tensorFromNumpy(X), wb, M, N, K, outputDtype="f32", normWeight=ops.tensorFromNumpy(nw - 1.0),
                        rmsNormEps=1e-6, useFusedRmsnormWideTile=True, rmsNormOffset=True)
    assert rel_l2(ops.readTensor(out), want - res) <= matmul_bar(M)


def test_f16_weight_matmul_and_lmhead_argmax():
    vocab, hidden = 5000, 1024
    E = synth.normal_f16_bits((vocab, hidden), seed=3000, scale=0.02)
    h = synth.normal_f32((1, hidden), seed=3001)
    eb = ops.createWeightBuffer(ops.tensorFromNumpy(E).buffer, "f16", "row", (vocab, hidden))
    ht = ops.tensorFromNumpy(h)
    want = oracle.f16w_matmul(h, E, 1, vocab, hidden)
    got = ops.readTensor(ops.runMatmul(ht, eb, 1, vocab, hidden, outputDtype="f32"))
    assert rel_l2(got, want) <= REL_L2_F32
    logits = ops.acquireBuffer(vocab * 4)
    tok = ops.recordLmHeadArgmaxF16(None, ht, eb, vocabSize=vocab, hiddenSize=hidden, logitsOutput=logits)
    assert int(ops.readBuffer(tok, 4, np.uint32)[0]) == oracle.argmax(want[0])
    assert rel_l2(ops.readBuffer(logits, vocab * 4, np.float32), want) <= REL_L2_F32
    pad = oracle.argmax(want[0])
    tok = ops.recordLmHeadArgmaxF16(None, ht, eb, vocabSize=vocab, hiddenSize=hidden, padTokenId=pad, outputIndex=3,
                                    outputBuffer=ops.acquireBuffer(16))
    assert int(ops.readBuffer(tok, 16, np.uint32)[3]) == oracle.argmax(want[0], pad_id=pad)
    # the final RMSNorm inside the LM head kernel (w and 1 + w), against norm then product in the oracle
    nw = synth.normal_f32(hidden, seed=3003, scale=0.3)
    nwt = ops.tensorFromNumpy(nw)
    for offset in (False, True):
        hn = oracle.rmsnorm(h, nw, 1e-6, weight_offset=offset).reshape(1, hidden)
        want_n = oracle.f16w_matmul(hn, E, 1, vocab, hidden)
        tok = ops.recordLmHeadArgmaxF16(None, ht, eb, vocabSize=vocab, hiddenSize=hidden, logitsOutput=logits,
                                        normWeight=nwt, rmsNormEps=1e-6, rmsNormWeightOffset=offset)
        fused = ops.readBuffer(logits, vocab * 4, np.float32).copy()
        assert rel_l2(fused, want_n) <= REL_L2_F32
        assert int(ops.readBuffer(tok, 4, np.uint32)[0]) == oracle.argmax(want_n[0])
        # the same bits as the norm as a launch of its own in front of the plain call
        normed = ops.runRMSNorm(ht, nwt, 1e-6, batchSize=1, hiddenSize=hidden, rmsNormWeightOffset=offset)
        ops.recordLmHeadArgmaxF16(None, normed, eb, vocabSize=vocab, hiddenSize=hidden, logitsOutput=logits)
        assert np.array_equal(ops.readBuffer(logits, vocab * 4, np.float32), fused)
    assert ops.lmHeadArgmaxNormFusable(4096) and not ops.lmHeadArgmaxNormFusable(5120)
    big = ops.tensorFromNumpy(synth.normal_f32((1, 5120), seed=3004))
    with pytest.raises(ops.DopplerHipError, match="hidden <= 4096"):
        ops.recordLmHeadArgmaxF16(None, big, eb, vocabSize=1000, hiddenSize=5120, normWeight=ops.tensorFromNumpy(
            np.ones(5120, np.float32)), rmsNormEps=1e-6)
    # batched dense rows
    A = synth.normal_f32((5, hidden), seed=3002)
    got = ops.readTensor(ops.runMatmul(ops.tensorFromNumpy(A), eb, 5, vocab, hidden, outputDtype="f32"))
    assert rel_l2(got, oracle.f16w_matmul(A, E, 5, vocab, hidden)) <= REL_L2_F32


def test_argmax_exact_ties_pad_softcap():
    g = synth.rng(3100)
    for vocab in (1, 7, 256, 257, 151936):
        x = g.integers(-50, 50, vocab).astype(np.float32)      # many exact ties
        t = ops.tensorFromNumpy(x)
        assert ops.runArgmax(t, vocab) == oracle.argmax(x)
        pad = oracle.argmax(x)
        assert ops.runArgmax(t, vocab, padTokenId=pad) == oracle.argmax(x, pad_id=pad)
    x = synth.normal_f32(4096, seed=3101, scale=40.0)
    assert ops.runArgmax(ops.tensorFromNumpy(x), 4096, logitSoftcap=30.0) == oracle.argmax(x, softcap=30.0)


def test_gpu_sample_topk_matches_oracle():
    """runGPUSample against the sampler oracle (exact top-k, f64 softmax, inverse CDF): vocabulary
    sizes on both sides of one sort tile and at the 9B-class size, ties, top_k from 2 to 256."""
    g = synth.rng(7100)
    cases = [(64, 4), (1000, 40), (1024, 256), (1025, 7), (5000, 50), (151936, 40), (151936, 256), (151936, 2)]
    for ci, (V, k) in enumerate(cases):
        logits = (g.standard_normal(V) * 3).astype(np.float32)
        if ci % 2 == 1:
            logits = (np.round(logits * 4) / 4).astype(np.float32)        # exact ties everywhere
        lt = ops.tensorFromNumpy(logits)
        for T in (0.7, 1.0, 1.8):
            for seed in (1, 42, 977):
                r = ops.seededRandom(seed + ci)
                assert r == oracle.seeded_random(seed + ci)
                got = ops.runGPUSample(lt, V, temperature=T, topK=k, randomSeed=seed + ci)
                assert got == oracle.sample_topk(logits, T, k, r), (V, k, T, seed)
    # extremes of the uniform draw, pad id, greedy fallbacks
    V = 3000
    logits = (g.standard_normal(V) * 2).astype(np.float32)
    lt = ops.tensorFromNumpy(logits)
    order = np.argsort(-logits, kind="stable")
    assert ops.runGPUSample(lt, V, temperature=1.0, topK=5, randomValue=0.0) == int(order[0])
    assert ops.runGPUSample(lt, V, temperature=1.0, topK=5, randomValue=1.0) == oracle.sample_topk(logits, 1.0, 5, 1.0)
    assert ops.runGPUSample(lt, V, temperature=1.0, topK=5, randomValue=0.0, padTokenId=int(order[0])) == int(order[1])
    assert ops.runGPUSample(lt, V, temperature=0.001, topK=5, randomSeed=3) == int(order[0])
    assert ops.runGPUSample(lt, V, temperature=1.0, topK=1, randomSeed=3) == int(order[0])
    buf = ops.acquireBuffer(16)
    ops.runGPUSample(lt, V, temperature=1.0, topK=8, randomValue=0.3, outputBuffer=buf, outputIndex=2, readback=False)
    assert int(ops.readBuffer(buf, 16, np.uint32)[2]) == oracle.sample_topk(logits, 1.0, 8, 0.3)
    with pytest.raises(DopplerHipError, match="topK must be in 1..256"):
        ops.runGPUSample(lt, V, temperature=1.0, topK=300, randomSeed=1)
    with pytest.raises(DopplerHipError, match="randomSeed"):
        ops.runGPUSample(lt, V, temperature=1.0, topK=5)


def test_gather_f16_exact():
    vocab, hidden = 300, 640
    E = synth.normal_f16_bits((vocab, hidden), seed=3200, scale=0.02)
    ids = np.array([5, 299, 300, 0, 4000000000, 17], np.uint32)
    out = ops.runGather(ops.tensorFromNumpy(ids).buffer, ops.tensorFromNumpy(E).buffer, 4, hidden, vocab,
                        embeddingDtype="f16", outputDtype="f32", indexOffset=1)
    want = oracle.gather_f16(ids[1:5], E, hidden, vocab)
    assert np.array_equal(ops.readTensor(out).reshape(4, hidden), want)
    with pytest.raises(DopplerHipError, match="embeddingDtype is required"):
        ops.runGather(ops.tensorFromNumpy(ids).buffer, ops.tensorFromNumpy(E).buffer, 4, hidden, vocab)
    # f16 rows out (the reference's f16-activation plan): the stored bits, zeros for ids past the table
    out16 = ops.runGather(ops.tensorFromNumpy(ids).buffer, ops.tensorFromNumpy(E).buffer, 4, hidden, vocab,
                          embeddingDtype="f16", outputDtype="f16", indexOffset=1)
    assert out16.dtype == "f16"
    assert np.array_equal(ops.readTensor(out16).view(np.float16).reshape(4, hidden).astype(np.float32), want)


# ----------------------------------------------------------------------------- norm / rope / kv / elementwise

@pytest.mark.parametrize("hidden", [640, 1024, 1152, 4096, 100])
def test_rmsnorm_options(hidden):
    B = 3
    x = synth.normal_f32((B, hidden), seed=4000 + hidden, scale=3.0)
    w = synth.normal_f32(hidden, seed=4001, scale=0.1)
    r = synth.normal_f32((B, hidden), seed=4002)
    xt, wt, rt = ops.tensorFromNumpy(x), ops.tensorFromNumpy(w), ops.tensorFromNumpy(r)
    got = ops.readTensor(ops.runRMSNorm(xt, wt, 1e-6, batchSize=B, hiddenSize=hidden))
    assert rel_l2(got, oracle.rmsnorm(x, w, 1e-6)) <= 1e-5
    got = ops.readTensor(ops.runRMSNorm(xt, wt, 1e-6, batchSize=B, hiddenSize=hidden, rmsNormWeightOffset=True,
                                        residual=rt, outputScale=0.5))
    assert rel_l2(got, oracle.rmsnorm(x, w, 1e-6, weight_offset=True, post_residual=r, output_scale=0.5)) <= 1e-5
    pre_out = ops.acquireBuffer(B * hidden * 4)
    got = ops.readTensor(ops.runRMSNorm(xt, wt, 1e-6, batchSize=B, hiddenSize=hidden, preResidual=rt,
                                        residualSumOutput=pre_out))
    want, want_pre = oracle.rmsnorm(x, w, 1e-6, pre_residual=r, want_prenorm=True)
    assert rel_l2(got, want) <= 1e-5
    assert np.array_equal(ops.readBuffer(pre_out, B * hidden * 4, np.float32).reshape(B, hidden), want_pre)
    w16 = w.astype(np.float16)
    got = ops.readTensor(ops.runRMSNorm(xt, ops.tensorFromNumpy(w16.view(np.uint16), "f16"), 1e-6, batchSize=B, hiddenSize=hidden))
    assert rel_l2(got, oracle.rmsnorm(x, w16.astype(np.float32), 1e-6)) <= 1e-5


@pytest.mark.parametrize("T,H,Hkv,D,offset", [(3, 16, 8, 128, False), (1, 32, 8, 128, True), (5, 4, 2, 64, False),
                                              (2, 3, 1, 80, True)])
def test_rmsnorm_qk_one_launch(T, H, Hkv, D, offset):
    """Per-head RMSNorm of q and k together (rmsnorm-qk.js): equals the oracle's RMSNorm row by row, f32 and f16 weights."""
    q = synth.normal_f32((T * H, D), seed=4100 + D, scale=2.0)
    k = synth.normal_f32((T * Hkv, D), seed=4101 + D, scale=0.5)
    qw = synth.normal_f32(D, seed=4102, scale=0.1) + (0.0 if offset else 1.0)
    kw16 = (synth.normal_f32(D, seed=4103, scale=0.1) + (0.0 if offset else 1.0)).astype(np.float16)
    qt, kt = ops.tensorFromNumpy(q), ops.tensorFromNumpy(k)
    assert ops.canUseRMSNormQK(qt, kt) and not ops.canUseRMSNormQK(qt, qt) and not ops.canUseRMSNormQK(qt, kt, skipKNorm=True)
    r = ops.runRMSNormQK(qt, kt, ops.tensorFromNumpy(qw), ops.tensorFromNumpy(kw16.view(np.uint16), "f16"), 1e-6,
                         numTokens=T, numHeads=H, numKVHeads=Hkv, headDim=D, rmsNormWeightOffset=offset)
    assert r["q"].shape == (T * H, D) and r["k"].shape == (T * Hkv, D)
    assert rel_l2(ops.readTensor(r["q"]), oracle.rmsnorm(q, qw, 1e-6, weight_offset=offset)) <= 1e-5
    assert rel_l2(ops.readTensor(r["k"]), oracle.rmsnorm(k, kw16.astype(np.float32), 1e-6, weight_offset=offset)) <= 1e-5
    # the inputs are left alone
    assert np.array_equal(ops.readTensor(qt), q.reshape(-1)) or np.array_equal(ops.readTensor(qt).reshape(q.shape), q)
    with pytest.raises(DopplerHipError, match="positive integer numHeads"):
        ops.runRMSNormQK(qt, kt, ops.tensorFromNumpy(qw), ops.tensorFromNumpy(qw), 1e-6, numTokens=T, numHeads=0,
                         numKVHeads=Hkv, headDim=D)
    with pytest.raises(DopplerHipError, match="Q input buffer"):
        ops.runRMSNormQK(qt, kt, ops.tensorFromNumpy(qw), ops.tensorFromNumpy(qw), 1e-6, numTokens=T + 1, numHeads=H,
                         numKVHeads=Hkv, headDim=D)


@pytest.mark.parametrize("hidden,B,with_residual,offset", [(1152, 3, True, True), (4096, 2, False, False), (100, 5, True, False)])
def test_rmsnorm_sandwich_pair(hidden, B, with_residual, offset):
    """rmsnorm-pair.js sandwich form: post = residual + rmsnorm(x, w_post), pre = rmsnorm(post, w_pre)."""
    x = synth.normal_f32((B, hidden), seed=4200 + hidden, scale=3.0)
    r = synth.normal_f32((B, hidden), seed=4201)
    wp = synth.normal_f32(hidden, seed=4202, scale=0.1) + (0.0 if offset else 1.0)
    wq16 = (synth.normal_f32(hidden, seed=4203, scale=0.1) + (0.0 if offset else 1.0)).astype(np.float16)
    out = ops.runSandwichRMSNormPair(ops.tensorFromNumpy(x), ops.tensorFromNumpy(r) if with_residual else None,
                                     ops.tensorFromNumpy(wp), ops.tensorFromNumpy(wq16.view(np.uint16), "f16"), 1e-6,
                                     batchSize=B, hiddenSize=hidden, rmsNormWeightOffset=offset)
    want_post = oracle.rmsnorm(x, wp, 1e-6, weight_offset=offset, post_residual=r if with_residual else None)
    want_pre = oracle.rmsnorm(want_post.reshape(B, hidden), wq16.astype(np.float32), 1e-6, weight_offset=offset)
    assert rel_l2(ops.readTensor(out["postAttn"]), want_post) <= 1e-5
    assert rel_l2(ops.readTensor(out["ffnInput"]), want_pre) <= 1e-5


@pytest.mark.parametrize("hidden,B,scale", [(1152, 3, 1.0), (4096, 1, 0.5), (100, 4, 2.0)])
def test_residual_next_rmsnorm_pair(hidden, B, scale):
    """rmsnorm-pair.js residual-next form: residual = (x + r) * scale (bit exact), next = rmsnorm(residual, w)."""
    x = synth.normal_f32((B, hidden), seed=4300 + hidden, scale=2.0)
    r = synth.normal_f32((B, hidden), seed=4301)
    w = synth.normal_f32(hidden, seed=4302, scale=0.1)
    out = ops.runResidualNextRMSNormPair(ops.tensorFromNumpy(x), ops.tensorFromNumpy(r), ops.tensorFromNumpy(w), 1e-6,
                                         batchSize=B, hiddenSize=hidden, rmsNormWeightOffset=True, outputScale=scale)
    want_res = ((x + r) * np.float32(scale)).astype(np.float32)
    assert np.array_equal(ops.readTensor(out["residual"]).reshape(B, hidden), want_res)
    assert rel_l2(ops.readTensor(out["nextInput"]), oracle.rmsnorm(want_res, w, 1e-6, weight_offset=True)) <= 1e-5
    with pytest.raises(DopplerHipError, match="outputScale must be finite"):
        ops.runResidualNextRMSNormPair(ops.tensorFromNumpy(x), ops.tensorFromNumpy(r), ops.tensorFromNumpy(w), 1e-6,
                                       batchSize=B, hiddenSize=hidden, outputScale=float("inf"))


def test_rope_variants():
    S, H, D, start = 5, 16, 128, 32000
    cos, sin = synth.rope_tables(D, start + S, 1e6)
    x = synth.normal_f32((S, H, D), seed=4100)
    ct, st = ops.tensorFromNumpy(cos), ops.tensorFromNumpy(sin)
    xt = ops.tensorFromNumpy(x)
    out = ops.runRoPE(xt, ct, st, S, numHeads=H, headDim=D, startPos=start)
    assert out.buffer is xt.buffer
    assert rel_l2(ops.readTensor(out), oracle.rope_apply(x, cos, sin, S, H, D, start)) <= 1e-6
    got = ops.readTensor(ops.runRoPE(ops.tensorFromNumpy(x), ct, st, S, numHeads=H, headDim=D, startPos=start, interleaved=True))
    assert rel_l2(got, oracle.rope_apply(x, cos, sin, S, H, D, start, interleaved=True)) <= 1e-6
    c32, s32 = synth.rope_tables(32, start + S, 1e4)
    for span in (32, 128):
        got = ops.readTensor(ops.runRoPE(ops.tensorFromNumpy(x), ops.tensorFromNumpy(c32), ops.tensorFromNumpy(s32), S,
                                         numHeads=H, headDim=D, rotaryDim=32, pairSpanDim=span, startPos=start))
        assert rel_l2(got, oracle.rope_apply(x, c32, s32, S, H, D, start, rotary_dim=32, pair_span_dim=span)) <= 1e-6
    with pytest.raises(DopplerHipError, match="rotaryDim must be even"):
        ops.runRoPE(xt, ct, st, S, numHeads=H, headDim=D, rotaryDim=31)
    # f16 activations (src/gpu/kernels/rope.js:44-63): rotated in f32, rounded to f16 once, in place
    x16 = x.astype(np.float16)
    t16 = ops.tensorFromNumpy(x16)
    out16 = ops.runRoPE(t16, ct, st, S, numHeads=H, headDim=D, startPos=start)
    assert out16.buffer is t16.buffer and out16.dtype == "f16"
    want16 = oracle.rope_apply(x16.astype(np.float32), cos, sin, S, H, D, start).reshape(-1)
    got16 = ops.readTensor(out16).view(np.float16).astype(np.float32)
    assert np.max(np.abs(got16 - want16) / np.maximum(np.abs(want16), 1e-3)) <= 2 ** -10


def test_rope_qk_one_launch_equals_two_single_buffer_calls():
    """rope-qk.js: q and k rotated by one launch; bit-identical to runRoPE on each buffer, oracle-close."""
    S, H, Hkv, D, start = 3, 16, 8, 128, 2047
    cos, sin = synth.rope_tables(D, start + S, 1e6)
    c32, s32 = synth.rope_tables(32, start + S, 1e4)
    q, k = synth.normal_f32((S, H, D), seed=4150), synth.normal_f32((S, Hkv, D), seed=4151)
    for tables, kw in (((cos, sin), {}), ((cos, sin), {"interleaved": True}),
                       ((c32, s32), {"rotaryDim": 32, "pairSpanDim": 128})):
        ct, st = ops.tensorFromNumpy(tables[0]), ops.tensorFromNumpy(tables[1])
        qt, kt = ops.tensorFromNumpy(q), ops.tensorFromNumpy(k)
        assert ops.canUseRoPEQK(qt, kt) and not ops.canUseRoPEQK(qt, qt)
        out = ops.runRoPEQK(qt, kt, ct, st, S, numQHeads=H, numKVHeads=Hkv, headDim=D, startPos=start, **kw)
        assert out["q"].buffer is qt.buffer and out["k"].buffer is kt.buffer
        one_q = ops.readTensor(ops.runRoPE(ops.tensorFromNumpy(q), ct, st, S, numHeads=H, headDim=D, startPos=start, **kw))
        one_k = ops.readTensor(ops.runRoPE(ops.tensorFromNumpy(k), ct, st, S, numHeads=Hkv, headDim=D, startPos=start, **kw))
        assert np.array_equal(ops.readTensor(out["q"]), one_q) and np.array_equal(ops.readTensor(out["k"]), one_k)
        okw = {"interleaved": kw.get("interleaved", False)}
        if "rotaryDim" in kw:
            okw.update(rotary_dim=32, pair_span_dim=128)
        assert rel_l2(ops.readTensor(out["q"]), oracle.rope_apply(q, tables[0], tables[1], S, H, D, start, **okw)) <= 1e-6
        assert rel_l2(ops.readTensor(out["k"]), oracle.rope_apply(k, tables[0], tables[1], S, Hkv, D, start, **okw)) <= 1e-6
    qt, kt = ops.tensorFromNumpy(q), ops.tensorFromNumpy(k)
    ops.runRoPEQK(qt, kt, ct, st, 0, numQHeads=H, numKVHeads=Hkv, headDim=D)       # seqLen 0: nothing is touched
    assert np.array_equal(ops.readTensor(qt).reshape(q.shape), q)
    with pytest.raises(DopplerHipError, match="pairSpanDim must be in"):
        ops.runRoPEQK(qt, kt, ct, st, S, numQHeads=H, numKVHeads=Hkv, headDim=D, rotaryDim=64, pairSpanDim=32)
    with pytest.raises(DopplerHipError, match="numKVHeads to be a positive integer"):
        ops.runRoPEQK(qt, kt, ct, st, S, numQHeads=H, numKVHeads=0, headDim=D)
    with pytest.raises(DopplerHipError, match="cos frequencies buffer is smaller"):
        ops.runRoPEQK(qt, kt, ct, st, S, numQHeads=H, numKVHeads=Hkv, headDim=D, startPos=start + 1)


def test_kv_cache_write_bit_exact():
    n = 8 * 128 * 3
    k = synth.normal_f32(n + 64, seed=4200)
    v = synth.normal_f32(n + 64, seed=4201)
    k[64:70] = [65504.0, 65520.0, 1e-8, 2.0 ** -24, 1.0 + 2.0 ** -11, -(1.0 + 3 * 2.0 ** -11)]   # overflow, underflow, ties
    ck, cv = ops.acquireBuffer(4096 * 2 * 2), ops.acquireBuffer(4096 * 2 * 2)
    ops.runKVCacheWriteF32ToF16(ops.tensorFromNumpy(k).buffer, ops.tensorFromNumpy(v).buffer, ck, cv,
                                srcOffset=64, dstOffset=1024, elementCount=n)
    wk, wv = np.zeros(8192, np.uint16), np.zeros(8192, np.uint16)
    oracle.kv_write_f16(k, v, wk, wv, 64, 1024, n)
    assert np.array_equal(ops.readBuffer(ck, dtype=np.uint16), wk)
    assert np.array_equal(ops.readBuffer(cv, dtype=np.uint16), wv)
    with pytest.raises(DopplerHipError, match="smaller than requested range"):
        ops.runKVCacheWriteF32ToF16(ops.tensorFromNumpy(k).buffer, ops.tensorFromNumpy(v).buffer, ck, cv,
                                    srcOffset=0, dstOffset=8000, elementCount=n)


@pytest.mark.parametrize("T,H,Hkv,D", [(1, 32, 8, 128), (3, 16, 8, 128), (2, 4, 2, 64)])
def test_split_qkv_rmsnorm_rope_kvwrite(T, H, Hkv, D):
    start, max_seq = 37, 64
    cos, sin = synth.rope_tables(D, max_seq, 1e6)
    qkv = synth.normal_f32((T, (H + 2 * Hkv) * D), seed=4300)
    qw = 1 + synth.normal_f32(D, seed=4301, scale=0.1)
    kw = 1 + synth.normal_f32(D, seed=4302, scale=0.1)
    ck, cv = ops.acquireBuffer(max_seq * Hkv * D * 2), ops.acquireBuffer(max_seq * Hkv * D * 2)
    res = ops.runSplitQKVRMSNormRoPEQK(ops.tensorFromNumpy(qkv), ops.tensorFromNumpy(qw), ops.tensorFromNumpy(kw),
                                       ops.tensorFromNumpy(cos), ops.tensorFromNumpy(sin), 1e-6, numTokens=T,
                                       numHeads=H, numKVHeads=Hkv, headDim=D, qSize=H * D, kSize=Hkv * D, vSize=Hkv * D,
                                       startPos=start,
                                       f16KVCacheWrite=dict(keysBuffer=ck, valuesBuffer=cv, dstOffset=start * Hkv * D))
    assert res["wroteF16KVCache"] and res["K"] is None
    wk = np.zeros((max_seq, Hkv, D), np.uint16)
    wv = np.zeros((max_seq, Hkv, D), np.uint16)
    want_q = oracle.qkv_norm_rope_kvwrite(qkv, qw, kw, cos, sin, T, H, Hkv, D, start, wk, wv, start * Hkv * D)
    assert rel_l2(ops.readTensor(res["Q"]), want_q) <= 1e-5
    got_k = ops.readBuffer(ck, dtype=np.uint16).reshape(max_seq, Hkv, D)
    # V is a pure narrowing: exact.  K goes through fp32 norm+rotation before rounding: values may
    # differ from the f64 oracle by one f16 ulp at rounding boundaries.
    assert np.array_equal(ops.readBuffer(cv, dtype=np.uint16).reshape(max_seq, Hkv, D), wv)
    assert not got_k[:start].any() and not got_k[start + T:].any()
    gk, ek = got_k.view(np.float16).astype(np.float64), wk.view(np.float16).astype(np.float64)
    assert rel_l2(gk, ek) <= 5e-4
    assert np.mean(got_k != wk) < 0.02


def test_bias_add_and_scale_bit_exact():
    """residual.js runBiasAdd (in place, byte offsets, f32 or f16 bias) and scale.js runScale: one IEEE add or
    multiply per element, so the f32 results are fixed bit for bit."""
    T, dim = 5, 1536
    x = synth.normal_f32((T + 1, dim), seed=4450, scale=3.0)
    bias = synth.normal_f32((2, dim), seed=4451)
    xt = ops.tensorFromNumpy(x)
    out = ops.runBiasAdd(xt, ops.tensorFromNumpy(bias), T, dim, dataOffset=dim * 4, biasOffset=dim * 4)
    assert out.buffer is xt.buffer and tuple(out.shape) == (T, dim)
    want = x.copy()
    want[1:] += bias[1]
    assert np.array_equal(ops.readTensor(xt).reshape(T + 1, dim), want)
    b16 = bias[0].astype(np.float16)
    xt = ops.tensorFromNumpy(x)
    ops.runBiasAdd(xt, ops.tensorFromNumpy(b16.view(np.uint16), "f16"), T + 1, dim)
    assert np.array_equal(ops.readTensor(xt).reshape(T + 1, dim), x + b16.astype(np.float32))
    with pytest.raises(DopplerHipError, match="data buffer is smaller"):
        ops.runBiasAdd(xt, ops.tensorFromNumpy(bias), T + 2, dim)
    s = np.float32(1536 ** 0.5)
    xt = ops.tensorFromNumpy(x)
    assert np.array_equal(ops.readTensor(ops.runScale(xt, float(s))).reshape(x.shape), x * s)
    part = ops.runScale(xt, 0.3, count=dim)
    assert np.array_equal(ops.readTensor(part).reshape(-1)[:dim], x[0] * np.float32(0.3))
    same = ops.runScale(xt, float(s), inplace=True)
    assert same.buffer is xt.buffer and np.array_equal(ops.readTensor(xt).reshape(x.shape), x * s)


def test_split_qkv_exact():
    """split_qkv.js: a pure copy, so every output element equals its source bit for bit."""
    T, qs, ks, vs = 7, 2048, 512, 384
    x = synth.normal_f32((T, qs + ks + vs), seed=4460)
    out = ops.runSplitQKV(ops.tensorFromNumpy(x), numTokens=T, qSize=qs, kSize=ks, vSize=vs)
    assert np.array_equal(ops.readTensor(out["Q"]).reshape(T, qs), x[:, :qs])
    assert np.array_equal(ops.readTensor(out["K"]).reshape(T, ks), x[:, qs:qs + ks])
    assert np.array_equal(ops.readTensor(out["V"]).reshape(T, vs), x[:, qs + ks:])
    mine = ops.tensorFromNumpy(np.zeros((T, ks), np.float32))
    again = ops.runSplitQKV(ops.tensorFromNumpy(x), numTokens=T, qSize=qs, kSize=ks, vSize=vs, kTensor=mine)
    assert again["K"] is mine and np.array_equal(ops.readTensor(mine).reshape(T, ks), x[:, qs:qs + ks])
    with pytest.raises(DopplerHipError, match="qkv buffer is smaller"):
        ops.runSplitQKV(ops.tensorFromNumpy(x), numTokens=T + 1, qSize=qs, kSize=ks, vSize=vs)


def test_residual_and_gated_activations():
    n = 12288
    a, b = synth.normal_f32(n, seed=4400, scale=4.0), synth.normal_f32(n, seed=4401)
    at, bt = ops.tensorFromNumpy(a), ops.tensorFromNumpy(b)
    assert np.array_equal(ops.readTensor(ops.runResidualAdd(at, bt, n)), oracle.residual_add(a, b))
    assert rel_l2(ops.readTensor(ops.runResidualAdd(at, bt, n, outputScale=0.25)), oracle.residual_add(a, b, 0.25)) <= 1e-7
    assert rel_l2(ops.readTensor(ops.runSiLU(bt, size=n, gate=at)), oracle.act_gate(a, b, "silu")) <= 1e-5
    assert rel_l2(ops.readTensor(ops.runSiLU(bt, size=n, gate=at, swigluLimit=0.5)), oracle.act_gate(a, b, "silu", 0.5)) <= 1e-5
    assert rel_l2(ops.readTensor(ops.runGeLU(bt, size=n, gate=at)), oracle.act_gate(a, b, "gelu")) <= 1e-5
    x = synth.normal_f32((4, 2 * 768), seed=4402, scale=3.0)
    for act in ("silu", "gelu"):
        got = ops.readTensor(ops.runSiLURowSplit(ops.tensorFromNumpy(x), numTokens=4, dim=768, activation=act))
        assert rel_l2(got, oracle.act_gate_rowsplit(x, 4, 768, act)) <= 1e-5


# ----------------------------------------------------------------------------- decode attention

def _attn_inputs(H, Hkv, D, ctx, seed, theta=1e6):
    """Config-3 recipe: N(0,1)/sqrt(D) values, RoPE applied to Q at ctx-1 and to K row p at p,
    then K, V and Q rounded to f16 (Q widened back to f32)."""
    cos, sin = synth.rope_tables(D, ctx, theta)
    q = synth.normal_f32((1, H, D), seed, D ** -0.5)
    k = synth.normal_f32((ctx, Hkv, D), seed + 1, D ** -0.5)
    v = synth.normal_f32((ctx, Hkv, D), seed + 2, D ** -0.5)
    q = oracle.rope_apply(q, cos, sin, 1, H, D, start_pos=ctx - 1)
    k = oracle.rope_apply(k, cos, sin, ctx, Hkv, D, start_pos=0)
    qf = q.astype(np.float16).astype(np.float32).reshape(H, D)
    return qf, k.astype(np.float16).view(np.uint16), v.astype(np.float16).view(np.uint16)


@pytest.mark.parametrize("ctx", [1, 63, 512, 4096, 32768])
def test_attention_decode_cfg3(ctx):
    H, Hkv, D = synth.CFG3["H"], synth.CFG3["Hkv"], synth.CFG3["D"]
    q, kb, vb = _attn_inputs(H, Hkv, D, ctx, seed=5000 + ctx)
    out = ops.runAttention(ops.tensorFromNumpy(q), ops.tensorFromNumpy(kb), ops.tensorFromNumpy(vb), None, H, D,
                           seqLen=1, kvLen=ctx, numKVHeads=Hkv, causal=True, startPos=ctx - 1)
    assert out.shape == (1, H, D)
    want = oracle.attention_decode_f16kv(q, kb, vb, H, Hkv, D, ctx)
    assert rel_l2(ops.readTensor(out), want) <= REL_L2_F32
    if ctx == 512:
        # f16 Q in, f16 out (the reference's *_f16 variants): the f32 result of the f16-rounded query, rounded once
        q16 = q.astype(np.float16)
        out16 = ops.runAttention(ops.tensorFromNumpy(q16), ops.tensorFromNumpy(kb), ops.tensorFromNumpy(vb), None, H, D,
                                 seqLen=1, kvLen=ctx, numKVHeads=Hkv, causal=True, startPos=ctx - 1)
        assert out16.dtype == "f16" and out16.shape == (1, H, D)
        want16 = oracle.attention_decode_f16kv(q16.astype(np.float32), kb, vb, H, Hkv, D, ctx)
        assert rel_l2(ops.readTensor(out16).view(np.float16).astype(np.float32), want16) <= 1e-3


def test_attention_decode_key_count_on_the_device():
    """runAttention's kvLenBuffer (src/gpu/kernels/attention.js:1071,1224-1232; kv_len_source == 1 in
    attention_decode_online_f16kv.wgsl:55-58): the kernels read the key count from a device word.
    Counts on both sides of every 64-key chunk boundary and of the point where the split count
    changes, against the oracle; the same launch arguments serve every count."""
    import torch
    H, Hkv, D, cap = 32, 8, 128, 4400
    q, kb, vb = _attn_inputs(H, Hkv, D, cap, seed=5050)
    qt, kt, vt = ops.tensorFromNumpy(q), ops.tensorFromNumpy(kb), ops.tensorFromNumpy(vb)
    word = torch.zeros(4, dtype=torch.int32, device="cuda")
    for n in (1, 2, 63, 64, 65, 128, 129, 2047, 2048, 2049, 2112, 2113, 4095, 4097, cap):
        word[0] = n
        torch.cuda.synchronize()
        got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, seqLen=1, kvLen=cap, numKVHeads=Hkv, causal=True,
                                              startPos=-1, kvLenBuffer=word))
        want = oracle.attention_decode_f16kv(q, kb, vb, H, Hkv, D, n)
        assert rel_l2(got, want) <= REL_L2_F32, n
        # identical to the launch that gets the count as an argument
        same = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, seqLen=1, kvLen=n, numKVHeads=Hkv, causal=True,
                                               startPos=n - 1))
        assert rel_l2(got, same) <= 1e-6, n
    # a fixed query position below the key count: the causal mask hides the keys behind it
    word[0] = 3000
    torch.cuda.synchronize()
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, kvLen=cap, numKVHeads=Hkv, startPos=700, kvLenBuffer=word))
    assert rel_l2(got, oracle.attention_decode_f16kv(q, kb, vb, H, Hkv, D, 3000, start_pos=700)) <= REL_L2_F32
    # sliding window follows the position
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, kvLen=cap, numKVHeads=Hkv, startPos=-1, slidingWindow=200,
                                          kvLenBuffer=word))
    assert rel_l2(got, oracle.attention_decode_f16kv(q, kb, vb, H, Hkv, D, 3000, sliding_window=200)) <= REL_L2_F32
    # no key: zeros; a count beyond the bound is clamped to it
    word[0] = 0
    torch.cuda.synchronize()
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, kvLen=cap, numKVHeads=Hkv, startPos=-1, kvLenBuffer=word))
    assert not got.any()
    word[0] = cap + 100000
    torch.cuda.synchronize()
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, kvLen=cap, numKVHeads=Hkv, startPos=-1, kvLenBuffer=word))
    assert rel_l2(got, oracle.attention_decode_f16kv(q, kb, vb, H, Hkv, D, cap)) <= REL_L2_F32
    with pytest.raises(DopplerHipError, match="decode"):
        ops.runAttention(qt, kt, vt, None, H, D, seqLen=2, kvLen=cap, numKVHeads=Hkv, kvLenBuffer=word)


@pytest.mark.parametrize("H,Hkv,D", [(32, 8, 128), (8, 8, 128), (8, 1, 64), (6, 2, 64)])
def test_attention_decode_head_geometries(H, Hkv, D):
    ctx = 777
    q, kb, vb = _attn_inputs(H, Hkv, D, ctx, seed=5100 + H)
    out = ops.runAttention(ops.tensorFromNumpy(q), ops.tensorFromNumpy(kb), ops.tensorFromNumpy(vb), None, H, D,
                           kvLen=ctx, numKVHeads=Hkv, startPos=ctx - 1)
    assert rel_l2(ops.readTensor(out), oracle.attention_decode_f16kv(q, kb, vb, H, Hkv, D, ctx)) <= REL_L2_F32


def test_attention_decode_options():
    H, Hkv, D, ctx = 16, 8, 128, 1500
    q, kb, vb = _attn_inputs(H, Hkv, D, ctx, seed=5200)
    qt, kt, vt = ops.tensorFromNumpy(q * 20), ops.tensorFromNumpy(kb), ops.tensorFromNumpy(vb)
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, kvLen=ctx, numKVHeads=Hkv, startPos=ctx - 1,
                                          scale=0.3, attnSoftcap=4.0))
    assert rel_l2(got, oracle.attention_decode_f16kv(q * 20, kb, vb, H, Hkv, D, ctx, scale=0.3, softcap=4.0)) <= REL_L2_F32
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, kvLen=ctx, numKVHeads=Hkv, startPos=ctx - 1,
                                          slidingWindow=200))
    assert rel_l2(got, oracle.attention_decode_f16kv(q * 20, kb, vb, H, Hkv, D, ctx, sliding_window=200)) <= REL_L2_F32
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, kvLen=ctx, numKVHeads=Hkv, startPos=700))
    assert rel_l2(got, oracle.attention_decode_f16kv(q * 20, kb, vb, H, Hkv, D, ctx, start_pos=700)) <= REL_L2_F32
    # ring layout, window 256
    win = 256
    ring_k = np.zeros((win, Hkv, D), np.uint16)
    ring_v = np.zeros((win, Hkv, D), np.uint16)
    kk, vv = kb.reshape(ctx, Hkv, D), vb.reshape(ctx, Hkv, D)
    for pos in range(ctx):
        ring_k[pos % win], ring_v[pos % win] = kk[pos], vv[pos]
    got = ops.readTensor(ops.runAttention(qt, ops.tensorFromNumpy(ring_k), ops.tensorFromNumpy(ring_v), None, H, D,
                                          kvLen=win, numKVHeads=Hkv, startPos=ctx - 1, slidingWindow=win,
                                          kvStart=ctx - win, kvLayout="ring"))
    want = oracle.attention_decode_f16kv(q * 20, ring_k, ring_v, H, Hkv, D, win, sliding_window=win, kv_start=ctx - win,
                                         kv_layout=1, start_pos=ctx - 1)
    assert rel_l2(got, want) <= REL_L2_F32
    # nothing visible -> zeros
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, kvLen=0, numKVHeads=Hkv, startPos=0))
    assert not got.any()
    with pytest.raises(DopplerHipError, match="kvLayout"):
        ops.runAttention(qt, kt, vt, None, H, D, kvLen=ctx, numKVHeads=Hkv, kvLayout="paged")


# ------------------------------------------------- decode attention straight from the stacked q/k/v

def _fused_case(H, Hkv, D, pos, seed, rotary=None, interleaved=False, window=0, ring=False, softcap=0.0,
                weight_offset=False):
    """History of `pos` cached rows, then one step at `pos` through the fused entry point; checks the
    attention output and the appended cache row against the oracle's two separate ops."""
    rotary = rotary or D
    max_seq = pos + 1
    cos, sin = synth.rope_tables(rotary, max_seq, 1e6)
    rows = window if ring else max_seq
    hist_k = synth.normal_f32((max_seq, Hkv, D), seed, D ** -0.5).astype(np.float16).view(np.uint16)
    hist_v = synth.normal_f32((max_seq, Hkv, D), seed + 1, D ** -0.5).astype(np.float16).view(np.uint16)
    ck = np.zeros((rows, Hkv, D), np.uint16)
    cv = np.zeros((rows, Hkv, D), np.uint16)
    for p_ in range(max(0, pos - rows), pos):
        ck[p_ % rows], cv[p_ % rows] = hist_k[p_], hist_v[p_]
    new_row = pos % rows
    ck[new_row], cv[new_row] = 0x7E00, 0x7E00          # stale NaN where the new row goes: must never be used
    qkv = synth.normal_f32((1, (H + 2 * Hkv) * D), seed + 2)
    qw = 1 + synth.normal_f32(D, seed + 3, scale=0.1) - (1.0 if weight_offset else 0.0)
    kw = 1 + synth.normal_f32(D, seed + 4, scale=0.1) - (1.0 if weight_offset else 0.0)
    kbuf, vbuf = ops.tensorFromNumpy(ck), ops.tensorFromNumpy(cv)
    kv_start = max(0, pos + 1 - rows) if ring else 0
    out = ops.runDecodeAttentionFromQKV(ops.tensorFromNumpy(qkv), ops.tensorFromNumpy(qw), ops.tensorFromNumpy(kw),
                                        ops.tensorFromNumpy(cos), ops.tensorFromNumpy(sin), 1e-6, kbuf.buffer,
                                        vbuf.buffer, H, Hkv, D, pos, rotaryDim=rotary, interleaved=interleaved,
                                        rmsNormWeightOffset=weight_offset, attnSoftcap=softcap, slidingWindow=window,
                                        kvStart=kv_start, kvLayout="ring" if ring else "contiguous")
    wk, wv = ck.copy(), cv.copy()
    q = oracle.qkv_norm_rope_kvwrite(qkv, qw, kw, cos, sin, 1, H, Hkv, D, pos, wk.reshape(-1), wv.reshape(-1),
                                     new_row * Hkv * D, rotary_dim=rotary, interleaved=interleaved,
                                     weight_offset=weight_offset)
    want = oracle.attention_decode_f16kv(q, wk, wv, H, Hkv, D, pos - kv_start + 1, start_pos=pos, softcap=softcap,
                                         sliding_window=window, kv_start=kv_start, kv_layout=1 if ring else 0)
    got_k = ops.readBuffer(kbuf.buffer, dtype=np.uint16).reshape(rows, Hkv, D)
    got_v = ops.readBuffer(vbuf.buffer, dtype=np.uint16).reshape(rows, Hkv, D)
    assert np.array_equal(got_v, wv)                    # V: a pure narrowing, and no other row touched
    others = np.arange(rows) != new_row
    assert np.array_equal(got_k[others], wk[others])
    gk, ek = got_k[new_row].view(np.float16).astype(np.float64), wk[new_row].view(np.float16).astype(np.float64)
    assert rel_l2(gk, ek) <= 5e-4 and np.mean(got_k[new_row] != wk[new_row]) < 0.02
    # the oracle attends to ITS f16 key; ours may differ from it by an f16 ulp in a few elements
    assert rel_l2(ops.readTensor(out), want) <= 2e-4, (H, Hkv, D, pos)


@pytest.mark.parametrize("pos", [0, 1, 63, 64, 65, 575, 640, 2047, 9000])
def test_attention_decode_from_qkv_positions(pos):
    _fused_case(32, 8, 128, pos, seed=5300 + pos)


@pytest.mark.parametrize("H,Hkv,D,rotary,interleaved", [(8, 8, 128, 128, False), (16, 2, 128, 64, False),
                                                        (8, 1, 64, 64, False), (6, 2, 64, 64, True),
                                                        (16, 8, 128, 96, True), (4, 4, 64, 16, True),
                                                        (16, 8, 128, 32, False), (4, 4, 64, 4, False),
                                                        (8, 1, 128, 8, False), (12, 4, 128, 6, True)])
def test_attention_decode_from_qkv_geometries(H, Hkv, D, rotary, interleaved):
    assert ops.decodeAttentionFromQKVSupported(H, Hkv, D, rotary, interleaved)
    _fused_case(H, Hkv, D, 333, seed=5400 + H + rotary, rotary=rotary, interleaved=interleaved)


def test_attention_decode_from_qkv_options():
    _fused_case(32, 32, 128, 2500, seed=5500)                       # more chunks than splits: the owner loops
    _fused_case(16, 8, 128, 1499, seed=5501, window=200)            # sliding window, contiguous rows
    _fused_case(16, 8, 128, 1499, seed=5502, window=256, ring=True) # ring rows, wrapped
    _fused_case(16, 8, 128, 100, seed=5503, window=256, ring=True)  # ring not yet full
    _fused_case(16, 8, 128, 900, seed=5504, softcap=3.0, weight_offset=True)
    assert not ops.decodeAttentionFromQKVSupported(16, 8, 128, 96, False)     # partners not a lane apart
    assert not ops.decodeAttentionFromQKVSupported(16, 8, 128, 4, False)
    assert not ops.decodeAttentionFromQKVSupported(16, 8, 256, 256, False)
    z = ops.tensorFromNumpy(np.zeros(64, np.float32))
    with pytest.raises(DopplerHipError, match="not served"):
        ops.runDecodeAttentionFromQKV(ops.tensorFromNumpy(np.zeros(32 * 128, np.float32)), z, z, z, z, 1e-6,
                                      ops.acquireBuffer(4096), ops.acquireBuffer(4096), 16, 8, 128, 0, rotaryDim=96)


def test_attention_decode_from_qkv_matches_separate_ops_without_norm():
    H, Hkv, D, pos = 32, 8, 128, 700
    cos, sin = synth.rope_tables(D, pos + 1, 1e6)
    ck = synth.normal_f32((pos + 1, Hkv, D), 5600, D ** -0.5).astype(np.float16).view(np.uint16)
    cv = synth.normal_f32((pos + 1, Hkv, D), 5601, D ** -0.5).astype(np.float16).view(np.uint16)
    qkv = synth.normal_f32((1, (H + 2 * Hkv) * D), 5602, D ** -0.5)
    L = capi.load()
    t = {k_: ops.tensorFromNumpy(v_) for k_, v_ in dict(qkv=qkv, cos=cos, sin=sin).items()}
    outs = []
    for fused in (False, True):
        kb, vb = ops.tensorFromNumpy(ck), ops.tensorFromNumpy(cv)
        if fused:
            o = ops.runDecodeAttentionFromQKV(t["qkv"], None, None, t["cos"], t["sin"], 1e-6, kb.buffer, vb.buffer, H,
                                              Hkv, D, pos, useNorm=False)
        else:
            qb = ops.acquireBuffer(H * D * 4)
            capi.check(L.dh_qkv_norm_rope_kvwrite(t["qkv"].buffer.data_ptr(), None, None, t["cos"].buffer.data_ptr(),
                                                  t["sin"].buffer.data_ptr(), qb.data_ptr(), kb.buffer.data_ptr(),
                                                  vb.buffer.data_ptr(), 1, H, Hkv, D, pos, D, 0, 1e-6, 0,
                                                  pos * Hkv * D, 0))
            o = ops.runAttention(ops.Tensor(qb, "f32", (H, D), "q"), kb, vb, None, H, D, kvLen=pos + 1, numKVHeads=Hkv,
                                 startPos=pos)
        outs.append((ops.readTensor(o), ops.readBuffer(kb.buffer, dtype=np.uint16), ops.readBuffer(vb.buffer, dtype=np.uint16)))
    assert np.array_equal(outs[0][2], outs[1][2])
    # K: the two kernels may contract the rotation into fused multiply-adds differently
    assert np.mean(outs[0][1] != outs[1][1]) < 1e-4
    assert rel_l2(outs[1][1].view(np.float16).astype(np.float64), outs[0][1].view(np.float16).astype(np.float64)) <= 1e-4
    assert rel_l2(outs[1][0], outs[0][0]) <= 1e-5


# ----------------------------------------------------------------------------- prefill attention

def _prefill_oracle(q, kb, vb, T, H, Hkv, D, kv_len, start_pos, causal=True, window=0, softcap=0.0, scale=None):
    """Oracle for T query rows: each row is one decode-attention problem at its own position."""
    out = np.empty((T, H, D), np.float32)
    for t in range(T):
        out[t] = oracle.attention_decode_f16kv(q[t], kb, vb, H, Hkv, D, kv_len, scale=scale, causal=causal,
                                               start_pos=start_pos + t, sliding_window=window, softcap=softcap).reshape(H, D)
    return out


@pytest.mark.parametrize("T,start,H,Hkv,D", [(64, 0, 16, 8, 128), (200, 56, 16, 8, 128), (7, 0, 4, 4, 64),
                                            (130, 300, 8, 2, 64), (512, 0, 32, 8, 128), (33, 1000, 32, 8, 128)])
def test_attention_prefill_causal(T, start, H, Hkv, D):
    """seqLen > 1: query t at position start + t sees keys 0..start + t (the reference's causal
    prefill, attention.js:1047-1080 with createCausalMask semantics).  f16 matrix-core inputs."""
    kv_len = start + T
    cos, sin = synth.rope_tables(D, kv_len, 1e6)
    q = synth.normal_f32((T, H, D), 6000 + T, D ** -0.5)
    k = synth.normal_f32((kv_len, Hkv, D), 6001 + T, D ** -0.5)
    v = synth.normal_f32((kv_len, Hkv, D), 6002 + T, D ** -0.5)
    q = oracle.rope_apply(q, cos, sin, T, H, D, start_pos=start).reshape(T, H, D) * 4.0
    k = oracle.rope_apply(k, cos, sin, kv_len, Hkv, D, start_pos=0)
    kb, vb = k.astype(np.float16).view(np.uint16), v.astype(np.float16).view(np.uint16)
    out = ops.runAttention(ops.tensorFromNumpy(q), ops.tensorFromNumpy(kb), ops.tensorFromNumpy(vb), None, H, D,
                           seqLen=T, kvLen=kv_len, numKVHeads=Hkv, causal=True, startPos=start)
    assert out.shape == (T, H, D)
    got = ops.readTensor(out).reshape(T, H, D)
    want = _prefill_oracle(q, kb, vb, T, H, Hkv, D, kv_len, start)
    assert rel_l2(got, want) <= REL_L2_F16_MFMA
    # row by row as well: early rows see few keys and must not be polluted by masked ones
    for t in (0, T // 2, T - 1):
        assert rel_l2(got[t], want[t]) <= REL_L2_F16_MFMA, t


def test_attention_prefill_options_and_errors():
    T, start, H, Hkv, D = 96, 40, 8, 4, 128
    kv_len = start + T
    q = synth.normal_f32((T, H, D), 6100, 1.0)
    kb = synth.normal_f32((kv_len, Hkv, D), 6101, D ** -0.5).astype(np.float16).view(np.uint16)
    vb = synth.normal_f32((kv_len, Hkv, D), 6102, 1.0).astype(np.float16).view(np.uint16)
    qt, kt, vt = ops.tensorFromNumpy(q), ops.tensorFromNumpy(kb), ops.tensorFromNumpy(vb)
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, seqLen=T, kvLen=kv_len, numKVHeads=Hkv, startPos=start,
                                          slidingWindow=50, scale=0.2))
    want = _prefill_oracle(q, kb, vb, T, H, Hkv, D, kv_len, start, window=50, scale=0.2)
    assert rel_l2(got, want) <= REL_L2_F16_MFMA
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, seqLen=T, kvLen=kv_len, numKVHeads=Hkv, startPos=start,
                                          attnSoftcap=3.0, scale=0.5))
    want = _prefill_oracle(q, kb, vb, T, H, Hkv, D, kv_len, start, softcap=3.0, scale=0.5)
    assert rel_l2(got, want) <= REL_L2_F16_MFMA
    # not causal: every query sees every key
    got = ops.readTensor(ops.runAttention(qt, kt, vt, None, H, D, seqLen=T, kvLen=kv_len, numKVHeads=Hkv, causal=False,
                                          startPos=start, scale=0.2))
    want = _prefill_oracle(q, kb, vb, T, H, Hkv, D, kv_len, start, causal=False, scale=0.2)
    assert rel_l2(got, want) <= REL_L2_F16_MFMA
    with pytest.raises(DopplerHipError, match="exceeds kvLen"):
        ops.runAttention(qt, kt, vt, None, H, D, seqLen=T, kvLen=kv_len - 1, numKVHeads=Hkv, startPos=start)
    with pytest.raises(DopplerHipError, match="contiguous cache"):
        ops.runAttention(qt, kt, vt, None, H, D, seqLen=T, kvLen=kv_len, numKVHeads=Hkv, startPos=start, kvLayout="ring",
                         slidingWindow=64)


# ----------------------------------------------------------------------------- dense matmul + RMSNorm

@pytest.mark.parametrize("N,K,transposeB,offset,residual,w16", [
    (1152, 6912, True, True, True, False),      # Gemma-3 1B down projection + post-FFN norm
    (1152, 6912, False, True, True, False),
    (4096, 8192, True, False, False, False),    # the largest shape the reference routes here
    (4096, 8192, False, False, True, True),
    (256, 1000, True, False, False, True), (7, 13, False, True, True, False), (1, 5, True, False, False, False),
    (1001, 301, False, False, True, True), (1001, 301, True, True, False, False)])
def test_matmul_rmsnorm_fused(N, K, transposeB, offset, residual, w16):
    g = synth.rng(7000 + N + K)
    x = g.standard_normal(K).astype(np.float32)
    W = (g.standard_normal((N, K)) * K ** -0.5).astype(np.float32)
    w = g.standard_normal(N).astype(np.float32)
    if w16:
        w = w.astype(np.float16).astype(np.float32)
    r = g.standard_normal(N).astype(np.float32) if residual else None
    stored = W if transposeB else np.ascontiguousarray(W.T)
    nw = ops.tensorFromNumpy(w.astype(np.float16).view(np.uint16)) if w16 else ops.tensorFromNumpy(w)
    assert ops.shouldUseFusedMatmulRMSNorm(1, N, K)
    out = ops.runMatmulRMSNormFused(ops.tensorFromNumpy(x), ops.tensorFromNumpy(stored), nw,
                                    {"N": N, "K": K, "eps": 1e-6, "transposeB": transposeB, "rmsNormWeightOffset": offset,
                                     "residual": ops.tensorFromNumpy(r) if residual else None})
    assert out.shape == (1, N) and out.dtype == "f32"
    want = oracle.matmul_rmsnorm_fused(x, stored, w, N, K, 1e-6, transpose_b=transposeB, weight_offset=offset, residual=r)
    assert rel_l2(ops.readTensor(out), want) <= 1e-5
    # equals the unfused pair of ops of this library to rounding
    if transposeB and not w16:
        a = ops.readTensor(out)
        again = ops.readTensor(ops.recordMatmulRMSNormFused(None, ops.tensorFromNumpy(x), ops.tensorFromNumpy(stored), nw,
                                                            N=N, K=K, eps=1e-6, transposeB=True, rmsNormWeightOffset=offset,
                                                            residual=ops.tensorFromNumpy(r) if residual else None))
        assert a.tobytes() == again.tobytes()       # run to run deterministic


@pytest.mark.parametrize("N,K,transposeB,offset,residual,w16", [
    (1152, 6912, True, True, True, True), (1152, 6912, False, False, True, False),
    (4096, 8192, True, False, False, False), (4096, 8192, False, True, True, True),
    (250, 1000, True, False, True, False), (7, 13, False, True, False, True), (1001, 301, True, True, True, True),
    (1004, 304, False, False, False, False)])
def test_matmul_rmsnorm_fused_f16(N, K, transposeB, offset, residual, w16):
    """The all-f16 variants (fused_matmul_rmsnorm_f16.wgsl): f16 activations, weights, residual and
    output, sums in f32.  Checked against the f64 evaluation of the same f16 inputs; the bar is the
    rounding of the f16 result (relative 2^-11 per element, and the reference's medium variant
    rounds the product to f16 once more before it normalises)."""
    g = synth.rng(7200 + N + K)
    x = g.standard_normal(K).astype(np.float16)
    W = (g.standard_normal((N, K)) * K ** -0.5).astype(np.float16)
    w = g.standard_normal(N).astype(np.float16 if w16 else np.float32)
    r = g.standard_normal(N).astype(np.float16) if residual else None
    stored = W if transposeB else np.ascontiguousarray(W.T)
    up16 = lambda a: ops.tensorFromNumpy(a.view(np.uint16))
    assert ops.selectMatmulRMSNormFusedVariant(N, "f16") == ("small_f16" if N <= 256 else "medium_f16")
    out = ops.runMatmulRMSNormFused(up16(x), ops.createWeightBuffer(up16(stored).buffer, "f16", "row", stored.shape), 
                                    up16(w) if w16 else ops.tensorFromNumpy(w),
                                    {"N": N, "K": K, "eps": 1e-6, "transposeB": transposeB, "rmsNormWeightOffset": offset,
                                     "residual": up16(r) if residual else None})
    assert out.shape == (1, N) and out.dtype == "f16"
    got = ops.readTensor(out).view(np.float16).astype(np.float32)
    want = oracle.matmul_rmsnorm_fused(x.astype(np.float32), stored.astype(np.float32), w.astype(np.float32), N, K, 1e-6,
                                       transpose_b=transposeB, weight_offset=offset,
                                       residual=r.astype(np.float32) if residual else None)
    assert rel_l2(got, want) <= 5e-4
    assert np.all(np.abs(got - want) <= 2.0 ** -10 * np.maximum(np.abs(want), 2.0 ** -14) + 1e-6)


def test_matmul_rmsnorm_fused_errors_and_selection():
    x = ops.tensorFromNumpy(np.zeros(8, np.float32))
    W = ops.tensorFromNumpy(np.zeros((4, 8), np.float32))
    nw = ops.tensorFromNumpy(np.ones(4, np.float32))
    with pytest.raises(DopplerHipError, match="transposeB is required"):
        ops.runMatmulRMSNormFused(x, W, nw, {"N": 4, "K": 8, "eps": 1e-6, "rmsNormWeightOffset": False})
    with pytest.raises(DopplerHipError, match="rmsNormWeightOffset is required"):
        ops.runMatmulRMSNormFused(x, W, nw, {"N": 4, "K": 8, "eps": 1e-6, "transposeB": True})
    with pytest.raises(DopplerHipError, match="eps is required"):
        ops.runMatmulRMSNormFused(x, W, nw, {"N": 4, "K": 8, "transposeB": True, "rmsNormWeightOffset": False})
    with pytest.raises(DopplerHipError, match="exceeds maxMediumN=4096"):
        ops.runMatmulRMSNormFused(x, W, nw, {"N": 4097, "K": 8, "eps": 1e-6, "transposeB": True, "rmsNormWeightOffset": False})
    with pytest.raises(DopplerHipError, match="does not match hiddenSize=4"):
        ops.runMatmulRMSNormFused(x, W, ops.tensorFromNumpy(np.ones(1, np.float32)),
                                  {"N": 4, "K": 8, "eps": 1e-6, "transposeB": True, "rmsNormWeightOffset": False})
    with pytest.raises(DopplerHipError, match="dense f16 weights required for f16 activations"):
        ops.runMatmulRMSNormFused(ops.tensorFromNumpy(np.zeros(8, np.uint16)), W, nw,
                                  {"N": 4, "K": 8, "eps": 1e-6, "transposeB": True, "rmsNormWeightOffset": False})
    with pytest.raises(DopplerHipError, match="exceeds maxMediumN"):
        capi.check(capi.init(0).dh_matmul_rmsnorm_f32(x.buffer.data_ptr(), W.buffer.data_ptr(), 1, nw.buffer.data_ptr(),
                                                      capi.F32, 1e-6, 0, None, x.buffer.data_ptr(), 5000, 8))


# ----------------------------------------------------------------------------- finiteness guard

@pytest.mark.parametrize("dtype", ["f32", "f16"])
def test_check_finiteness_status_word(dtype):
    npdt = np.float16 if dtype == "f16" else np.float32
    n = 200_003
    clean = (synth.normal_f32((n,), 7100) * 100).astype(npdt)
    clean[5] = 65500 if dtype == "f32" else 65472      # at the threshold is not beyond it
    up = lambda a: ops.tensorFromNumpy(a.view(np.uint16) if dtype == "f16" else a)
    status = ops.createFinitenessStatusBuffer()
    want = np.zeros(4, np.uint32)
    ops.recordCheckFiniteness(None, up(clean), n, status, 3, 9)
    oracle.check_finiteness(clean, want, 3, 9)
    assert ops.readBuffer(status, 16, np.uint32).tolist() == want.tolist() == [0, 0, 0, 0]
    # one bad element anywhere, of every kind, in the last position too
    bads = [np.inf, -np.inf, np.nan, 65504.0, -65504.0] + ([1e30, 65500.01] if dtype == "f32" else [])
    for i, bad in enumerate(bads):
        dirty = clean.copy()
        dirty[n - 1 if i % 2 else (i * 7919) % n] = bad
        st = ops.createFinitenessStatusBuffer()
        ops.recordCheckFiniteness(None, up(dirty), n, st, 10 + i, 20 + i)
        want = oracle.check_finiteness(dirty, np.zeros(4, np.uint32), 10 + i, 20 + i)
        assert want[0] == 1
        assert ops.readBuffer(st, 16, np.uint32).tolist() == want.tolist(), bad
        # a set status keeps its first layer and step
        ops.recordCheckFiniteness(None, up(dirty), n, st, 99, 98)
        assert ops.readBuffer(st, 16, np.uint32).tolist() == want.tolist()
        assert ops.parseFinitenessStatusWords(ops.readBuffer(st, 16, np.uint32)) == \
            oracle.finiteness_parse_status(want)
    # the element past `size` is not looked at; a custom threshold; a bad threshold falls back to 65500
    dirty = clean.copy()
    dirty[1000] = np.inf
    st = ops.createFinitenessStatusBuffer()
    ops.recordCheckFiniteness(None, up(dirty), 1000, st, 1, 1)
    assert ops.readBuffer(st, 16, np.uint32).tolist() == [0, 0, 0, 0]
    ops.recordCheckFiniteness(None, up(clean), n, st, 4, 5, absThreshold=50.0)
    assert ops.readBuffer(st, 16, np.uint32).tolist() == oracle.check_finiteness(clean, np.zeros(4, np.uint32), 4, 5, 50.0).tolist()
    st = ops.createFinitenessStatusBuffer()
    ops.recordCheckFiniteness(None, up(clean), n, st, 4, 5, absThreshold=-1)
    assert ops.readBuffer(st, 16, np.uint32).tolist() == [0, 0, 0, 0]
    ops.recordCheckFiniteness(None, up(clean), 0, st, 4, 5)
