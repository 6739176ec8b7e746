"""Pins the CPU oracle to facts that do not come from the oracle itself: the reference's
recorded digests for a real 9B tensor, numpy/torch library routines, exact rational
arithmetic and brute force.  A wrong index, sign, rounding or operand order in
oracle/doppler_oracle.c fails at least one test here."""
import hashlib
import math
import os
import shutil
import subprocess
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle
from doppler_amd import synth


# ----------------------------------------------------------------------------- f16

def test_f16_to_f32_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_bits_to_f32(bits)
    want = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_f32_to_f16_rne_matches_ieee():
    # every exact tie between neighbouring f16 values, its two f32 neighbours, all f16
    # values themselves, and a dense random sample over the full f32 range
    h = np.arange(0x7C00, dtype=np.uint16).view(np.float16).astype(np.float64)
    ties = ((h[:-1] + h[1:]) / 2).astype(np.float32)
    assert np.array_equal(ties.astype(np.float64), (h[:-1] + h[1:]) / 2)
    tb = ties.view(np.uint32)
    cases = [ties, (tb + 1).view(np.float32), (tb - 1).view(np.float32), h.astype(np.float32)]
    g = np.random.default_rng(1)
    cases.append(g.integers(0, 2**32, 2_000_000, dtype=np.uint32).view(np.float32))
    cases.append(np.array([65504, 65519.99, 65520, 65536, 1e30, np.inf, 2**-24, 2**-25,
                           2**-25 * 1.0001, 2**-26, 0.0], np.float32))
    x = np.concatenate(cases)
    x = np.concatenate([x, -x])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = oracle.f32_to_f16_bits(x)
    assert np.array_equal(got, want)


def test_f32_to_f16_reference_host_variants_differ_only_where_documented():
    L = oracle.lib()
    # exact tie 1 + 2^-11 : RNE keeps the even mantissa, half-up rounds away, trunc chops
    tie = np.float32(1.0 + 2.0**-11)
    assert L.dor_f32_to_f16_rne(tie) == 0x3C00
    assert L.dor_f32_to_f16_half_up(tie) == 0x3C01
    assert L.dor_f32_to_f16_trunc(np.float32(1.0 + 2.0**-10 - 2.0**-20)) == 0x3C00
    g = np.random.default_rng(2)
    x = g.standard_normal(20000).astype(np.float32)
    for v in x[:5000]:
        a, b = L.dor_f32_to_f16_rne(v), L.dor_f32_to_f16_half_up(v)
        is_tie = (int(v.view(np.uint32)) & 0x1FFF) == 0x1000 and abs(v) >= 2.0**-14
        assert a == b or (is_tie and b == a + 1)   # the two roundings part only on exact ties


# ----------------------------------------------------------------------------- Q4_K: receipt

def test_receipt_block_d_widening(receipt):
    sha = receipt["sha256"]
    d = oracle.f16_bits_to_f32(receipt["d_bits"])
    dmin = oracle.f16_bits_to_f32(receipt["dmin_bits"])
    assert hashlib.sha256(d.tobytes()).hexdigest() == sha["blockD"]
    assert hashlib.sha256(dmin.tobytes()).hexdigest() == sha["blockDmin"]


def _receipt_blocks(receipt, seed=7):
    nb = receipt["d_bits"].size
    q = synth.rng(seed).integers(0, 16, size=(nb, 256), dtype=np.uint8)
    blocks = synth.q4k_pack_block_fields(receipt["d_bits"], receipt["dmin_bits"],
                                         receipt["scale_bits"].reshape(nb, 8),
                                         receipt["min_bits"].reshape(nb, 8), q)
    return blocks, q


def test_receipt_scale_unpack_roundtrip_and_decoded_digests(receipt):
    """Real 6-bit scales/mins packed with the quantizer's rule (reference
    tests/kernels/reference/dequant.js:209-239) must come back unchanged from the oracle's
    unpack, and f32(d*sc), f32(dmin*mn) must hash to the digests the reference recorded."""
    sha = receipt["sha256"]
    assert sha["blockCount"] == receipt["d_bits"].size
    assert hashlib.sha256(receipt["scale_bits"].tobytes()).hexdigest() == sha["packedScaleBits"]
    blocks, _ = _receipt_blocks(receipt)
    for b in (0, 1, 17, 196607):
        sc, mn = oracle.q4k_unpack_scale_bits(blocks[b])
        assert np.array_equal(sc, receipt["scale_bits"][b * 8:b * 8 + 8])
        assert np.array_equal(mn, receipt["min_bits"][b * 8:b * 8 + 8])
    scales, mins = oracle.q4k_decoded_scales(blocks.reshape(-1))
    assert hashlib.sha256(scales.tobytes()).hexdigest() == sha["decodedScales"]
    assert hashlib.sha256(mins.tobytes()).hexdigest() == sha["decodedMinima"]


def test_receipt_dequant_matches_fields(receipt):
    """Whole-block decode on real scales: w[64c+j] uses sub-block 2c and the low nibble of
    byte j, w[64c+32+j] sub-block 2c+1 and the high nibble (checked against the fields
    the blocks were assembled from, in float64)."""
    blocks, q = _receipt_blocks(receipt)
    nb = 4096
    w = oracle.q4k_dequant_blocks(blocks[:nb].reshape(-1)).reshape(nb, 8, 32)
    d = receipt["d_bits"][:nb].view(np.float16).astype(np.float64)
    dmin = receipt["dmin_bits"][:nb].view(np.float16).astype(np.float64)
    sc = receipt["scale_bits"][:nb * 8].reshape(nb, 8).astype(np.float64)
    mn = receipt["min_bits"][:nb * 8].reshape(nb, 8).astype(np.float64)
    want = (d[:, None] * sc)[:, :, None] * q[:nb].reshape(nb, 8, 32) - (dmin[:, None] * mn)[:, :, None]
    assert np.array_equal(w, want.astype(np.float32))


def test_fast_f32_dequant_equals_double_dequant(receipt):
    blocks, _ = _receipt_blocks(receipt, seed=9)
    sub = blocks[:30000].reshape(-1)
    assert oracle.q4k_dequant_blocks_fast(sub).tobytes() == oracle.q4k_dequant_blocks(sub).tobytes()
    g = np.random.default_rng(10)
    n = 20000
    rnd = synth.q4k_pack_block_fields(g.integers(0, 0x7C00, n, dtype=np.uint16), g.integers(0, 0x7C00, n, dtype=np.uint16),
                                      g.integers(0, 64, (n, 8), dtype=np.uint8), g.integers(0, 64, (n, 8), dtype=np.uint8),
                                      g.integers(0, 16, (n, 256), dtype=np.uint8)).reshape(-1)
    with np.errstate(over="ignore", invalid="ignore"):
        a, b = oracle.q4k_dequant_blocks_fast(rnd), oracle.q4k_dequant_blocks(rnd)
    assert a.tobytes() == b.tobytes()


# ----------------------------------------------------------------------------- Q4_K: closed forms

def test_dequant_is_single_correct_rounding_of_exact_value():
    g = np.random.default_rng(3)
    n = 3000
    d_bits = g.integers(0, 0x7C00, n, dtype=np.uint16)        # every finite non-negative f16
    dmin_bits = g.integers(0, 0x7C00, n, dtype=np.uint16)
    d_bits[:8] = [0, 1, 2, 0x3FF, 0x400, 0x7BFF, 0x3C00, 0x0001]
    sc = g.integers(0, 64, (n, 8), dtype=np.uint8)
    mn = g.integers(0, 64, (n, 8), dtype=np.uint8)
    q = g.integers(0, 16, (n, 256), dtype=np.uint8)
    blocks = synth.q4k_pack_block_fields(d_bits, dmin_bits, sc, mn, q)
    with np.errstate(over="ignore", invalid="ignore"):
        w = oracle.q4k_dequant_blocks(blocks.reshape(-1)).reshape(n, 8, 32)
    for b in range(0, n, 7):
        fd = Fraction(float(d_bits[b:b + 1].view(np.float16)[0]))
        fm = Fraction(float(dmin_bits[b:b + 1].view(np.float16)[0]))
        for sb in (0, 3, 4, 7):
            for j in (0, 13, 31):
                exact = fd * int(sc[b, sb]) * int(q[b, sb * 32 + j]) - fm * int(mn[b, sb])
                as_double = float(exact)
                assert Fraction(as_double) == exact            # exact in double -> one rounding
                with np.errstate(over="ignore"):
                    assert np.float32(as_double).tobytes() == w[b, sb, j].tobytes()


def test_nibble_and_subblock_order_one_hot():
    one = np.array([0x3C00], np.uint16)   # d = dmin = 1.0
    for chunk in range(4):
        for j in (0, 5, 31):
            for hi in (0, 1):
                sc = np.arange(1, 9, dtype=np.uint8)[None, :]         # scale of sub-block s is s+1
                mn = np.zeros((1, 8), np.uint8)
                blk = synth.q4k_pack_block_fields(one, one, sc, mn, np.zeros((1, 256), np.uint8))
                blk[0, 16 + chunk * 32 + j] = 0x90 if hi else 0x09      # nibble value 9
                w = oracle.q4k_dequant_blocks(blk.reshape(-1))
                elem = 64 * chunk + 32 * hi + j
                want = np.zeros(256, np.float32)
                want[elem] = 9.0 * (elem // 32 + 1)
                assert np.array_equal(w, want)


def test_scale_bit_fields_high_subblocks():
    # sub-blocks 4..7 take their low 4 bits from bytes 12..15 and their top 2 bits from the
    # top of bytes 4..7 (scales) / 8..11 (mins)
    blk = np.zeros(144, np.uint8)
    blk[4 + 1] = 0b10_000101       # sc[1] = 5, top bits of sc[5] = 2
    blk[8 + 1] = 0b01_000011       # mn[1] = 3, top bits of mn[5] = 1
    blk[12 + 1] = 0xA7             # sc[5] low = 7, mn[5] low = 10
    sc, mn = oracle.q4k_unpack_scale_bits(blk)
    assert list(sc) == [0, 5, 0, 0, 0, 2 * 16 + 7, 0, 0]
    assert list(mn) == [0, 3, 0, 0, 0, 1 * 16 + 10, 0, 0]


def test_dequant_rows_drops_row_padding():
    N, K = 5, 300
    W = synth.q4k_tensor(N, K, seed=11)
    rows = oracle.q4k_dequant_rows(W, N, K)
    flat = oracle.q4k_dequant_blocks(W).reshape(N, 2 * 256)
    assert np.array_equal(rows, flat[:, :K])


# ----------------------------------------------------------------------------- Q4_K matmul

def test_q4k_matmul_equals_dequant_then_sequential_f64_dot():
    M, N, K = 3, 9, 640
    W = synth.q4k_tensor(N, K, seed=21)
    A = synth.normal_f32((M, K), seed=22)
    C = oracle.q4k_matmul(A, W, M, N, K, alpha=0.5)
    Wd = oracle.q4k_dequant_rows(W, N, K)
    for m in range(M):
        for n in range(N):
            s = 0.0
            for k in range(K):
                s += float(A[m, k]) * float(Wd[n, k])
            assert np.float32(s * 0.5) == C[m, n]


@pytest.mark.skipif(shutil.which("node") is None, reason="node is not installed")
def test_js_port_of_the_reference_agrees_with_the_c_oracle(tmp_path):
    """oracle/js/reference_port.mjs restates the reference's JS decode + f64 dot a second time,
    independently of the C oracle (different language, written from the reference's text):
    both must produce the same f32 results, including a K that is not a multiple of 256 and
    subnormal / large d, dmin."""
    M, N, K = 3, 40, 640
    W = synth.q4k_tensor(N, K, seed=77).copy()
    blocks = W.reshape(-1, 144)
    blocks[0, 0:4] = [0x01, 0x00, 0xff, 0x03]        # subnormal d, largest subnormal dmin
    blocks[1, 0:4] = [0x00, 0x3c, 0x00, 0x44]        # d = 1, dmin = 4
    A = synth.normal_f32((M, K), seed=78)
    src, dst = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(src, "wb") as f:
        f.write(np.array([M, N, K], np.int32).tobytes())
        f.write(A.tobytes())
        f.write(W.tobytes())
    script = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "oracle", "js", "reference_port.mjs")
    subprocess.run(["node", script, "gemv", str(src), str(dst)], check=True, timeout=120)
    got = np.fromfile(dst, np.float32).reshape(M, N)
    want = oracle.q4k_matmul(A, W, M, N, K)
    assert np.array_equal(got, want)


def test_q4k_matmul_properties():
    M, N, K = 2, 64, 1152        # K % 256 != 0: last block of each row is half padding
    W = synth.q4k_tensor(N, K, seed=31)
    A = synth.normal_f32((M, K), seed=32)
    C = oracle.q4k_matmul(A, W, M, N, K)
    Wd = oracle.q4k_dequant_rows(W, N, K).astype(np.float64)
    np.testing.assert_allclose(C, A.astype(np.float64) @ Wd.T, rtol=1e-6, atol=1e-4)
    # one-hot activation returns a dequantized column, bit for bit
    for k in (0, 31, 32, 255, 256, 1151):
        e = np.zeros((1, K), np.float32)
        e[0, k] = 1.0
        assert np.array_equal(oracle.q4k_matmul(e, W, 1, N, K)[0], Wd[:, k].astype(np.float32))
    # the padded tail of the last block never contributes
    W2 = W.reshape(N, 5, 144).copy()
    W2[:, 4, 16 + 64:] ^= 0xFF     # elements 128..255 of block 4 = k 1152..1279
    assert np.array_equal(oracle.q4k_matmul(A, W2.reshape(-1), M, N, K), C)
    # linear in the activation
    B = synth.normal_f32((M, K), seed=33)
    np.testing.assert_allclose(oracle.q4k_matmul(A + B, W, M, N, K),
                               C + oracle.q4k_matmul(B, W, M, N, K), rtol=2e-5, atol=2e-3)


def test_f16w_matmul_vs_numpy():
    M, N, K = 2, 33, 96
    Wb = synth.normal_f16_bits((N, K), seed=41, scale=0.02)
    A = synth.normal_f32((M, K), seed=42)
    C = oracle.f16w_matmul(A, Wb, M, N, K)
    want = A.astype(np.float64) @ Wb.view(np.float16).astype(np.float64).T
    np.testing.assert_allclose(C, want, rtol=1e-6, atol=1e-7)


def test_ffn_gate_up_vs_torch():
    M, hidden, inter = 3, 512, 40
    Wg = synth.q4k_tensor(inter, hidden, seed=51)
    Wu = synth.q4k_tensor(inter, hidden, seed=52)
    X = synth.normal_f32((M, hidden), seed=53, scale=0.05)
    g = torch.from_numpy(X.astype(np.float64) @ oracle.q4k_dequant_rows(Wg, inter, hidden).astype(np.float64).T)
    u = torch.from_numpy(X.astype(np.float64) @ oracle.q4k_dequant_rows(Wu, inter, hidden).astype(np.float64).T)
    silu = (torch.nn.functional.silu(g) * u * 0.25).clamp(-3.0, 3.0)
    got = oracle.q4k_ffn_gate_up(X, Wg, Wu, M, hidden, inter, alpha=0.25, activation="silu", swiglu_limit=3.0)
    np.testing.assert_allclose(got, silu.numpy(), rtol=1e-6, atol=1e-6)
    assert got.max() == 3.0 or got.min() == -3.0   # the clamp is exercised
    gelu = torch.nn.functional.gelu(g, approximate="tanh") * u
    got = oracle.q4k_ffn_gate_up(X, Wg, Wu, M, hidden, inter, activation="gelu", swiglu_limit=3.0)
    np.testing.assert_allclose(got, gelu.numpy(), rtol=1e-6, atol=1e-5)   # no clamp for gelu


# ----------------------------------------------------------------------------- elementwise

def test_act_gate_residual_vs_torch():
    g = synth.normal_f32(1000, seed=61, scale=4.0)
    u = synth.normal_f32(1000, seed=62)
    tg, tu = torch.from_numpy(g).double(), torch.from_numpy(u).double()
    np.testing.assert_allclose(oracle.act_gate(g, u, "silu"), (torch.nn.functional.silu(tg) * tu).numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(oracle.act_gate(g, u, "gelu"),
                               (torch.nn.functional.gelu(tg, approximate="tanh") * tu).numpy(), rtol=1e-6, atol=1e-7)
    clamped = oracle.act_gate(g, u, "silu", swiglu_limit=0.5)
    np.testing.assert_allclose(clamped, (torch.nn.functional.silu(tg) * tu).clamp(-0.5, 0.5).numpy(), rtol=1e-6, atol=1e-7)
    x = np.concatenate([g.reshape(4, 250), u.reshape(4, 250)], axis=1)   # [T, 2*dim]
    assert np.array_equal(oracle.act_gate_rowsplit(x, 4, 250, "silu"), oracle.act_gate(g, u, "silu").reshape(4, 250))
    np.testing.assert_allclose(oracle.residual_add(g, u, 0.5), (tg + tu).numpy() * 0.5, rtol=1e-7)


def test_rmsnorm_vs_torch_and_options():
    B, Hd = 3, 640
    x = synth.normal_f32((B, Hd), seed=71, scale=3.0)
    w = synth.normal_f32(Hd, seed=72, scale=0.1)
    r = synth.normal_f32((B, Hd), seed=73)
    tx, tw, tr = (torch.from_numpy(a).double() for a in (x, w, r))

    def ref(v, weight):
        return v * torch.rsqrt((v * v).mean(-1, keepdim=True) + 1e-6) * weight

    np.testing.assert_allclose(oracle.rmsnorm(x, w, 1e-6), ref(tx, tw).numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(oracle.rmsnorm(x, w, 1e-6, weight_offset=True), ref(tx, 1 + tw).numpy(), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(oracle.rmsnorm(x, w, 1e-6, post_residual=r, output_scale=0.5),
                               ((ref(tx, tw) + tr) * 0.5).numpy(), rtol=1e-6, atol=1e-7)
    out, pre = oracle.rmsnorm(x, w, 1e-6, pre_residual=r, want_prenorm=True)
    s = torch.from_numpy(x + r).double()          # the sum is formed in f32
    assert np.array_equal(pre, x + r)
    np.testing.assert_allclose(out, ref(s, tw).numpy(), rtol=1e-6, atol=1e-7)
    assert np.array_equal(oracle.rmsnorm(x, None, 1e-6), oracle.rmsnorm(x, np.ones(Hd, np.float32), 1e-6))


# ----------------------------------------------------------------------------- RoPE

def test_rope_tables_closed_form():
    D, S, theta = 128, 64, 1e6
    for recipe in ("test", "production"):
        cos, sin = oracle.rope_tables(D, S, theta, recipe)
        i = np.arange(D // 2, dtype=np.float64)
        freq = theta ** (-2.0 * i / D)
        if recipe == "production":
            freq = freq.astype(np.float32).astype(np.float64)
        ang = np.arange(S, dtype=np.float64)[:, None] * freq[None, :]
        np.testing.assert_allclose(cos, np.cos(ang), rtol=0, atol=6e-8)
        np.testing.assert_allclose(sin, np.sin(ang), rtol=0, atol=6e-8)
    c2, s2 = synth.rope_tables(D, S, theta)
    assert np.array_equal(c2, cos) and np.array_equal(s2, sin)
    assert np.all(cos[0] == 1) and np.all(sin[0] == 0)


def test_rope_apply_is_complex_rotation():
    S, H, D, start = 5, 3, 16, 7
    cos, sin = oracle.rope_tables(D, 32, 1e4, "test")
    x = synth.normal_f32((S, H, D), seed=81)
    y = oracle.rope_apply(x, cos, sin, S, H, D, start_pos=start)
    z = (x[..., :D // 2].astype(np.float64) + 1j * x[..., D // 2:].astype(np.float64))
    rot = (cos[start:start + S].astype(np.float64) + 1j * sin[start:start + S].astype(np.float64))[:, None, :]
    zz = z * rot
    np.testing.assert_allclose(y[..., :D // 2], zz.real, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(y[..., D // 2:], zz.imag, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose((y.astype(np.float64) ** 2).sum(-1), (x.astype(np.float64) ** 2).sum(-1), rtol=1e-6)
    assert np.array_equal(oracle.rope_apply(x[:1], cos, sin, 1, H, D, start_pos=0), x[:1])
    # interleaved pairs (2i, 2i+1)
    yi = oracle.rope_apply(x, cos, sin, S, H, D, start_pos=start, interleaved=True)
    zi = (x[..., 0::2].astype(np.float64) + 1j * x[..., 1::2].astype(np.float64)) * rot
    np.testing.assert_allclose(yi[..., 0::2], zi.real, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(yi[..., 1::2], zi.imag, rtol=1e-6, atol=1e-7)
    # partial rotary: only the first rotary_dim elements move, partner at +rotary_dim/2
    c8, s8 = oracle.rope_tables(8, 32, 1e4, "test")
    yp = oracle.rope_apply(x, c8, s8, S, H, D, start_pos=start, rotary_dim=8)
    assert np.array_equal(yp[..., 8:], x[..., 8:])
    zp = (x[..., :4].astype(np.float64) + 1j * x[..., 4:8].astype(np.float64)) * \
        (c8[start:start + S].astype(np.float64) + 1j * s8[start:start + S].astype(np.float64))[:, None, :]
    np.testing.assert_allclose(yp[..., :4], zp.real, rtol=1e-6, atol=1e-7)
    # pairSpanDim = headDim with rotaryDim 8: partner at +D/2
    ys = oracle.rope_apply(x, c8, s8, S, H, D, start_pos=start, rotary_dim=8, pair_span_dim=D)
    zs = (x[..., :4].astype(np.float64) + 1j * x[..., 8:12].astype(np.float64)) * \
        (c8[start:start + S].astype(np.float64) + 1j * s8[start:start + S].astype(np.float64))[:, None, :]
    np.testing.assert_allclose(ys[..., :4], zs.real, rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(ys[..., 8:12], zs.imag, rtol=1e-6, atol=1e-7)


# ----------------------------------------------------------------------------- attention

def _sdpa(Q, K, V, H, Hkv, mask=None, scale=None):
    q = torch.from_numpy(Q).double().permute(1, 0, 2)                       # [H, S, D]
    k = torch.from_numpy(K).double().permute(1, 0, 2).repeat_interleave(H // Hkv, 0)
    v = torch.from_numpy(V).double().permute(1, 0, 2).repeat_interleave(H // Hkv, 0)
    m = torch.from_numpy(mask).double() if mask is not None else None
    o = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=m, scale=scale)
    return o.permute(1, 0, 2).numpy()


@pytest.mark.parametrize("seq,kv,H,Hkv,D", [(2, 4, 2, 1, 8), (1, 37, 16, 8, 128), (5, 5, 4, 2, 16)])
def test_attention_ref_vs_torch_sdpa(seq, kv, H, Hkv, D):
    Q = synth.normal_f32((seq, H, D), seed=91)
    K = synth.normal_f32((kv, Hkv, D), seed=92)
    V = synth.normal_f32((kv, Hkv, D), seed=93)
    np.testing.assert_allclose(oracle.attention_ref(Q, K, V, seq, kv, H, Hkv, D), _sdpa(Q, K, V, H, Hkv),
                               rtol=2e-6, atol=2e-7)
    mask = oracle.causal_mask(seq, kv)
    np.testing.assert_allclose(oracle.attention_ref(Q, K, V, seq, kv, H, Hkv, D, mask=mask),
                               _sdpa(Q, K, V, H, Hkv, mask=mask), rtol=2e-6, atol=2e-7)


def test_attention_invariants():
    H, Hkv, D = 4, 2, 16
    Q = synth.normal_f32((1, H, D), seed=94)
    V = synth.normal_f32((6, Hkv, D), seed=95)
    K = synth.normal_f32((6, Hkv, D), seed=96)
    o = oracle.attention_ref(Q, K[:1], V[:1], 1, 1, H, Hkv, D)            # one key: output is V
    assert np.array_equal(o[0, 0], V[0, 0]) and np.array_equal(o[0, 3], V[0, 1])
    o = oracle.attention_ref(Q * 0, K, V, 1, 6, H, Hkv, D)                # uniform scores: mean of V
    np.testing.assert_allclose(o[0, 1], V[:, 0].astype(np.float64).mean(0), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(o[0, 2], V[:, 1].astype(np.float64).mean(0), rtol=1e-6, atol=1e-7)


def test_attention_decode_f16kv():
    H, Hkv, D, kv = 16, 8, 128, 300
    Q = synth.normal_f32((H, D), seed=101, scale=D ** -0.5)
    Kb = synth.normal_f16_bits((kv, Hkv, D), seed=102, scale=D ** -0.5)
    Vb = synth.normal_f16_bits((kv, Hkv, D), seed=103, scale=D ** -0.5)
    Kf, Vf = Kb.view(np.float16).astype(np.float32), Vb.view(np.float16).astype(np.float32)
    o = oracle.attention_decode_f16kv(Q, Kb, Vb, H, Hkv, D, kv)
    # decode: causal masks nothing; same f32 scale on both sides (the kernel takes it as f32)
    assert np.array_equal(o, oracle.attention_ref(Q, Kf, Vf, 1, kv, H, Hkv, D, scale=float(np.float32(D ** -0.5)))[0])
    np.testing.assert_allclose(o, _sdpa(Q[None], Kf, Vf, H, Hkv)[0], rtol=2e-6, atol=1e-7)
    # explicit scale and soft cap
    o = oracle.attention_decode_f16kv(Q * 30, Kb, Vb, H, Hkv, D, kv, scale=0.2, softcap=5.0)
    s = np.einsum("hd,khd->hk", (Q * 30).astype(np.float64), np.repeat(Kf, 2, axis=1).astype(np.float64)) * 0.2
    s = np.tanh(s / 5.0) * 5.0
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    want = np.einsum("hk,khd->hd", p, np.repeat(Vf, 2, axis=1).astype(np.float64))
    np.testing.assert_allclose(o, want, rtol=1e-5, atol=1e-7)
    # sliding window 64 at query position 299: only keys 236..299 count
    o = oracle.attention_decode_f16kv(Q, Kb, Vb, H, Hkv, D, kv, sliding_window=64)
    np.testing.assert_allclose(o, _sdpa(Q[None], Kf[236:], Vf[236:], H, Hkv)[0], rtol=2e-6, atol=1e-7)
    # causal with start_pos inside the cache: keys after the query are masked
    o = oracle.attention_decode_f16kv(Q, Kb, Vb, H, Hkv, D, kv, start_pos=99)
    np.testing.assert_allclose(o, _sdpa(Q[None], Kf[:100], Vf[:100], H, Hkv)[0], rtol=2e-6, atol=1e-7)
    # ring layout: physical row = abs position % window
    win = 64
    ring_k = np.zeros((win, Hkv, D), np.uint16)
    ring_v = np.zeros((win, Hkv, D), np.uint16)
    for pos in range(kv):
        ring_k[pos % win], ring_v[pos % win] = Kb[pos], Vb[pos]
    o = oracle.attention_decode_f16kv(Q, ring_k, ring_v, H, Hkv, D, win, sliding_window=win,
                                      kv_start=kv - win, kv_layout=1)
    np.testing.assert_allclose(o, _sdpa(Q[None], Kf[236:], Vf[236:], H, Hkv)[0], rtol=2e-6, atol=1e-7)
    # nothing to attend to
    assert not oracle.attention_decode_f16kv(Q, Kb, Vb, H, Hkv, D, 0, start_pos=0).any()


# ----------------------------------------------------------------------------- KV write / fused / gather / argmax

def test_kv_write_and_gather():
    k = synth.normal_f32(512, seed=111)
    v = synth.normal_f32(512, seed=112)
    ck = np.zeros(2048, np.uint16)
    cv = np.zeros(2048, np.uint16)
    oracle.kv_write_f16(k, v, ck, cv, src_off=128, dst_off=1024, count=256)
    assert np.array_equal(ck[1024:1280], k[128:384].astype(np.float16).view(np.uint16))
    assert np.array_equal(cv[1024:1280], v[128:384].astype(np.float16).view(np.uint16))
    assert not ck[:1024].any() and not ck[1280:].any()
    table = synth.normal_f16_bits((50, 24), seed=113)
    ids = np.array([3, 49, 50, 0, 4000000000], np.uint32)
    out = oracle.gather_f16(ids, table, 24, 50)
    tf = table.view(np.float16).astype(np.float32)
    assert np.array_equal(out[0], tf[3]) and np.array_equal(out[1], tf[49]) and np.array_equal(out[3], tf[0])
    assert not out[2].any() and not out[4].any()


def test_qkv_norm_rope_kvwrite_vs_composition():
    T, H, Hkv, D, start = 3, 4, 2, 16, 5
    cos, sin = oracle.rope_tables(D, 16, 1e6, "production")
    qkv = synth.normal_f32((T, (H + 2 * Hkv) * D), seed=121)
    qw = 1 + synth.normal_f32(D, seed=122, scale=0.1)
    kw = 1 + synth.normal_f32(D, seed=123, scale=0.1)
    ck = np.zeros((16, Hkv, D), np.uint16)
    cv = np.zeros((16, Hkv, D), np.uint16)
    q = oracle.qkv_norm_rope_kvwrite(qkv, qw, kw, cos, sin, T, H, Hkv, D, start, ck, cv, start * Hkv * D)
    x = qkv.astype(np.float64)
    qs, ks = H * D, Hkv * D

    def norm_rope(rows, w):          # rows [T, heads, D]
        n = rows / np.sqrt((rows ** 2).mean(-1, keepdims=True) + 1e-6) * w.astype(np.float64)
        z = (n[..., :D // 2] + 1j * n[..., D // 2:]) * (cos[start:start + T] + 1j * sin[start:start + T].astype(np.float64))[:, None, :]
        return np.concatenate([z.real, z.imag], -1)

    np.testing.assert_allclose(q.reshape(T, H, D), norm_rope(x[:, :qs].reshape(T, H, D), qw), rtol=1e-6, atol=1e-7)
    kk = norm_rope(x[:, qs:qs + ks].reshape(T, Hkv, D), kw)
    got_k = ck[start:start + T].view(np.float16).astype(np.float64)
    assert np.abs(got_k - kk).max() <= np.abs(kk).max() * 2.0 ** -11
    assert np.array_equal(cv[start:start + T].reshape(T, ks), qkv[:, qs + ks:].astype(np.float16).view(np.uint16))
    assert not ck[:start].any() and not ck[start + T:].any()


def test_argmax_ties_pad_softcap():
    x = np.array([1.0, 5.0, 5.0, -2.0, 5.0], np.float32)
    assert oracle.argmax(x) == 1
    assert oracle.argmax(x, pad_id=1) == 2
    assert oracle.argmax(-x) == 3
    g = np.random.default_rng(5)
    for _ in range(50):
        v = g.integers(-3, 4, 40).astype(np.float32)
        assert oracle.argmax(v) == int(np.argmax(v))          # numpy also returns the first maximum
    big = np.array([100.0, 200.0, 50.0], np.float32)
    assert oracle.argmax(big, softcap=30.0) == 1            # tanh is monotone while it does not saturate
    sat = np.array([1000.0, 2000.0], np.float32)
    assert oracle.argmax(sat, softcap=30.0) == 0            # both saturate to 30.0 in f32: tie -> lowest index


# ----------------------------------------------------------------------------- whole step wiring

def tiny_model(seed=200, layers=2, hidden=256, inter=512, heads=4, kv_heads=2, head_dim=64, vocab=300, max_seq=16):
    cfg = dict(layers=layers, hidden=hidden, inter=inter, heads=heads, kv_heads=kv_heads, head_dim=head_dim,
               vocab=vocab, max_seq=max_seq, eps=1e-6, qk_norm=1)
    qs, ks = heads * head_dim, kv_heads * head_dim
    L = []
    for i in range(layers):
        s = seed + 20 * i
        L.append(dict(
            wq=synth.q4k_tensor(qs, hidden, s + 1), wk=synth.q4k_tensor(ks, hidden, s + 2),
            wv=synth.q4k_tensor(ks, hidden, s + 3), wo=synth.q4k_tensor(hidden, qs, s + 4),
            wgate=synth.q4k_tensor(inter, hidden, s + 5), wup=synth.q4k_tensor(inter, hidden, s + 6),
            wdown=synth.q4k_tensor(hidden, inter, s + 7),
            input_norm=1 + synth.normal_f32(hidden, s + 8, 0.02), post_attn_norm=1 + synth.normal_f32(hidden, s + 9, 0.02),
            q_norm=1 + synth.normal_f32(head_dim, s + 10, 0.02), k_norm=1 + synth.normal_f32(head_dim, s + 11, 0.02),
            cache_k=np.zeros((max_seq, kv_heads, head_dim), np.uint16),
            cache_v=np.zeros((max_seq, kv_heads, head_dim), np.uint16)))
    embed = synth.normal_f16_bits((vocab, hidden), seed + 900, 0.02)
    final_norm = 1 + synth.normal_f32(hidden, seed + 901, 0.02)
    cos, sin = synth.rope_tables(head_dim, max_seq, 1e6)
    return cfg, L, embed, final_norm, cos, sin


def test_sample_topk_matches_a_direct_restatement_of_the_js_reference():
    """dor_sample_topk against the reference's sampleTopKRef written out with Python's stable
    sort and math.exp (tests/kernels/reference/sample.js:62-92), including ties, top_k = 1 and
    the sub-0.01 temperature that falls back to argmax; seededRandom against Math.sin."""
    g = synth.rng(900)

    def ref(logits, T, k, r):
        if T < 0.01:
            return int(np.argmax(logits))
        order = sorted(range(len(logits)), key=lambda i: (-float(logits[i]), i))[:k]
        vals = [float(logits[i]) / T for i in order]
        mx = max(vals)
        ex = [math.exp(v - mx) for v in vals]
        tot = sum(ex)
        c = 0.0
        for i, e in zip(order, ex):
            c += e / tot
            if c >= r:
                return i
        return order[-1]

    for t in range(200):
        V = int(g.integers(3, 500))
        logits = g.standard_normal(V).astype(np.float32)
        if t % 3 == 0:
            logits = (np.round(logits * 2) / 2).astype(np.float32)      # many exact ties
        k = int(g.integers(1, min(V, 64) + 1))
        T = float(g.choice([0.001, 0.3, 1.0, 2.5]))
        r = float(g.random())
        assert oracle.sample_topk(logits, T, k, r) == ref(logits, T, k, r), (t, V, k, T, r)
    # the running sum never reaches 1.0 + : last candidate
    assert oracle.sample_topk(np.array([0.0, 1.0, 2.0], np.float32), 1.0, 2, 1.5) == 1
    # pad id can never be drawn
    assert oracle.sample_topk(np.array([5.0, 1.0, 0.0], np.float32), 1.0, 2, 0.0, pad_id=0) == 1
    for seed in (0, 1, 42, 12345.5):
        x = math.sin(seed) * 10000
        assert oracle.seeded_random(seed) == x - math.floor(x)


def test_decode_step_wiring_matches_op_by_op():
    cfg, L, embed, final_norm, cos, sin = tiny_model()
    dec = oracle.DecoderOracle(cfg, L, embed, final_norm, cos, sin)
    H, Hkv, D, Hd, I = cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["hidden"], cfg["inter"]
    qs, ks = H * D, Hkv * D
    shadow_k = [np.zeros_like(l["cache_k"]) for l in L]
    shadow_v = [np.zeros_like(l["cache_v"]) for l in L]
    tok = 17
    for pos in range(3):
        got_tok, logits = dec.step(tok, pos, want_logits=True)
        x = oracle.gather_f16([tok], embed, Hd, cfg["vocab"])
        for i, l in enumerate(L):
            n = oracle.rmsnorm(x, l["input_norm"], 1e-6)
            qkv = np.concatenate([oracle.q4k_matmul(n, l["wq"], 1, qs, Hd), oracle.q4k_matmul(n, l["wk"], 1, ks, Hd),
                                  oracle.q4k_matmul(n, l["wv"], 1, ks, Hd)], axis=1)
            q = oracle.qkv_norm_rope_kvwrite(qkv, l["q_norm"], l["k_norm"], cos, sin, 1, H, Hkv, D, pos,
                                             shadow_k[i], shadow_v[i], pos * ks)
            a = oracle.attention_decode_f16kv(q, shadow_k[i], shadow_v[i], H, Hkv, D, pos + 1)
            x = oracle.residual_add(oracle.q4k_matmul(a.reshape(1, qs), l["wo"], 1, Hd, qs), x)
            n = oracle.rmsnorm(x, l["post_attn_norm"], 1e-6)
            h = oracle.act_gate(oracle.q4k_matmul(n, l["wgate"], 1, I, Hd), oracle.q4k_matmul(n, l["wup"], 1, I, Hd))
            x = oracle.residual_add(oracle.q4k_matmul(h, l["wdown"], 1, Hd, I), x)
            assert np.array_equal(shadow_k[i], l["cache_k"]) and np.array_equal(shadow_v[i], l["cache_v"])
        want = oracle.f16w_matmul(oracle.rmsnorm(x, final_norm, 1e-6), embed, 1, cfg["vocab"], Hd)[0]
        assert np.array_equal(logits, want)
        assert got_tok == int(np.argmax(want))
        tok = got_tok


# ----------------------------------------------------------------------------- dense matmul + RMSNorm

def test_matmul_rmsnorm_fused_matches_torch_f64_and_closed_forms():
    g = np.random.default_rng(31)
    for N, K, tb, off, res in [(7, 13, True, False, False), (256, 96, False, True, True),
                               (1152, 300, True, True, True), (300, 1152, False, False, False)]:
        x = g.standard_normal(K).astype(np.float32)
        W = (g.standard_normal((N, K)) * 0.1).astype(np.float32)
        w = g.standard_normal(N).astype(np.float32)
        r = g.standard_normal(N).astype(np.float32) if res else None
        stored = W if tb else np.ascontiguousarray(W.T)
        got = oracle.matmul_rmsnorm_fused(x, stored, w, N, K, 1e-5, transpose_b=tb, weight_offset=off, residual=r)
        y = torch.from_numpy(W).double() @ torch.from_numpy(x).double()
        wt = torch.from_numpy(w).double() + (1.0 if off else 0.0)
        want = torch.nn.functional.rms_norm(y, (N,), wt, 1e-5)
        if res:
            want = want + torch.from_numpy(r).double()
        assert np.allclose(got, want.numpy(), rtol=2e-6, atol=2e-6), (N, K, tb, off, res)
    # identity matrix, unit weight, eps 0: x / rms(x), whose squares average to one; a dropped
    # 1/N or a norm over K instead of N fails here
    N = 64
    x = g.standard_normal(N).astype(np.float32)
    out = oracle.matmul_rmsnorm_fused(x, np.eye(N, dtype=np.float32), np.ones(N, np.float32), N, N, 0.0)
    assert np.allclose(out, x / np.sqrt(np.mean(x.astype(np.float64) ** 2)), rtol=1e-6)
    assert abs(np.mean(out.astype(np.float64) ** 2) - 1.0) < 1e-6
    # the residual comes after the norm: it shifts the output by exactly itself
    r = g.standard_normal(N).astype(np.float32)
    shifted = oracle.matmul_rmsnorm_fused(x, np.eye(N, dtype=np.float32), np.ones(N, np.float32), N, N, 0.0, residual=r)
    assert np.allclose(shifted - out, r, atol=1e-6)
    # a non-square one-hot matrix tells [N, K] from [K, N]
    W = np.zeros((3, 5), np.float32)
    W[2, 4] = 2.0
    x = np.arange(1, 6, dtype=np.float32)
    a = oracle.matmul_rmsnorm_fused(x, W, np.ones(3, np.float32), 3, 5, 0.0, transpose_b=True)
    b = oracle.matmul_rmsnorm_fused(x, np.ascontiguousarray(W.T), np.ones(3, np.float32), 3, 5, 0.0, transpose_b=False)
    assert np.allclose(a, [0, 0, math.sqrt(3.0)]) and np.allclose(b, a)


# ----------------------------------------------------------------------------- finiteness guard

def test_finiteness_guard_matches_the_reference_tests_vectors():
    # tests/inference/finiteness-overflow-gate.test.js
    assert oracle.finiteness_should_trigger(100) is False
    assert oracle.finiteness_should_trigger(65501, 65500) is True
    assert oracle.finiteness_should_trigger(-70000, 65500) is True
    for v in (float("inf"), float("-inf"), float("nan")):
        assert oracle.finiteness_should_trigger(v, 65500) is True
    assert oracle.finiteness_should_trigger(60000, -1) is False      # bad threshold -> 65500
    assert oracle.finiteness_should_trigger(60000, 50000) is True
    # tests/inference/finiteness-guard-status.test.js
    s = oracle.finiteness_parse_status(np.array([0, 7, 9], np.uint32), 0)
    assert s == {"triggered": False, "layer": 0, "step": 0, "metadata": ""}
    s = oracle.finiteness_parse_status(np.array([1, 8, 12], np.uint32), 0)
    assert s == {"triggered": True, "layer": 8, "step": 12, "metadata": " (layer 8, step 12)"}
    s = oracle.finiteness_parse_status(np.array([42, 1, 3, 15, 0], np.uint32), 1)
    assert s == {"triggered": True, "layer": 3, "step": 15, "metadata": " (layer 3, step 15)"}
    # the status word: clean input leaves it alone, the first trigger wins, later ones do not overwrite
    st = np.zeros(4, np.uint32)
    oracle.check_finiteness(np.array([1.0, -65500.0, 65500.0], np.float32), st, 3, 4)
    assert st.tolist() == [0, 0, 0, 0]
    oracle.check_finiteness(np.array([1.0, 65504.0], np.float16), st, 5, 6)
    assert st.tolist() == [1, 5, 6, 0]
    oracle.check_finiteness(np.array([np.nan], np.float32), st, 7, 8)
    assert st.tolist() == [1, 5, 6, 0]
    for bad in (np.inf, -np.inf, np.nan, 1e5, -1e5):
        st = np.zeros(4, np.uint32)
        oracle.check_finiteness(np.array([0.0, bad], np.float32), st, 1, 2)
        assert st.tolist() == [1, 1, 2, 0], bad
    st = np.zeros(4, np.uint32)
    oracle.check_finiteness(np.array([70000.0], np.float32), st, 1, 2, abs_threshold=1e6)
    assert st.tolist() == [0, 0, 0, 0]
