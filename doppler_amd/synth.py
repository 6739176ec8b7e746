"""Seeded synthetic inputs for the benchmark configurations.

Both sides of every parity check (HIP path and CPU checker) consume the bytes produced
here, so the generators are plain numpy with a fixed PRNG (PCG64) and a per-tensor seed.

Q4_K tensors: per 144-byte super-block, d and dmin are f16(|N(0,1)| * 0.01), the eight
6-bit scales and eight 6-bit mins are uniform on 0..63 and the 256 4-bit quants uniform on
0..15.  Bytes 4..143 of a block use every bit for exactly one of those fields, so uniform
fields are the same thing as uniform random bytes; only d/dmin need to be drawn separately.
"""
import numpy as np

QK_K = 256
Q4K_BLOCK_BYTES = 144


def rng(seed):
    return np.random.Generator(np.random.PCG64(seed))


def q4k_row_blocks(K):
    return (K + QK_K - 1) // QK_K


def q4k_nbytes(N, K):
    return N * q4k_row_blocks(K) * Q4K_BLOCK_BYTES


def q4k_tensor(N, K, seed):
    """Random Q4_K weight [N, K] in row layout: uint8[N * ceil(K/256) * 144]."""
    g = rng(seed)
    nblk = N * q4k_row_blocks(K)
    blocks = g.integers(0, 256, size=(nblk, Q4K_BLOCK_BYTES), dtype=np.uint8)
    dd = (np.abs(g.standard_normal((nblk, 2), dtype=np.float32)) * np.float32(0.01)).astype(np.float16)
    blocks[:, 0:4] = dd.view(np.uint8).reshape(nblk, 4)
    return blocks.reshape(-1)


def q4k_pack_block_fields(d_bits, dmin_bits, sc, mn, q):
    """Assemble super-blocks from fields (inverse of the decode): d_bits, dmin_bits
    uint16[nb]; sc, mn uint8[nb, 8] (0..63); q uint8[nb, 256] (0..15)."""
    nb = d_bits.shape[0]
    out = np.zeros((nb, Q4K_BLOCK_BYTES), np.uint8)
    out[:, 0] = d_bits & 0xFF
    out[:, 1] = d_bits >> 8
    out[:, 2] = dmin_bits & 0xFF
    out[:, 3] = dmin_bits >> 8
    sc = sc.astype(np.uint8)
    mn = mn.astype(np.uint8)
    out[:, 4:8] = (sc[:, 0:4] & 0x3F) | (((sc[:, 4:8] >> 4) & 0x03) << 6)
    out[:, 8:12] = (mn[:, 0:4] & 0x3F) | (((mn[:, 4:8] >> 4) & 0x03) << 6)
    out[:, 12:16] = (sc[:, 4:8] & 0x0F) | ((mn[:, 4:8] & 0x0F) << 4)
    qq = q.reshape(nb, 4, 2, 32).astype(np.uint8)
    out[:, 16:] = ((qq[:, :, 0, :] & 0x0F) | ((qq[:, :, 1, :] & 0x0F) << 4)).reshape(nb, 128)
    return out


def q4k_centred(W, shift=0):
    """A copy of Q4_K tensor W with zero-mean weights of the same spread: every sub-block's min is set
    to its scale and dmin to 7.5 d, so that w = d sc (q - 7.5); d is scaled by 2^-shift on the way.
    (The benchmark's own distribution, mins and dmin drawn independently, gives every weight the same
    large positive mean: a decoder stack of such matrices collapses onto the all-ones direction and
    its logits hardly depend on the token or on the KV cache.)"""
    w = np.ascontiguousarray(W).reshape(-1, Q4K_BLOCK_BYTES).copy()
    d = (w[:, 0:2].copy().view(np.float16).astype(np.float32) * np.float32(2.0 ** -shift)).astype(np.float16)
    w[:, 0:2] = d.view(np.uint8)
    w[:, 2:4] = (d.astype(np.float32) * np.float32(7.5)).astype(np.float16).view(np.uint8)
    w[:, 8:12] = w[:, 4:8]                                                  # mins 0..3 and the high bits of mins 4..7
    w[:, 12:16] = (w[:, 12:16] & 0x0F) | ((w[:, 12:16] & 0x0F) << 4)        # low bits of mins 4..7
    return w.reshape(-1)


def normal_f32(shape, seed, scale=1.0):
    return (rng(seed).standard_normal(shape, dtype=np.float32) * np.float32(scale)).astype(np.float32)


def normal_f16_bits(shape, seed, scale=1.0):
    """N(0, scale^2) rounded to nearest-even f16; returns the uint16 bit patterns."""
    return normal_f32(shape, seed, scale).astype(np.float16).view(np.uint16)


def normal_f16_bits_large(shape, seed, scale=1.0):
    """Same distribution as normal_f16_bits for tensors of 10^8+ elements (the 9B-class tied
    embedding): torch's CPU generator and vectorised f32->f16 (round-to-nearest-even) are an
    order of magnitude faster than numpy here.  Different PRNG, so different bytes than
    normal_f16_bits for the same seed; both parity sides always share one host array."""
    import torch
    g = torch.Generator().manual_seed(int(seed))
    n = int(np.prod(shape))
    x = torch.randn(n, generator=g, dtype=torch.float32)
    x.mul_(float(scale))
    return x.to(torch.float16).numpy().view(np.uint16).reshape(shape)


def rope_tables(rotary_dim, max_seq, theta, rope_scale=1.0):
    """cos/sin tables [max_seq, rotary_dim/2] f32: frequency rounded to f32, angle and
    cos/sin in f64 (the recipe of the reference's init-rope.js:21-26,120-133)."""
    half = rotary_dim // 2
    i = np.arange(half, dtype=np.float64)
    freq = (1.0 / np.power(float(theta), 2.0 * i / rotary_dim)).astype(np.float32).astype(np.float64)
    pos = np.arange(max_seq, dtype=np.float64)[:, None] / np.float64(np.float32(rope_scale))
    ang = pos * freq[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


# BASELINE configuration shapes ------------------------------------------------------

CFG0 = dict(N=2048, K=640)
CFG1_SHAPES = {  # name: (N, K) of one Qwen3-0.6B-shaped block
    "q_proj": (2048, 1024), "k_proj": (1024, 1024), "v_proj": (1024, 1024),
    "o_proj": (1024, 2048), "gate_proj": (3072, 1024), "up_proj": (3072, 1024),
    "down_proj": (1024, 3072),
}
CFG2 = dict(M=512, hidden=1152, inter=6912)
CFG3 = dict(H=16, Hkv=8, D=128, contexts=(512, 4096, 32768), theta=1e6)
CFG4 = dict(layers=36, hidden=4096, inter=12288, heads=32, kv_heads=8, head_dim=128,
            vocab=151936, eps=1e-6, theta=1e6, prefill=2048, steps=64, qk_norm=1)
