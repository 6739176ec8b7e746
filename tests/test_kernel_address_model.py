"""Host model of the address arithmetic of the two streaming Q4_K GEMV kernels (int8 matrix-core
kernel, q4k_gemv_i8.hip; few-row f16 matrix-core kernel, q4k_gemv_rows.hip).  No GPU: the launch
parameters come from the library's own dispatcher (dh_q4k_gemv_layout), are re-derived here from the
shape alone, and every address the kernels form from them (LDS offsets against the dynamic LDS
request, global offsets against the extents of weights, activations and outputs) is evaluated for the
first, an inner and the last workgroup, every wave, every lane, and the first, last and tail work
units, over every shape class the dispatcher sends to these kernels.  The formulas below restate the
kernels' index expressions; a change to either side that breaks a bound fails here, on the CPU.
"""
import ctypes
import itertools

import numpy as np
import pytest

from doppler_amd import capi

WAVES, TILE_ROWS, BLOCK, QK = 16, 16, 144, 256
STAGE = TILE_ROWS * BLOCK            # bytes of a ring stage (few-row kernel)
STAGE_I8 = 3 * 1024                  # int8 kernel: a stage takes three full 64-lane loads (a unit is the first 2304 bytes)
REC, ZERO = 848, 144                 # int8 kernel: bytes of an activation record, of the zero area
READ_AHEAD = 12 * 64                 # int8 kernel: the last partial-sum read reaches this far past its slot, per activation row
I8, ROWS = capi.PLAN_GEMV_I8, capi.PLAN_GEMV_ROWS
NCU = 256


def layout(M, N, K, normed, dual, ncu=NCU):
    out = (ctypes.c_int64 * 12)()
    fam = capi.load().dh_q4k_gemv_layout(M, N, K, int(normed), int(dual), ncu, out)
    keys = ("rows", "nlw", "grid", "tiles_base", "tiles_rem", "depth", "lds", "upt", "upt_mul", "nslots", "acc_max", "mt")
    return fam, dict(zip(keys, [int(v) for v in out]))


def ceil_div(a, b):
    return -(-a // b)


def tile_rows(N, ncu):
    """rows per tile: the largest count <= 16 that gives every workgroup the same number of tiles"""
    per_cu = ceil_div(N, ncu * TILE_ROWS)
    return max(1, min(TILE_ROWS, ceil_div(N, ncu * per_cu)))


def lanes():
    return np.arange(64)


# ------------------------------------------------------------------------------------------ int8 kernel

def check_i8(M, N, K, normed, dual, ncu=NCU):
    fam, lay = layout(M, N, K, normed, dual, ncu)
    assert fam == I8, (M, N, K, fam)
    nb, nmat, MT = ceil_div(K, QK), 2 if dual else 1, lay["mt"]
    # ---- the host's arithmetic, from the shape alone
    rows = tile_rows(N, ncu)
    ntiles = ceil_div(N, rows)
    grid = min(ntiles, ncu)
    upt = nb * nmat
    upt_mul = ((1 << 24) + upt - 1) // upt
    need = (WAVES * 4 + upt - 1) // upt + 2
    nslots = 2
    while nslots < need:
        nslots *= 2
    assert MT == (2 if M == 2 and lay["mt"] == 2 else 1)
    lds = WAVES * 1 * STAGE_I8 + nb * MT * REC + ZERO + 4 * nslots * upt * MT * 16 + 4 * (2 + 2 * nslots + nb) + READ_AHEAD * MT
    assert (lay["rows"], lay["nlw"], lay["grid"], lay["tiles_base"], lay["tiles_rem"]) == \
        (rows, ceil_div(9 * rows, 64), grid, ntiles // grid, ntiles % grid)
    assert (lay["upt"], lay["upt_mul"], lay["nslots"], lay["depth"], lay["lds"]) == (upt, upt_mul, nslots, 1, lds)
    assert lds <= 160 * 1024
    row_bytes = nb * BLOCK
    # ---- LDS layout: ring, records, zeros, partial sums, counters (+ read-ahead padding)
    o_xq = WAVES * 1 * STAGE_I8
    o_zero = o_xq + nb * MT * REC
    o_red = o_zero + ZERO
    o_ctr = o_red + 4 * nslots * upt * MT * 16
    o_end = o_ctr + 4 * (2 + 2 * nslots + nb)
    assert o_end + READ_AHEAD * MT == lds
    lane = lanes()
    j, kg = lane & 15, lane >> 4
    # ring: what the load unit writes (piece t * 64 + lane of a unit, 16 bytes) and what the lanes read back
    # (every lane of the three loads writes: the lanes past the unit's pieces land in the stage's tail)
    for t in range(3):
        assert np.all(t * 1024 + lane * 16 + 16 <= STAGE_I8)
    hdr = j * BLOCK
    q = hdr + 16 + 32 * (kg >> 1) + 16 * (kg & 1)
    assert np.all(hdr + 16 <= TILE_ROWS * BLOCK) and np.all(q + 64 + 16 <= TILE_ROWS * BLOCK)
    # records: digit operands (or the zero area), sub-block sums and factors, sum of squares
    g, dg = j >> 2, j & 3
    data_off = 256 * np.minimum(dg, 2) + 32 * g + 16 * (kg & 1)
    assert np.all(data_off + 128 + 16 <= 768)
    assert np.all(768 + 4 * kg + 4 * 4 + 4 <= 800) and np.all(768 + 4 * kg + 4 * 12 + 4 <= 832) and 832 + 4 <= REC
    assert 128 + 16 <= ZERO
    # ---- per workgroup: units, the reciprocal-multiply decode, slots, global addresses
    for bid in sorted({0, 1, grid // 2, lay["tiles_rem"] - 1, lay["tiles_rem"], grid - 1} & set(range(grid))):
        ntl = lay["tiles_base"] + (1 if bid < lay["tiles_rem"] else 0)
        total = ntl * upt
        us = np.unique(np.clip(np.concatenate([np.arange(0, min(total, 200)), np.arange(max(0, total - 200), total),
                                                np.arange(0, total, max(1, total // 997))]), 0, max(total - 1, 0)))
        if total == 0:
            continue
        prod = us.astype(np.uint64) * np.uint64(upt_mul)
        assert np.all(prod < (1 << 32))                              # formed in 32 bits by the kernel
        tl = (prod >> np.uint64(24)).astype(np.int64)
        assert np.array_equal(tl, us // upt)
        r = us - tl * upt
        mat = np.where(r >= nb, 1, 0) if dual else np.zeros_like(r)
        col = r - mat * nb
        assert np.all((col >= 0) & (col < nb)) and np.all(tl < ntl)
        tile = bid + tl * grid
        assert np.all(tile < ntiles)
        rows_left = N - tile * rows
        assert np.all(rows_left >= 1)
        base = tile * rows * row_bytes + col * BLOCK
        assert np.all(base + rows * row_bytes < (1 << 32))          # offsets inside a matrix are formed in 32 bits
        for t in range(3):
            p = t * 64 + lane
            valid = p < 9 * rows
            rr = p // 9
            piece = (p - rr * 9) * 16
            for b_, left in zip(base, rows_left):
                if left >= rows:
                    # full tile: lanes past the tile's pieces fetch piece 0 of row 0 again
                    off = b_ + np.where(valid, rr * row_bytes + piece, 0)
                else:
                    # last, partial tile: every lane's row is clamped to the last one
                    off = b_ + np.minimum(rr, left - 1) * row_bytes + piece
                assert np.all(off + 16 <= N * row_bytes), (bid, t)
                assert np.all(off >= 0)
        # partial sums: writes of a unit, and the finishing wave's four-columns-at-a-time reads
        slot = tl & (nslots - 1)
        for m in range(MT):
            w = o_red + (((slot * upt + (mat * nb + col)) * MT + m) * 16 + 15) * 4 + 4
            assert np.all(w <= o_ctr)
            for s_, c in itertools.product(range(nslots), range(nb)):
                for mt_ in range(nmat):
                    rd = o_red + (s_ * upt * MT * 64) + (((mt_ * nb + c) * MT + m) * 16 + 15) * 4 + 12 * MT * 64 + 4
                    assert rd <= lds
        # outputs and residual
        row = tile * rows + 15
        ok = (15 < rows) & (row < N)
        assert np.all((MT - 1) * N + row[ok] < M * N + (MT - M) * N)
    # ---- activation side: lane t holds elements 4t .. 4t+3 of columns wave, wave + 16, ..
    for wave in range(WAVES):
        for c in range(wave, nb, WAVES):
            k0 = c * QK + 4 * lane
            if K % 4 == 0:
                kc = np.where(k0 < K, k0, 0)
                assert np.all(kc + 4 <= K)
            else:
                for e in range(4):
                    assert np.all(np.minimum(k0 + e, K - 1) < K)
            for m in range(MT):
                assert min(m, M - 1) * K + (K - 1) < M * K
            rec = o_xq + (c * MT + (MT - 1)) * REC
            assert rec + REC <= o_zero
    # counters: next unit, per-slot counts and generations, column flags, the give-up word
    assert o_ctr + 4 * (1 + 2 * nslots + nb) + 4 <= o_end


I8_SHAPES = [
    # (M, N, K, normed, dual)
    (1, 2048, 640, 0, 0),                                           # config 0: K off the block size
    (1, 2048, 1024, 1, 0), (2, 1024, 1024, 0, 0), (1, 1024, 2048, 0, 0), (2, 3072, 1024, 1, 1), (1, 1024, 3072, 0, 0),   # config 1
    (1, 6144, 4096, 1, 0), (1, 4096, 4096, 0, 0), (1, 12288, 4096, 1, 1), (1, 4096, 12288, 0, 0),   # config 4
    (2, 6144, 4096, 1, 0), (2, 4096, 4096, 0, 0), (2, 12288, 4096, 1, 1), (2, 4096, 12288, 0, 0),
    (1, 151936, 4096, 0, 0),                                        # many tiles per workgroup
    (1, 4097, 4096, 0, 0), (2, 300, 700, 0, 0), (1, 17, 1023, 0, 0), (1, 5000, 2560, 1, 1),   # ragged N, K off 4
    (1, 4096, 25088, 1, 0), (2, 1024, 8192, 1, 0), (1, 64, 16384, 0, 0),   # the longest rows the kernel takes
    (1, 1_000_000, 4096, 0, 0),                                     # more than 200 tiles per workgroup
]


@pytest.mark.parametrize("shape", I8_SHAPES, ids=lambda s: "M%d_N%d_K%d_%s%s" % (s[0], s[1], s[2], "n" if s[3] else "", "d" if s[4] else ""))
def test_int8_gemv_addresses_stay_inside_their_buffers(shape):
    check_i8(*shape)


def test_int8_gemv_refuses_what_its_32_bit_unit_decode_cannot_hold():
    """The kernel decodes a unit number with a 32-bit multiply: more than 255 tiles per workgroup would
    wrap it and send loads to the wrong rows, so the dispatcher hands such shapes to another kernel."""
    fam, lay = layout(1, 256 * 16 * 300, 4096, 0, 0)
    assert fam != I8
    fam, lay = layout(1, 256 * 16 * 200, 4096, 0, 0)
    assert fam == I8 and (lay["tiles_base"] + 1) * lay["upt"] * lay["upt_mul"] < 1 << 32


# --------------------------------------------------------------------------------------- few-row kernel

def check_rows(M, N, K, normed, dual, ncu=NCU):
    fam, lay = layout(M, N, K, normed, dual, ncu)
    assert fam == ROWS, (M, N, K, fam)
    Mp = min(M, 8)                                 # rows of the first pass
    nb, nmat = ceil_div(K, QK), 2 if dual else 1
    rows = tile_rows(N, ncu)
    ntiles = ceil_div(N, rows)
    grid = min(ntiles, ncu)
    tiles_base, tiles_rem = ntiles // grid, ntiles % grid
    acc_max = (tiles_base + (1 if tiles_rem else 0)) * nmat
    ssq_floats, acc_bytes = 16, 512

    def lds_for(depth):
        return WAVES * depth * STAGE + (4 * WAVES * QK if normed else 0) + 4 * WAVES * ssq_floats + WAVES * acc_max * acc_bytes

    depth = 2
    while depth > 1 and lds_for(depth) > 160 * 1024:
        depth -= 1
    assert (lay["rows"], lay["nlw"], lay["grid"], lay["tiles_base"], lay["tiles_rem"], lay["acc_max"], lay["depth"], lay["lds"]) == \
        (rows, ceil_div(9 * rows, 64), grid, tiles_base, tiles_rem, acc_max, depth, lds_for(depth))
    assert lay["lds"] <= 160 * 1024 and lay["mt"] == Mp
    lds = lay["lds"]
    row_bytes = nb * BLOCK
    o_wn = WAVES * depth * STAGE
    o_ssq = o_wn + (4 * WAVES * QK if normed else 0)
    o_acc = o_ssq + 4 * WAVES * ssq_floats
    assert o_acc + WAVES * acc_max * acc_bytes == lds
    lane = lanes()
    j, kg = lane & 15, lane >> 4
    xrow, part = j >> 1, j & 1
    xk = 8 * kg + 4 * part
    # ring reads: header of row j, eight bytes of nibbles of the lane's k-group in each of the four chunks
    assert np.all(j * BLOCK + 16 <= STAGE) and np.all(j * BLOCK + 16 + 8 * kg + 96 + 8 <= STAGE)
    for bid in sorted({0, 1, grid // 2, tiles_rem - 1, tiles_rem, grid - 1} & set(range(grid))):
        ntl = tiles_base + (1 if bid < tiles_rem else 0)
        nacc = ntl * nmat
        total = nb * nacc
        assert nacc <= acc_max
        for wave in range(WAVES):
            q0, q1 = (wave * total) >> 4, ((wave + 1) * total) >> 4
            # accumulators: zero-fill, read-add-write of a unit, the reduction after the barrier
            my_acc = o_acc + wave * acc_max * acc_bytes
            assert my_acc + (nacc - 1) * acc_bytes + 8 * 63 + 8 <= lds if nacc else True
            if normed:
                assert 4 * 28 + 896 + 16 <= 4 * QK and o_wn + 4 * (wave + 1) * QK <= o_ssq      # the lane's norm weights, sub-blocks 0..7
                assert o_wn + 4 * wave * QK + 63 * 16 + 16 <= o_ssq                  # what the load unit writes
            assert o_ssq + 4 * (wave * ssq_floats + 7) + 4 <= o_acc
            for u in sorted({q0, q0 + 1, (q0 + q1) // 2, q1 - 1} & set(range(q0, q1))):
                col, acc = u // nacc, u % nacc
                assert col < nb
                itl, imat = (acc >> 1, acc & 1) if dual else (acc, 0)
                tile = bid + itl * grid
                assert tile < ntiles and imat < nmat
                base = tile * rows * row_bytes + col * BLOCK
                last = N - tile * rows - 1
                assert last >= 0
                for t in range(3):
                    p = t * 64 + lane
                    valid = p < 9 * rows
                    rr = p // 9
                    off = base + np.minimum(rr, last) * row_bytes + 16 * (p - rr * 9)
                    assert np.all((off + 16)[valid] <= N * row_bytes) and np.all(off[valid] >= 0)
                    assert np.all((t * 1024 + lane * 16 + 16)[valid] <= STAGE)
                # the column's activations (and the next column's, requested while this unit is multiplied)
                for c_ in {col, min(col + 1, nb - 1)}:
                    for s in range(8):
                        k = c_ * QK + 32 * s + xk
                        if K % 4 == 0:
                            o = np.minimum(xrow, Mp - 1) * K + np.minimum(k, K - 4)
                            assert np.all(o + 4 <= Mp * K) and np.all(o >= 0)
                        else:
                            for e in range(4):
                                assert np.all(np.minimum(xrow, Mp - 1) * K + np.minimum(k + e, K - 1) < Mp * K)
                    if normed and K % 4 == 0:
                        assert np.all(np.minimum(c_ * QK + 4 * lane, K - 4) + 4 <= K)
        # outputs: element e of accumulator tl of every wave
        for tl in range(ntl):
            for w in range(WAVES):
                rd = o_acc + 4 * ((w * acc_max + tl * nmat) * 128 + 127) + (4 * 128 if dual else 0) + 4
                assert rd <= lds
            tile = bid + tl * grid
            for oj in range(16):
                row = tile * rows + oj
                if oj < rows and row < N:
                    assert (Mp - 1) * N + row < Mp * N


ROWS_SHAPES = [
    (4, 1024, 3072, 0, 0), (8, 1024, 3072, 0, 0),                   # config 1's down projection
    (3, 6144, 4096, 1, 0), (4, 4096, 4096, 0, 0), (8, 12288, 4096, 1, 1), (8, 4096, 12288, 0, 0),   # config 4
    (12, 12288, 4096, 1, 1), (15, 4096, 12288, 0, 0),               # two passes
    (5, 4097, 4096, 0, 0), (7, 5000, 2560, 1, 1), (3, 3000, 4095, 0, 0), (8, 2048, 3000, 1, 0),   # ragged N, K off the block / off 4
    (8, 4096, 32768, 1, 0), (3, 40000, 4096, 0, 0), (1, 4096, 32768, 1, 0),
]


@pytest.mark.parametrize("shape", ROWS_SHAPES, ids=lambda s: "M%d_N%d_K%d_%s%s" % (s[0], s[1], s[2], "n" if s[3] else "", "d" if s[4] else ""))
def test_few_row_gemv_addresses_stay_inside_their_buffers(shape):
    check_rows(*shape)


def test_a_smaller_device_changes_the_layout_not_the_bounds():
    check_i8(1, 12288, 4096, 1, 1, ncu=64)
    check_i8(2, 4096, 12288, 0, 0, ncu=304)
    check_rows(8, 4096, 4096, 0, 0, ncu=64)
    check_rows(4, 4096, 12288, 0, 0, ncu=304)
