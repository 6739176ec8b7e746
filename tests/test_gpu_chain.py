"""dh_q4k_gemv_chain: the dependent products between two attentions of a decoder layer in ONE launch
(o-projection + residual, RMSNorm + gate/up + SiLU, down-projection + residual, RMSNorm + next q/k/v),
against the CPU oracle's chain and, bit for bit, against the same products as separate calls; replays
(eager and from a captured graph); and the failure path: a launch whose waits cannot be served gives
up, every wave exits, and the next synchronising call reports it.
"""
import ctypes

import numpy as np
import pytest
import torch

import oracle
from doppler_amd import capi, synth
from doppler_amd.capi import DopplerHipError

pytestmark = pytest.mark.gpu

EPS = 1e-6


def rel_l2(got, want):
    got = np.asarray(got, np.float64).reshape(-1)
    want = np.asarray(want, np.float64).reshape(-1)
    return float(np.linalg.norm(got - want) / max(np.linalg.norm(want), 1e-30))


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1)).cuda()


def f32(n):
    return torch.zeros(n, dtype=torch.float32, device="cuda")


class Layer:
    """Weights and vectors of one "o, gate/up, down, next qkv" run."""

    def __init__(self, Hd, I, QS, QKV, seed):
        self.dims = (Hd, I, QS, QKV)
        self.h = dict(wo=synth.q4k_tensor(Hd, QS, seed + 1), wg=synth.q4k_tensor(I, Hd, seed + 2),
                      wu=synth.q4k_tensor(I, Hd, seed + 3), wd=synth.q4k_tensor(Hd, I, seed + 4),
                      wq=synth.q4k_tensor(QKV, Hd, seed + 5),
                      n1=(1 + synth.normal_f32(Hd, seed + 6, 0.02)).astype(np.float32),
                      n2=(1 + synth.normal_f32(Hd, seed + 7, 0.02)).astype(np.float32),
                      attn=synth.normal_f32(QS, seed + 8), x=synth.normal_f32(Hd, seed + 9))
        # the gate/up pair of random weights of this size reaches 1e5: scaled inputs keep SiLU in its curved range
        self.h["attn"] *= np.float32(0.01)
        self.h["x"] *= np.float32(0.01)
        self.d = {k: dev(v) for k, v in self.h.items()}
        self.out = dict(x2=f32(Hd), act=f32(I), x3=f32(Hd), qkv=f32(QKV))

    def phases(self, out=None, n=4):
        Hd, I, QS, QKV = self.dims
        o, d = out or self.out, self.d
        ph = [dict(W=d["wo"].data_ptr(), C=o["x2"].data_ptr(), residual=d["x"].data_ptr(), N=Hd, K=QS),
              dict(W=d["wg"].data_ptr(), W2=d["wu"].data_ptr(), C=o["act"].data_ptr(), norm_weight=d["n1"].data_ptr(),
                   N=I, K=Hd, activation=capi.ACT_SILU, norm_eps=EPS),
              dict(W=d["wd"].data_ptr(), C=o["x3"].data_ptr(), residual=o["x2"].data_ptr(), N=Hd, K=I),
              dict(W=d["wq"].data_ptr(), C=o["qkv"].data_ptr(), norm_weight=d["n2"].data_ptr(), N=QKV, K=Hd, norm_eps=EPS)]
        return ph[:n]

    def separate(self, L, out):
        Hd, I, QS, QKV = self.dims
        d, ck = self.d, capi.check
        ck(L.dh_q4k_matmul(d["attn"].data_ptr(), capi.F32, d["wo"].data_ptr(), out["x2"].data_ptr(), capi.F32, 1, Hd, QS, 1.0,
                           d["x"].data_ptr()))
        ck(L.dh_q4k_ffn_gate_up_rmsnorm(out["x2"].data_ptr(), d["n1"].data_ptr(), EPS, 0, d["wg"].data_ptr(), d["wu"].data_ptr(),
                                        out["act"].data_ptr(), 1, Hd, I, capi.ACT_SILU, 1.0, 0.0))
        ck(L.dh_q4k_matmul(out["act"].data_ptr(), capi.F32, d["wd"].data_ptr(), out["x3"].data_ptr(), capi.F32, 1, Hd, I, 1.0,
                           out["x2"].data_ptr()))
        ck(L.dh_q4k_matmul_rmsnorm(out["x3"].data_ptr(), d["n2"].data_ptr(), EPS, 0, d["wq"].data_ptr(), out["qkv"].data_ptr(),
                                   capi.F32, 1, QKV, Hd, 1.0, None))

    def oracle_chain(self):
        Hd, I, QS, QKV = self.dims
        h = self.h
        x2 = oracle.q4k_matmul(h["attn"].reshape(1, QS), h["wo"], 1, Hd, QS).reshape(-1) + h["x"]
        n = oracle.rmsnorm(x2.reshape(1, Hd), h["n1"], EPS, batch=1, hidden=Hd)
        act = oracle.q4k_ffn_gate_up(np.asarray(n, np.float32).reshape(1, Hd), h["wg"], h["wu"], 1, Hd, I, activation="silu").reshape(-1)
        x3 = oracle.q4k_matmul(act.reshape(1, I), h["wd"], 1, Hd, I).reshape(-1) + x2
        n = oracle.rmsnorm(x3.reshape(1, Hd), h["n2"], EPS, batch=1, hidden=Hd)
        qkv = oracle.q4k_matmul(np.asarray(n, np.float32).reshape(1, Hd), h["wq"], 1, QKV, Hd).reshape(-1)
        return dict(x2=x2, act=act, x3=x3, qkv=qkv)


def _read(t):
    return t.cpu().numpy().copy()


@pytest.mark.parametrize("dims", [(2048, 4096, 2048, 3072), (4096, 12288, 4096, 6144), (2048, 2304, 4096, 2501)],
                         ids=["small", "cfg4-layer", "ragged-tiles"])
def test_chain_against_oracle_and_separate_calls(dims):
    L = capi.init(0)
    lay = Layer(*dims, seed=7000 + dims[1])
    sep = {k: torch.zeros_like(v) for k, v in lay.out.items()}
    lay.separate(L, sep)
    capi.check(L.dh_sync())
    want = lay.oracle_chain()
    names = ["x2", "act", "x3", "qkv"]
    for n in (1, 2, 3, 4):
        for t in lay.out.values():
            t.fill_(float("nan"))
        arr = capi.chain_phases(lay.phases(n=n))
        capi.check(L.dh_q4k_gemv_chain(lay.d["attn"].data_ptr(), arr, n))
        capi.check(L.dh_sync())
        for name in names[:n]:
            got = _read(lay.out[name])
            assert rel_l2(got, want[name]) <= 1e-3, (n, name)
            # the same arithmetic as the separate launches: identical bits
            assert got.tobytes() == _read(sep[name]).tobytes(), (n, name)
        for name in names[n:]:
            assert np.isnan(_read(lay.out[name])).all(), (n, name)      # untouched


def test_chain_replays_eager_and_from_a_graph():
    """The exchange's sequence numbers come from a launch counter on the device, so the same launch can
    be repeated, also from a captured graph, with other work and synchronisations in between."""
    L = capi.init(0)
    lay = Layer(2048, 4096, 2048, 3072, seed=7100)
    arr = capi.chain_phases(lay.phases())
    x0 = lay.d["attn"].data_ptr()
    capi.check(L.dh_q4k_gemv_chain(x0, arr, 4))
    capi.check(L.dh_sync())
    first = {k: _read(v) for k, v in lay.out.items()}
    for rep in range(5):
        for t in lay.out.values():
            t.zero_()
        torch.cuda.synchronize()
        capi.check(L.dh_q4k_gemv_chain(x0, arr, 4))
        capi.check(L.dh_sync())
        for k, v in lay.out.items():
            assert _read(v).tobytes() == first[k].tobytes(), (rep, k)
    capi.check(L.dh_graph_begin())
    try:
        capi.check(L.dh_q4k_gemv_chain(x0, arr, 4))
    finally:
        g = ctypes.c_void_p()
        rc = L.dh_graph_end(0, ctypes.byref(g))
    capi.check(rc)
    try:
        for rep in range(4):
            for t in lay.out.values():
                t.zero_()
            torch.cuda.synchronize()
            capi.check(L.dh_graph_launch(g, 0))
            capi.check(L.dh_sync())
            for k, v in lay.out.items():
                assert _read(v).tobytes() == first[k].tobytes(), ("graph", rep, k)
            # an eager launch between replays moves the launch counter on
            capi.check(L.dh_q4k_gemv_chain(x0, arr, 2))
            capi.check(L.dh_sync())
    finally:
        capi.check(L.dh_graph_destroy(g))


def test_chain_gives_up_a_wait_that_cannot_be_served():
    """One workgroup of the chain alone: the other workgroups' outputs never arrive, so its bounded
    waits run into the (tiny) limit; every wave exits, the launch ends, and the next synchronising
    call fails with the reason.  The library then starts the exchange over and the next chain is right."""
    L = capi.init(0)
    lay = Layer(2048, 4096, 2048, 3072, seed=7200)
    arr = capi.chain_phases(lay.phases())
    x0 = lay.d["attn"].data_ptr()
    capi.check(L.dh_q4k_gemv_chain(x0, arr, 4))
    capi.check(L.dh_sync())
    good = {k: _read(v) for k, v in lay.out.items()}
    capi.check(L.dh_q4k_gemv_chain_limited(x0, arr, 4, 1, 64))
    with pytest.raises(DopplerHipError, match="gave up a bounded wait"):
        capi.check(L.dh_sync())
    capi.check(L.dh_sync())                      # reported once
    for t in lay.out.values():
        t.zero_()
    torch.cuda.synchronize()
    capi.check(L.dh_q4k_gemv_chain(x0, arr, 4))
    capi.check(L.dh_sync())
    for k, v in lay.out.items():
        assert _read(v).tobytes() == good[k].tobytes(), k


def test_chain_argument_errors():
    L = capi.init(0)
    lay = Layer(2048, 4096, 2048, 3072, seed=7300)
    x0 = lay.d["attn"].data_ptr()
    ph = lay.phases()

    def fails(phases, n, match, x=x0):
        arr = capi.chain_phases(phases)
        with pytest.raises(DopplerHipError, match=match):
            capi.check(L.dh_q4k_gemv_chain(x, arr, n))

    fails(ph, 0, "1..4 products")
    fails(ph + ph[:1], 5, "1..4 products")
    bad = [dict(p) for p in ph]
    bad[1]["K"] = 1024
    fails(bad, 4, "makes N=2048 outputs")
    bad = [dict(p) for p in ph]
    bad[0]["K"] = 2000
    fails(bad, 1, "multiple of 256")
    bad = [dict(p) for p in ph]
    bad[0]["C"] = x0
    fails(bad, 1, "writes over the chain's input")
    bad = [dict(p) for p in ph]
    bad[1]["residual"] = bad[0]["C"]
    fails(bad, 2, "takes no residual")
    bad = [dict(p) for p in ph]
    bad[0]["W"] += 4
    fails(bad, 1, "16-byte aligned")
    short = [dict(W=lay.d["wo"].data_ptr(), C=lay.out["x2"].data_ptr(), N=512, K=1024)]
    fails(short, 1, "too short for a chain")
    with pytest.raises(DopplerHipError, match="workgroups must be"):
        capi.check(L.dh_q4k_gemv_chain_limited(x0, capi.chain_phases(ph), 4, 0, 64))


# ---- the chain's first product fed by the attention's split-K partial results ---------------------------------

class AttnLayer(Layer):
    """A layer whose o-projection input is the decode attention of a step: caches prefilled with seeded
    rows, the step's raw q/k/v in one stacked vector."""

    def __init__(self, H, Hkv, D, Hd, I, ctx_max, seed):
        super().__init__(Hd, I, H * D, (H + 2 * Hkv) * D, seed)
        self.H, self.Hkv, self.D, self.ctx_max = H, Hkv, D, ctx_max
        rng = np.random.default_rng(seed)
        self.cache_k = torch.from_numpy((rng.standard_normal((ctx_max, Hkv * D)) / np.sqrt(D)).astype(np.float16)).cuda()
        self.cache_v = torch.from_numpy((rng.standard_normal((ctx_max, Hkv * D)) / np.sqrt(D)).astype(np.float16)).cuda()
        self.qkv_in = torch.from_numpy(rng.standard_normal((H + 2 * Hkv) * D).astype(np.float32)).cuda()
        self.qw = torch.from_numpy((1 + 0.02 * rng.standard_normal(D)).astype(np.float32)).cuda()
        self.kw = torch.from_numpy((1 + 0.02 * rng.standard_normal(D)).astype(np.float32)).cuda()
        inv = 1.0 / (1e6 ** (np.arange(0, D, 2, dtype=np.float64) / D))
        ang = np.arange(ctx_max, dtype=np.float64)[:, None] * inv[None, :]
        self.cos = torch.from_numpy(np.cos(ang).astype(np.float32)).cuda()
        self.sin = torch.from_numpy(np.sin(ang).astype(np.float32)).cuda()
        L = capi.init(0)
        self.ws = torch.zeros(int(L.dh_attn_decode_workspace_bytes(H, D, ctx_max)), dtype=torch.uint8, device="cuda")
        self.attn_out = f32(H * D)
        self.kvlen = torch.zeros(1, dtype=torch.int32, device="cuda")

    def attn_args(self):
        return (self.qkv_in.data_ptr(), self.qw.data_ptr(), self.kw.data_ptr(), self.cos.data_ptr(), self.sin.data_ptr(),
                self.cache_k.data_ptr(), self.cache_v.data_ptr())

    def tail(self):
        return (self.D, 0, EPS, 0, 1, 1.0 / np.sqrt(self.D), 0.0, 0, 0, capi.KV_CONTIGUOUS, self.ws.data_ptr())


@pytest.mark.parametrize("pos", [0, 63, 700, 2047, 4100])
def test_chain_merges_the_attention_partials_like_the_merge_kernel(pos):
    """attention (merge kernel) -> chain against attention partials -> chain that merges them: same bits in
    every product, with the split count given by the host and with the key count on the device."""
    L = capi.init(0)
    H, Hkv, D = 32, 8, 128
    lay = AttnLayer(H, Hkv, D, 2048, 4096, 4608, seed=7400 + pos)
    assert L.dh_q4k_gemv_chain_attn_supported(H, Hkv, D, lay.ctx_max) == 1
    arr = capi.chain_phases(lay.phases())
    # first a launch at another key count (it appends the step's key/value there, so it comes before the
    # reference is taken): the launches below follow the device word back to this test's position
    lay.kvlen.fill_(max(1, pos // 2))
    torch.cuda.synchronize()
    capi.check(L.dh_attn_decode_qkv_kvlen_partials(*lay.attn_args(), H, Hkv, D, lay.kvlen.data_ptr(), lay.ctx_max, *lay.tail()))
    src = capi.ChainAttnSource(lay.ws.data_ptr(), H, Hkv, D, 0, lay.kvlen.data_ptr(), lay.ctx_max, 0, 0)
    capi.check(L.dh_q4k_gemv_chain_attn(ctypes.byref(src), arr, 4))
    capi.check(L.dh_sync())
    assert all(np.isfinite(_read(v)).all() for v in lay.out.values())
    # reference path: attention with its own merge, then the chain on the merged vector
    capi.check(L.dh_attn_decode_qkv(*lay.attn_args(), lay.attn_out.data_ptr(), H, Hkv, D, pos, *lay.tail()))
    want_out = {k: torch.zeros_like(v) for k, v in lay.out.items()}
    ph = lay.phases(want_out)
    ph[0]["residual"] = lay.d["x"].data_ptr()
    capi.check(L.dh_q4k_gemv_chain(lay.attn_out.data_ptr(), capi.chain_phases(ph), 4))
    capi.check(L.dh_sync())
    want = {k: _read(v) for k, v in want_out.items()}
    assert all(np.isfinite(v).all() for v in want.values())
    # host-known split count
    for t in lay.out.values():
        t.fill_(float("nan"))
    nsplit = ctypes.c_int(0)
    capi.check(L.dh_attn_decode_qkv_partials(*lay.attn_args(), H, Hkv, D, pos, *lay.tail(), ctypes.byref(nsplit)))
    assert 1 <= nsplit.value <= 64
    src = capi.ChainAttnSource(lay.ws.data_ptr(), H, Hkv, D, nsplit.value, None, 0, 0, 0)
    capi.check(L.dh_q4k_gemv_chain_attn(ctypes.byref(src), arr, 4))
    capi.check(L.dh_sync())
    for k, v in lay.out.items():
        assert _read(v).tobytes() == want[k].tobytes(), ("host", k)
    # key count on the device, twice in a row
    for rep in range(2):
        for t in lay.out.values():
            t.fill_(float("nan"))
        lay.kvlen.fill_(pos + 1)
        torch.cuda.synchronize()
        capi.check(L.dh_attn_decode_qkv_kvlen_partials(*lay.attn_args(), H, Hkv, D, lay.kvlen.data_ptr(), lay.ctx_max,
                                                       *lay.tail()))
        src = capi.ChainAttnSource(lay.ws.data_ptr(), H, Hkv, D, 0, lay.kvlen.data_ptr(), lay.ctx_max, 0, 0)
        capi.check(L.dh_q4k_gemv_chain_attn(ctypes.byref(src), arr, 4))
        capi.check(L.dh_sync())
        for k, v in lay.out.items():
            assert _read(v).tobytes() == want[k].tobytes(), ("device", rep, k)


def test_chain_attn_argument_errors():
    L = capi.init(0)
    lay = AttnLayer(32, 8, 128, 2048, 4096, 1024, seed=7500)
    arr = capi.chain_phases(lay.phases())

    def fails(src, match, n=4):
        with pytest.raises(DopplerHipError, match=match):
            capi.check(L.dh_q4k_gemv_chain_attn(ctypes.byref(src), arr, n))

    ws = lay.ws.data_ptr()
    fails(capi.ChainAttnSource(None, 32, 8, 128, 4, None, 0, 0, 0), "workspace is null")
    fails(capi.ChainAttnSource(ws, 16, 8, 128, 4, None, 0, 0, 0), "product 0 takes K=4096")
    fails(capi.ChainAttnSource(ws, 32, 8, 128, 0, None, 0, 0, 0), "nsplit must be at least 1")
    fails(capi.ChainAttnSource(ws, 32, 8, 128, 65, None, 0, 0, 0), "up to 64 splits")
    fails(capi.ChainAttnSource(ws, 32, 8, 128, 0, lay.kvlen.data_ptr(), 0, 0, 0), "max_kv_len >= 1")
    assert L.dh_q4k_gemv_chain_attn_supported(32, 8, 96, 1024) == 0
    assert L.dh_q4k_gemv_chain_attn_supported(32, 5, 128, 1024) == 0
