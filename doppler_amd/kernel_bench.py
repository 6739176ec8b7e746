"""Per-kernel measurements of the HIP path on the benchmark configurations.

    python -m doppler_amd.kernel_bench [--only gemv,chain,gemm,attn,prefill_attn,lmhead,dense] [--json out.jsonl]

Every case is timed with events around back-to-back launches on the library's stream.  Weights
(and KV caches) rotate through enough copies that their total exceeds the 256 MB Infinity Cache
plus the L2s, so "rotating" figures are reads from HBM; "warm" repeats one copy and shows what
the caches add for the small shapes.  Rates use algorithmic bytes (Q4_K weight bytes + f32
activations in and out) or flops (2 M N K per product), never bytes actually moved.

Configurations: 0 = one 640 -> 2048 GEMV; 1 = the linear layers of a hidden-1024 block at
M in {1, 2, 4, 8}; 2 = prefill FFN GEMM at M = 512; 3 = decode attention, 16/8 heads of 128 at
three context lengths; 4 = the GEMVs and the LM head of the 9B-class decoder.
"""
import argparse
import ctypes
import json
import sys

import torch

from . import capi, synth

HBM_PEAK_GBS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
COLD_BYTES = 640 << 20           # rotate through at least this much so nothing stays cached


class Timer:
    def __init__(self, L):
        self.L = L
        self.e0, self.e1 = ctypes.c_void_p(), ctypes.c_void_p()
        capi.check(L.dh_event_create(ctypes.byref(self.e0)))
        capi.check(L.dh_event_create(ctypes.byref(self.e1)))

    def us(self, fn, n):
        L = self.L
        for i in range(3):
            fn(i)
        capi.check(L.dh_sync())
        capi.check(L.dh_event_record(self.e0))
        for i in range(n):
            fn(i)
        capi.check(L.dh_event_record(self.e1))
        capi.check(L.dh_sync())
        ms = ctypes.c_float()
        capi.check(L.dh_event_elapsed_ms(self.e0, self.e1, ctypes.byref(ms)))
        return ms.value * 1e3 / n


def q4k_copies(nbytes, copies):
    """`copies` random Q4_K tensors of nbytes each (finite d/dmin), as views of one buffer."""
    stride = (nbytes + 255) // 256 * 256
    buf = torch.randint(0, 256, (copies * stride,), dtype=torch.uint8, device="cuda")
    views = [buf[i * stride:i * stride + nbytes] for i in range(copies)]
    hdr = torch.tensor([0x00, 0x20, 0x00, 0x20], dtype=torch.uint8, device="cuda")   # d = dmin = 2^-7
    for v in views:
        v.view(-1, synth.Q4K_BLOCK_BYTES)[:, 0:4] = hdr
    return views


def n_copies(nbytes, cap=512):
    return max(2, min(cap, -(-COLD_BYTES // nbytes)))


def emit(rows, **r):
    rows.append(r)
    if r["unit"] == "GB/s":
        r["frac"] = round(r["achieved"] / HBM_PEAK_GBS, 4)
        r["bound"] = "hbm"
    else:
        r["frac"] = round(r["achieved"] / MFMA_F16_PEAK_TFLOPS, 4)
        r["bound"] = "mfma"
    print("%-34s %-28s %-9s %9.2f us %10.1f %-8s %5.1f%% of peak" % (
        r["kernel"], r["shape"], r["mode"], r["us"], r["achieved"], r["unit"], 100 * r["frac"]), flush=True)


def gemv_cases(L, T, rows, reps):
    def run(cfg, name, M, N, K, dual=False, norm=False, residual=False):
        wbytes = synth.q4k_nbytes(N, K)
        nmat = 2 if dual else 1
        algo = nmat * wbytes + M * K * 4 + M * N * 4 + (M * N * 4 if residual else 0) + (K * 4 if norm else 0)
        A = torch.randn(M, K, device="cuda") * (0.05 if dual else 1.0)
        C = torch.zeros(M, N, device="cuda")
        R = torch.randn(M, N, device="cuda") if residual else None
        nw = torch.ones(K, device="cuda") if norm else None
        for mode in ("rotating", "warm"):
            copies = n_copies(nmat * wbytes) * nmat if mode == "rotating" else nmat
            Ws = q4k_copies(wbytes, copies)
            p = [w.data_ptr() for w in Ws]

            def fn(i):
                w = p[(nmat * i) % copies]
                if dual:
                    w2 = p[(nmat * i + 1) % copies]
                    if norm:
                        rc = L.dh_q4k_ffn_gate_up_rmsnorm(A.data_ptr(), nw.data_ptr(), 1e-6, 0, w, w2, C.data_ptr(),
                                                          M, K, N, capi.ACT_SILU, 1.0, 0.0)
                    else:
                        rc = L.dh_q4k_ffn_gate_up(A.data_ptr(), w, w2, C.data_ptr(), M, K, N, capi.ACT_SILU, 1.0, 0.0)
                elif norm:
                    rc = L.dh_q4k_matmul_rmsnorm(A.data_ptr(), nw.data_ptr(), 1e-6, 0, w, C.data_ptr(), 0, M, N, K,
                                                 1.0, R.data_ptr() if residual else None)
                else:
                    rc = L.dh_q4k_matmul(A.data_ptr(), 0, w, C.data_ptr(), 0, M, N, K, 1.0,
                                         R.data_ptr() if residual else None)
                capi.check(rc)

            us = T.us(fn, reps)
            emit(rows, config=cfg, kernel="q4k_gemv " + name, shape="M=%d N=%d K=%d%s" % (M, N, K, " x2" if dual else ""),
                 mode=mode, us=round(us, 3), achieved=round(algo / us / 1e3, 1), unit="GB/s", algorithmic_bytes=algo)
            del Ws

    run(0, "ffn (cfg0)", 1, 2048, 640)
    for M in (1, 2, 4, 8):
        for name, N, K in (("q", 2048, 1024), ("k/v", 1024, 1024), ("o", 1024, 2048), ("gate|up", 3072, 1024),
                           ("down", 1024, 3072)):
            run(1, name + " (cfg1)", M, N, K)
    for M in (1, 2, 4, 8):
        run(4, "norm+qkv (cfg4)", M, 6144, 4096, norm=True)
        run(4, "o+residual (cfg4)", M, 4096, 4096, residual=True)
        run(4, "norm+gate/up+silu (cfg4)", M, 12288, 4096, dual=True, norm=True)
        run(4, "down+residual (cfg4)", M, 4096, 12288, residual=True)


def chain_cases(L, T, rows, reps):
    """The four dependent products of a cfg4 decoder layer as one launch (dh_q4k_gemv_chain) against the
    same products as four launches; weights rotating through enough layers to stay out of the caches."""
    Hd, I, QS, QKV = 4096, 12288, 4096, 6144
    shapes = [(Hd, QS), (I, Hd), (I, Hd), (Hd, I), (QKV, Hd)]                 # o, gate, up, down, next qkv
    per_layer = sum(synth.q4k_nbytes(n, k) for n, k in shapes)
    algo = per_layer + 4 * (QS + 2 * Hd + Hd + Hd + I + I + Hd + Hd + Hd + Hd + QKV)
    f32 = lambda n: torch.zeros(n, device="cuda")
    attn, x, x2, act, x3, qkv = torch.randn(QS, device="cuda") * 0.01, torch.randn(Hd, device="cuda") * 0.01, f32(Hd), f32(I), f32(Hd), f32(QKV)
    n1, n2 = torch.ones(Hd, device="cuda"), torch.ones(Hd, device="cuda")
    for mode in ("rotating", "warm"):
        layers = n_copies(per_layer, 16) if mode == "rotating" else 1
        W = [[q4k_copies(synth.q4k_nbytes(n, k), 1)[0] for n, k in shapes] for _ in range(layers)]
        chains = []
        for wo, wg, wu, wd, wq in W:
            chains.append(capi.chain_phases([
                dict(W=wo.data_ptr(), C=x2.data_ptr(), residual=x.data_ptr(), N=Hd, K=QS),
                dict(W=wg.data_ptr(), W2=wu.data_ptr(), C=act.data_ptr(), norm_weight=n1.data_ptr(), N=I, K=Hd,
                     activation=capi.ACT_SILU, norm_eps=1e-6),
                dict(W=wd.data_ptr(), C=x3.data_ptr(), residual=x2.data_ptr(), N=Hd, K=I),
                dict(W=wq.data_ptr(), C=qkv.data_ptr(), norm_weight=n2.data_ptr(), N=QKV, K=Hd, norm_eps=1e-6)]))

        def chained(i):
            capi.check(L.dh_q4k_gemv_chain(attn.data_ptr(), chains[i % layers], 4))

        def separate(i):
            wo, wg, wu, wd, wq = W[i % layers]
            capi.check(L.dh_q4k_matmul(attn.data_ptr(), 0, wo.data_ptr(), x2.data_ptr(), 0, 1, Hd, QS, 1.0, x.data_ptr()))
            capi.check(L.dh_q4k_ffn_gate_up_rmsnorm(x2.data_ptr(), n1.data_ptr(), 1e-6, 0, wg.data_ptr(), wu.data_ptr(),
                                                    act.data_ptr(), 1, Hd, I, capi.ACT_SILU, 1.0, 0.0))
            capi.check(L.dh_q4k_matmul(act.data_ptr(), 0, wd.data_ptr(), x3.data_ptr(), 0, 1, Hd, I, 1.0, x2.data_ptr()))
            capi.check(L.dh_q4k_matmul_rmsnorm(x3.data_ptr(), n2.data_ptr(), 1e-6, 0, wq.data_ptr(), qkv.data_ptr(), 0, 1, QKV,
                                               Hd, 1.0, None))
        for name, fn in (("q4k_gemv_chain o,gate/up,down,qkv (cfg4)", chained), ("the same as four launches (cfg4)", separate)):
            us = T.us(fn, reps)
            emit(rows, config=4, kernel=name, shape="one decoder layer, M=1", mode=mode, us=round(us, 3),
                 achieved=round(algo / us / 1e3, 1), unit="GB/s", algorithmic_bytes=algo)
        del W, chains


def gemm_cases(L, T, rows, reps):
    M, hidden, inter = 512, 1152, 6912
    cg = n_copies(2 * synth.q4k_nbytes(inter, hidden), 64) * 2
    cd = n_copies(synth.q4k_nbytes(hidden, inter), 64)
    Wg = q4k_copies(synth.q4k_nbytes(inter, hidden), cg)
    Wd = q4k_copies(synth.q4k_nbytes(hidden, inter), cd)
    X = torch.randn(M, hidden, device="cuda") * 0.05
    H = torch.zeros(M, inter, device="cuda")
    Y = torch.zeros(M, hidden, device="cuda")
    t1 = T.us(lambda i: capi.check(L.dh_q4k_ffn_gate_up(X.data_ptr(), Wg[(2 * i) % cg].data_ptr(),
                                                        Wg[(2 * i + 1) % cg].data_ptr(), H.data_ptr(), M, hidden, inter,
                                                        capi.ACT_GELU, 1.0, 0.0)), reps)
    t2 = T.us(lambda i: capi.check(L.dh_q4k_matmul(H.data_ptr(), 0, Wd[i % cd].data_ptr(), Y.data_ptr(), 0, M, hidden,
                                                   inter, 1.0, None)), reps)
    f1, f2 = 2 * 2 * M * inter * hidden, 2 * M * hidden * inter
    emit(rows, config=2, kernel="q4k_gemm gate/up+gelu (cfg2)", shape="M=512 N=6912 K=1152 x2", mode="rotating",
         us=round(t1, 2), achieved=round(f1 / t1 / 1e6, 1), unit="TFLOP/s", flops=f1)
    emit(rows, config=2, kernel="q4k_gemm down (cfg2)", shape="M=512 N=1152 K=6912", mode="rotating",
         us=round(t2, 2), achieved=round(f2 / t2 / 1e6, 1), unit="TFLOP/s", flops=f2)
    emit(rows, config=2, kernel="q4k_gemm FFN total (cfg2)", shape="24.46 GFLOP", mode="rotating",
         us=round(t1 + t2, 2), achieved=round((f1 + f2) / (t1 + t2) / 1e6, 1), unit="TFLOP/s", flops=f1 + f2)
    del Wg, Wd
    for (M2, N2, K2) in ((2048, 12288, 4096), (2048, 4096, 12288)):
        W = q4k_copies(synth.q4k_nbytes(N2, K2), 2)
        A = torch.randn(M2, K2, device="cuda")
        C = torch.zeros(M2, N2, device="cuda")
        t = T.us(lambda i: capi.check(L.dh_q4k_matmul(A.data_ptr(), 0, W[i % 2].data_ptr(), C.data_ptr(), 0, M2, N2, K2,
                                                      1.0, None)), max(4, reps // 8))
        emit(rows, config=4, kernel="q4k_gemm prefill (cfg4 shapes)", shape="M=%d N=%d K=%d" % (M2, N2, K2),
             mode="rotating", us=round(t, 2), achieved=round(2 * M2 * N2 * K2 / t / 1e6, 1), unit="TFLOP/s",
             flops=2 * M2 * N2 * K2)
        del W, A, C


def attn_cases(L, T, rows, reps):
    for (H, Hkv, cfg) in ((16, 8, 3), (32, 8, 4)):
        D = 128
        for ctx in ((512, 4096, 32768) if cfg == 3 else (2048,)):
            kv_bytes = 2 * ctx * Hkv * D * 2
            copies = n_copies(kv_bytes, 320)
            K = torch.randn(copies, ctx, Hkv, D, device="cuda", dtype=torch.float16) * (1.0 / D ** 0.5)
            V = torch.randn(copies, ctx, Hkv, D, device="cuda", dtype=torch.float16) * (1.0 / D ** 0.5)
            q = torch.randn(H, D, device="cuda")
            o = torch.zeros(H, D, device="cuda")
            ws = torch.zeros(int(L.dh_attn_decode_workspace_bytes(H, D, ctx)), dtype=torch.uint8, device="cuda")
            step = ctx * Hkv * D * 2
            for mode in ("rotating", "warm"):
                n = copies if mode == "rotating" else 1
                us = T.us(lambda i: capi.check(L.dh_attn_decode(
                    q.data_ptr(), K.data_ptr() + (i % n) * step, V.data_ptr() + (i % n) * step, o.data_ptr(), H, Hkv, D,
                    ctx, 1.0 / D ** 0.5, 1, ctx - 1, 0.0, 0, 0, 0, ws.data_ptr())), reps)
                algo = kv_bytes + H * D * 8
                emit(rows, config=cfg, kernel="attn_decode (cfg%d)" % cfg, shape="H=%d/%d D=128 ctx=%d" % (H, Hkv, ctx),
                     mode=mode, us=round(us, 3), achieved=round(algo / us / 1e3, 1), unit="GB/s", algorithmic_bytes=algo)
            if ctx >= 2048:
                # the same step taken straight from the stacked projection (q/k norm, RoPE and KV append inside)
                qkv = torch.randn((H + 2 * Hkv) * D, device="cuda")
                w = torch.ones(D, device="cuda")
                cs = torch.rand(ctx, D // 2, device="cuda")
                for mode in ("rotating", "warm"):
                    n = copies if mode == "rotating" else 1
                    us = T.us(lambda i: capi.check(L.dh_attn_decode_qkv(
                        qkv.data_ptr(), w.data_ptr(), w.data_ptr(), cs.data_ptr(), cs.data_ptr(),
                        K.data_ptr() + (i % n) * step, V.data_ptr() + (i % n) * step, o.data_ptr(), H, Hkv, D, ctx - 1, D, 0,
                        1e-6, 0, 1, 1.0 / D ** 0.5, 0.0, 0, 0, 0, ws.data_ptr())), reps)
                    algo = kv_bytes + (H + 2 * Hkv) * D * 4 + H * D * 4
                    emit(rows, config=cfg, kernel="attn_decode_qkv (cfg%d)" % cfg, shape="H=%d/%d D=128 ctx=%d" % (H, Hkv, ctx),
                         mode=mode, us=round(us, 3), achieved=round(algo / us / 1e3, 1), unit="GB/s", algorithmic_bytes=algo)
                if cfg == 4:
                    # what the decoder launches: the split kernel alone, its partial results left for the
                    # chained launch that follows (which merges them: + ~1.5 us there, see the chain rows)
                    nsplit = ctypes.c_int(0)
                    for mode in ("rotating", "warm"):
                        n = copies if mode == "rotating" else 1
                        us = T.us(lambda i: capi.check(L.dh_attn_decode_qkv_partials(
                            qkv.data_ptr(), w.data_ptr(), w.data_ptr(), cs.data_ptr(), cs.data_ptr(),
                            K.data_ptr() + (i % n) * step, V.data_ptr() + (i % n) * step, H, Hkv, D, ctx - 1, D, 0,
                            1e-6, 0, 1, 1.0 / D ** 0.5, 0.0, 0, 0, 0, ws.data_ptr(), ctypes.byref(nsplit))), reps)
                        emit(rows, config=cfg, kernel="attn_decode_qkv partials only (cfg%d)" % cfg,
                             shape="H=%d/%d D=128 ctx=%d" % (H, Hkv, ctx), mode=mode, us=round(us, 3),
                             achieved=round(algo / us / 1e3, 1), unit="GB/s", algorithmic_bytes=algo)
            del K, V


def attn_prefill_cases(L, T, rows, reps):
    """Causal prefill attention from an empty cache: flops = 4 H D sum_t (t + 1)."""
    D = 128
    for (H, Hkv, Tq, cfg) in ((16, 8, 512, 3), (16, 8, 4096, 3), (32, 8, 2048, 4)):
        K = torch.randn(Tq, Hkv, D, device="cuda", dtype=torch.float16) * (1.0 / D ** 0.5)
        V = torch.randn(Tq, Hkv, D, device="cuda", dtype=torch.float16) * (1.0 / D ** 0.5)
        q = torch.randn(Tq, H, D, device="cuda")
        o = torch.zeros(Tq, H, D, device="cuda")
        us = T.us(lambda i: capi.check(L.dh_attn_prefill(q.data_ptr(), K.data_ptr(), V.data_ptr(), o.data_ptr(), Tq, H, Hkv,
                                                         D, Tq, 1.0 / D ** 0.5, 1, 0, 0.0, 0)), max(8, reps // 4))
        flops = 4 * H * D * Tq * (Tq + 1) // 2
        emit(rows, config=cfg, kernel="attn_prefill causal (cfg%d heads)" % cfg, shape="H=%d/%d D=128 T=%d" % (H, Hkv, Tq),
             mode="warm", us=round(us, 2), achieved=round(flops / us / 1e6, 1), unit="TFLOP/s", flops=flops)


def lmhead_cases(L, T, rows, reps):
    vocab, hidden = 151936, 4096
    E = (torch.randn(vocab, hidden, device="cuda") * 0.02).half()
    h = torch.randn(hidden, device="cuda")
    ws = torch.zeros(int(L.dh_lmhead_argmax_workspace_bytes(vocab)), dtype=torch.uint8, device="cuda")
    tok = torch.zeros(4, dtype=torch.int32, device="cuda")
    us = T.us(lambda i: capi.check(L.dh_lmhead_argmax_f16(h.data_ptr(), E.data_ptr(), vocab, hidden, -1, 0.0,
                                                          ws.data_ptr(), tok.data_ptr(), 0, None)), max(8, reps // 8))
    algo = vocab * hidden * 2 + hidden * 4
    emit(rows, config=4, kernel="lm_head+argmax f16 (cfg4)", shape="V=151936 K=4096", mode="rotating",
         us=round(us, 2), achieved=round(algo / us / 1e3, 1), unit="GB/s", algorithmic_bytes=algo)


def sample_cases(L, T, rows, reps):
    vocab = 151936
    logits = torch.randn(vocab, device="cuda") * 3
    tok = torch.zeros(4, dtype=torch.int32, device="cuda")
    for k in (40, 256):
        ws = torch.zeros(int(L.dh_sample_topk_workspace_bytes(vocab, k)), dtype=torch.uint8, device="cuda")
        us = T.us(lambda i: capi.check(L.dh_sample_topk(logits.data_ptr(), vocab, 0.8, k, 0.37, -1, 0.0, ws.data_ptr(),
                                                        tok.data_ptr(), 0)), max(8, reps // 4))
        algo = vocab * 4
        emit(rows, config=4, kernel="sample top-k (vocab 151936)", shape="topK=%d T=0.8" % k, mode="warm", us=round(us, 2),
             achieved=round(algo / us / 1e3, 1), unit="GB/s", algorithmic_bytes=algo)


def dense_cases(L, T, rows, reps):
    """Dense f32 matmul + RMSNorm over the output row (one activation row), f16 activations into the
    Q4_K matmul, and the finiteness check of one hidden row."""
    for N, K in ((1152, 6912), (4096, 8192)):
        copies = n_copies(N * K * 4, 16)
        Ws = [torch.randn(N * K, device="cuda") * K ** -0.5 for _ in range(copies)]
        x = torch.randn(K, device="cuda")
        nw, res, out = torch.randn(N, device="cuda"), torch.randn(N, device="cuda"), torch.zeros(N, device="cuda")
        algo = N * K * 4 + K * 4 + 3 * N * 4
        for tb in (1, 0):
            us = T.us(lambda i: capi.check(L.dh_matmul_rmsnorm_f32(x.data_ptr(), Ws[i % copies].data_ptr(), tb,
                                                                   nw.data_ptr(), capi.F32, 1e-6, 1, res.data_ptr(),
                                                                   out.data_ptr(), N, K)), max(8, reps // 4))
            emit(rows, config=4, kernel="dense matmul+rmsnorm f32", shape="N=%d K=%d %s" % (N, K, "[N,K]" if tb else "[K,N]"),
                 mode="rotating", us=round(us, 2), achieved=round(algo / us / 1e3, 1), unit="GB/s", algorithmic_bytes=algo)
        del Ws
        Wh = [(torch.randn(N * K, device="cuda") * K ** -0.5).half() for _ in range(2 * copies)]
        xh, resh, outh = x.half(), res.half(), torch.zeros(N, dtype=torch.float16, device="cuda")
        algo = N * K * 2 + K * 2 + N * 4 + 2 * N * 2
        for tb in (1, 0):
            us = T.us(lambda i: capi.check(L.dh_matmul_rmsnorm_f16(xh.data_ptr(), Wh[i % (2 * copies)].data_ptr(), tb,
                                                                   nw.data_ptr(), capi.F32, 1e-6, 1, resh.data_ptr(),
                                                                   outh.data_ptr(), N, K)), max(8, reps // 4))
            emit(rows, config=4, kernel="dense matmul+rmsnorm f16", shape="N=%d K=%d %s" % (N, K, "[N,K]" if tb else "[K,N]"),
                 mode="rotating", us=round(us, 2), achieved=round(algo / us / 1e3, 1), unit="GB/s", algorithmic_bytes=algo)
        del Wh
    M, N, K = 4, 6144, 1536
    nbytes = synth.q4k_nbytes(N, K)
    copies = n_copies(nbytes)
    Ws = q4k_copies(nbytes, copies)
    a16 = torch.randn(M * K, device="cuda").half()
    a32 = a16.float()
    c = torch.zeros(M * N, dtype=torch.float16, device="cuda")
    algo = nbytes + M * K * 2 + M * N * 2
    for name, a, dt in (("q4k matmul f16 activations", a16, capi.F16), ("q4k matmul f32 activations", a32, capi.F32)):
        us = T.us(lambda i: capi.check(L.dh_q4k_matmul(a.data_ptr(), dt, Ws[i % copies].data_ptr(), c.data_ptr(), capi.F16,
                                                       M, N, K, 1.0, None)), reps)
        emit(rows, config=1, kernel=name, shape="M=%d N=%d K=%d" % (M, N, K), mode="rotating", us=round(us, 2),
             achieved=round((algo + (M * K * 2 if dt == capi.F32 else 0)) / us / 1e3, 1), unit="GB/s",
             algorithmic_bytes=algo + (M * K * 2 if dt == capi.F32 else 0))
    h = torch.randn(4096, device="cuda")
    status = torch.zeros(4, dtype=torch.int32, device="cuda")
    us = T.us(lambda i: capi.check(L.dh_check_finiteness(h.data_ptr(), capi.F32, 4096, status.data_ptr(), 0, i, 65500.0)), reps)
    emit(rows, config=4, kernel="check_finiteness f32", shape="hidden=4096", mode="warm", us=round(us, 2),
         achieved=round(4096 * 4 / us / 1e3, 1), unit="GB/s", algorithmic_bytes=4096 * 4)


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--only", default="gemv,chain,gemm,attn,prefill_attn,lmhead,dense")
    ap.add_argument("--reps", type=int, default=96)
    ap.add_argument("--json", default=None, help="also write one JSON object per case to this file")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("kernel_bench needs a GPU")
    L = capi.init(0)
    T = Timer(L)
    rows = []
    which = set(args.only.split(","))
    if "gemv" in which:
        gemv_cases(L, T, rows, args.reps)
    if "chain" in which:
        chain_cases(L, T, rows, args.reps)
    if "gemm" in which:
        gemm_cases(L, T, rows, max(8, args.reps // 4))
    if "attn" in which:
        attn_cases(L, T, rows, args.reps)
    if "prefill_attn" in which:
        attn_prefill_cases(L, T, rows, args.reps)
    if "lmhead" in which:
        lmhead_cases(L, T, rows, args.reps)
        sample_cases(L, T, rows, args.reps)
    if "dense" in which:
        dense_cases(L, T, rows, args.reps)
    if args.json:
        with open(args.json, "w") as f:
            for r in rows:
                f.write(json.dumps(r) + "\n")


if __name__ == "__main__":
    main()
