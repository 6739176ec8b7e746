"""The allocation-free decode attention entry point (dh_attn_decode_static) against
dh_attn_decode with a caller's workspace: same kernels, so the outputs must be bit-identical,
on two calls in a row, the second with a smaller input (the library's fixed scratch keeps the
first call's partials).  Both are also checked against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from doppler_amd import capi, synth

pytestmark = pytest.mark.gpu


def _inputs(H, Hkv, D, ctx, seed):
    cos, sin = synth.rope_tables(D, ctx, 1e6)
    q = synth.normal_f32((1, H, D), seed, D ** -0.5)
    k = synth.normal_f32((ctx, Hkv, D), seed + 1, D ** -0.5)
    v = synth.normal_f32((ctx, Hkv, D), seed + 2, D ** -0.5)
    q = oracle.rope_apply(q, cos, sin, 1, H, D, start_pos=ctx - 1)
    k = oracle.rope_apply(k, cos, sin, ctx, Hkv, D, start_pos=0)
    qf = q.astype(np.float16).astype(np.float32).reshape(H, D)
    return qf, k.astype(np.float16).view(np.uint16), v.astype(np.float16).view(np.uint16)


def _run_both(L, H, Hkv, D, ctx, seed):
    q, kb, vb = _inputs(H, Hkv, D, ctx, seed)
    dq = torch.from_numpy(q).cuda()
    dk = torch.from_numpy(kb.view(np.int16)).cuda()
    dv = torch.from_numpy(vb.view(np.int16)).cuda()
    ws = torch.zeros(int(L.dh_attn_decode_workspace_bytes(H, D, ctx)), dtype=torch.uint8, device="cuda")
    ref = torch.zeros(H * D, dtype=torch.float32, device="cuda")
    got = torch.full((H * D,), float("nan"), dtype=torch.float32, device="cuda")
    scale = 1.0 / np.sqrt(D)
    capi.check(L.dh_attn_decode(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), ref.data_ptr(), H, Hkv, D, ctx, scale, 1,
                                ctx - 1, 0.0, 0, 0, capi.KV_CONTIGUOUS, ws.data_ptr()))
    capi.check(L.dh_attn_decode_static(dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), got.data_ptr(), H, Hkv, D, ctx,
                                       scale, 1, ctx - 1, 0.0, 0, 0, capi.KV_CONTIGUOUS))
    capi.check(L.dh_sync())
    want = oracle.attention_decode_f16kv(q, kb, vb, H, Hkv, D, ctx)
    return ref.cpu().numpy(), got.cpu().numpy(), np.asarray(want, np.float64).reshape(-1)


def test_static_scratch_attention_matches_workspace_attention_twice():
    L = capi.init(torch.cuda.current_device())
    assert L.dh_attn_decode_static_max_bytes() == 4 << 20
    # first call: 32/8 heads over 4096 keys (many splits); second: fewer heads, 300 keys
    for (H, Hkv, D, ctx, seed) in ((32, 8, 128, 4096, 9100), (8, 2, 64, 300, 9200)):
        ref, got, want = _run_both(L, H, Hkv, D, ctx, seed)
        assert np.array_equal(ref.view(np.uint32), got.view(np.uint32)), (H, Hkv, D, ctx)
        err = np.linalg.norm(got - want) / np.linalg.norm(want)
        assert err <= 1e-3, (H, Hkv, D, ctx, err)


def test_static_scratch_attention_rejects_what_does_not_fit():
    L = capi.init(torch.cuda.current_device())
    H, Hkv, D, ctx = 8192, 8192, 128, 4096          # one query head per kv head: 8192 heads x 2 splits = 8.5 MB
    dq = torch.zeros(H * D, dtype=torch.float32, device="cuda")
    dk = torch.zeros(16, dtype=torch.int16, device="cuda")      # never read: the call fails before any launch
    out = torch.zeros(H * D, dtype=torch.float32, device="cuda")
    rc = L.dh_attn_decode_static(dq.data_ptr(), dk.data_ptr(), dk.data_ptr(), out.data_ptr(), H, Hkv, D, ctx,
                                 0.1, 1, ctx - 1, 0.0, 0, 0, capi.KV_CONTIGUOUS)
    assert rc != 0
    msg = L.dh_last_error().decode()
    assert "dh_attn_decode_static" in msg and "scratch holds" in msg
