"""Single-stream greedy decoder for a Q4_K transformer, built only from the C-ABI ops.

Op order per layer follows the reference's execution graph for Qwen3-class models
(src/config/conversion/qwen3/qwen-3-embedding-0-6b-q4k-ehf16-af32.json `execution.decode`,
driven by src/inference/pipelines/text/generator-steps.js:588-820 decodeStep):

    gather -> [ input_norm -> q,k,v (one fused Q4_K GEMV over the stacked rows) ->
                q/k RMSNorm + RoPE + f16 KV write -> decode attention -> o_proj (+residual) ->
                post_attn_norm -> gate,up + SiLU gate (fused) -> down_proj (+residual) ] x L
           -> final_norm -> tied f16 LM head + argmax -> 4-byte token readback

All buffers are allocated once; a step enqueues ~8 launches per layer on the library's
stream and reads back one token id, the reference's only device->host crossing per token.
"""
import ctypes
import math
import warnings

import numpy as np
import torch

from . import capi, synth

_P = ctypes.c_void_p


def _dev_bytes(arr):
    """Upload a numpy array into a fresh torch.uint8 CUDA buffer."""
    arr = np.ascontiguousarray(arr)
    with warnings.catch_warnings():
        # read-only sources (memory-mapped shards) are only read from here
        warnings.filterwarnings("ignore", message="The given NumPy array is not writable")
        t = torch.from_numpy(arr.view(np.uint8).reshape(-1)).cuda()
    return t


class FinitenessError(RuntimeError):
    """An activation left the f16 range (or the configured bound) during a decode step:
    src/inference/pipelines/text/generator-steps.js:164-169."""


class HipDecoder:
    TOKEN_RING = 64      # tokens one decode_batch submit can produce

    def __init__(self, cfg, layers, embed_bits, final_norm, cos, sin, max_seq, fuse_norm=True,
                 fuse_qkv_attention=True, finiteness_guard=False, finiteness_abs_threshold=None, chain_gemvs=None,
                 chain_merge_attention=True):
        """cfg: dict(layers, hidden, inter, heads, kv_heads, head_dim, vocab, eps, qk_norm);
        layers: list of dicts of numpy arrays (wq, wk, wv, wo, wgate, wup, wdown: Q4_K bytes;
        input_norm, post_attn_norm, q_norm, k_norm: f32); embed_bits: uint16 [vocab, hidden].
        finiteness_guard: check every layer's output against the overflow bound (one more launch
        per layer) and read the 4-word status back beside the token, as the reference does when
        activations are f16 (src/inference/pipelines/text/layer.js:1237-1252,
        generator-steps.js:786-798, :837-843); off by default, the activations here are f32.
        chain_gemvs: see set_chain_gemvs; None (default) turns it on where it is served."""
        self.cfg = dict(cfg)
        self.chain_gemvs = False
        self.chain_merges_attention = False
        self.finiteness_guard = bool(finiteness_guard)
        self.finiteness_abs_threshold = float(finiteness_abs_threshold) if finiteness_abs_threshold else 65500.0
        # RMSNorm runs inside the q/k/v and gate/up GEMVs (their prologue) unless told otherwise
        self.fuse_norm = fuse_norm
        self.L = capi.init(torch.cuda.current_device())
        c = self.cfg
        # decode steps: q/k norm + RoPE + KV append run inside the attention kernel when the head
        # geometry allows it (one launch fewer per layer)
        self.fuse_qkv_attention = bool(fuse_qkv_attention and self.L.dh_attn_decode_qkv_supported(
            c["heads"], c["kv_heads"], c["head_dim"], c["head_dim"], 0))
        self.max_seq = max_seq
        H, Hkv, D, Hd, I = c["heads"], c["kv_heads"], c["head_dim"], c["hidden"], c["inter"]
        if chain_gemvs is None:
            chain_gemvs = self.chain_gemvs_served()
        self.set_chain_gemvs(chain_gemvs, chain_merge_attention)
        self.qs, self.ks = H * D, Hkv * D
        self.layers = []
        for l in layers:
            d = {}
            # q, k, v rows stacked: one GEMV produces the fused qkv vector the K8 kernel consumes
            d["wqkv"] = _dev_bytes(np.concatenate([l["wq"], l["wk"], l["wv"]]))
            d["wo"] = _dev_bytes(l["wo"])
            d["wgate"] = _dev_bytes(l["wgate"])
            d["wup"] = _dev_bytes(l["wup"])
            d["wdown"] = _dev_bytes(l["wdown"])
            for n in ("input_norm", "post_attn_norm", "q_norm", "k_norm"):
                d[n] = _dev_bytes(l[n].astype(np.float32))
            d["cache_k"] = torch.zeros(max_seq * self.ks, dtype=torch.float16, device="cuda")
            d["cache_v"] = torch.zeros(max_seq * self.ks, dtype=torch.float16, device="cuda")
            self.layers.append(d)
        self.embed = _dev_bytes(embed_bits)
        self.final_norm = _dev_bytes(final_norm.astype(np.float32))
        self.cos = _dev_bytes(cos[:max_seq])
        self.sin = _dev_bytes(sin[:max_seq])
        f32 = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")
        self.x = f32(Hd)            # residual stream
        self.x2 = f32(Hd)
        self.normed = f32(Hd)
        self.qkv = f32(self.qs + 2 * self.ks)
        self.q = f32(self.qs)
        self.attn = f32(self.qs)
        self.act = f32(I)
        self.logits = f32(c["vocab"])
        # sampled tokens, then the finiteness status [status, layer, step, pad]: a single step
        # with the guard on puts its token in the ring's last slot, so that one 20-byte read
        # brings token and status back together
        self.token = torch.zeros(self.TOKEN_RING + 4, dtype=torch.int32, device="cuda")
        self.ids = torch.zeros(4, dtype=torch.int32, device="cuda")
        self.attn_ws = torch.zeros(int(self.L.dh_attn_decode_workspace_bytes(H, D, max_seq)), dtype=torch.uint8,
                                   device="cuda")
        self.lm_ws = torch.zeros(int(self.L.dh_lmhead_argmax_workspace_bytes(c["vocab"])), dtype=torch.uint8,
                                 device="cuda")
        self.scale = 1.0 / math.sqrt(D)
        self._host_token = np.zeros(1, np.uint32)
        self._host_ids = np.zeros(2, np.uint32)
        torch.cuda.synchronize()

    def chain_gemvs_served(self):
        """Whether set_chain_gemvs(True) accepts this model: hidden, FFN and attention widths that are
        multiples of 256 in 2048..32768, norms fused, finiteness guard off."""
        c = self.cfg
        dims = (c["hidden"], c["inter"], c["heads"] * c["head_dim"])
        return bool(all(k % 256 == 0 and 2048 <= k <= 32768 for k in dims) and self.fuse_norm and not self.finiteness_guard)

    def set_chain_gemvs(self, on, merge_attention=True):
        """on: the four products between two attentions (o, gate/up, down, next q/k/v) go out as one
        dh_q4k_gemv_chain launch (same bits as the separate launches).  merge_attention: the chain's first
        product also merges the attention's key splits itself, from the partial results the attention
        leaves in its workspace (dh_q4k_gemv_chain_attn: two launches per layer instead of six), where
        the fused attention serves the head geometry and its splits fit."""
        c = self.cfg
        if on and not self.chain_gemvs_served():
            raise ValueError("chain_gemvs serves hidden, FFN and attention widths that are multiples of 256 in "
                             "2048..32768, with the norms fused and the finiteness guard off (got %s)"
                             % ((c["hidden"], c["inter"], c["heads"] * c["head_dim"]),))
        self.chain_gemvs = bool(on)
        self.chain_merges_attention = bool(on and merge_attention and self.fuse_qkv_attention and
                                           self.L.dh_q4k_gemv_chain_attn_supported(c["heads"], c["kv_heads"], c["head_dim"],
                                                                                   self.max_seq))
        self._chains = {}

    def weight_bytes_per_token(self, ctx):
        """Algorithmic HBM bytes one decode step must read: all Q4_K weights, the f16 LM head
        and the KV cache rows up to ctx."""
        c = self.cfg
        q4 = 0
        for (n, k) in ((self.qs + 2 * self.ks, c["hidden"]), (c["hidden"], self.qs), (c["inter"], c["hidden"]),
                       (c["inter"], c["hidden"]), (c["hidden"], c["inter"])):
            q4 += synth.q4k_nbytes(n, k)
        return c["layers"] * q4 + c["vocab"] * c["hidden"] * 2 + c["layers"] * 2 * self.ks * 2 * ctx

    def enqueue_step(self, pos, want_logits=False, from_device_token=False, in_index=0, out_index=0,
                     device_kv_len=False):
        """Enqueue one decode step for the token id in self.ids[0] (or, when from_device_token,
        the argmax an earlier step left in self.token[in_index]) at position `pos`; the new
        token goes to self.token[out_index].  No host synchronisation.  device_kv_len: the
        attention kernels take the key count (position + 1) from self.ids[1] instead of `pos`, so
        that the enqueued step, captured into a graph, serves every later position as it is."""
        L, c = self.L, self.cfg
        ck = capi.check
        H, Hkv, D, Hd, I = c["heads"], c["kv_heads"], c["head_dim"], c["hidden"], c["inter"]
        if not 0 <= pos < self.max_seq:
            # the ops take no cache capacity: a position past the caches would write K/V and read
            # the rotary tables out of bounds
            raise ValueError("decode position %d is outside the KV cache (max_seq=%d)" % (pos, self.max_seq))
        ids = self.token if from_device_token else self.ids
        ck(L.dh_gather_f16(ids.data_ptr(), self.embed.data_ptr(), self.x.data_ptr(), 1, Hd, c["vocab"],
                           in_index if from_device_token else 0))
        self._out_index = out_index
        x, x2 = self.x, self.x2
        if self.chain_gemvs and self.fuse_norm and not self.finiteness_guard:
            self._enqueue_layers_chained(pos, device_kv_len)
        else:
            self._enqueue_layers(pos, device_kv_len)
        self._enqueue_head(x.data_ptr(), self._out_index, self.logits.data_ptr() if want_logits else None)

    def _enqueue_head(self, hidden_ptr, out_index, logits_ptr):
        """Final RMSNorm + tied f16 LM head + argmax of one hidden row (recordLogitsGPU + recordLmHeadArgmaxF16,
        src/inference/pipelines/text/logits/gpu.js:1122-1157): one launch with the norm inside the LM head kernel
        where the hidden size allows it, else the norm as a launch of its own in front."""
        L, c, ck = self.L, self.cfg, capi.check
        Hd = c["hidden"]
        if Hd <= 4096 and Hd % 8 == 0:
            ck(L.dh_lmhead_argmax_f16_rmsnorm(hidden_ptr, self.final_norm.data_ptr(), c["eps"], 0, self.embed.data_ptr(),
                                              c["vocab"], Hd, -1, 0.0, self.lm_ws.data_ptr(), self.token.data_ptr(),
                                              out_index, logits_ptr))
            return
        ck(L.dh_rmsnorm(hidden_ptr, self.final_norm.data_ptr(), capi.F32, self.normed.data_ptr(), 1, Hd, c["eps"],
                        0, None, None, None, 1.0))
        ck(L.dh_lmhead_argmax_f16(self.normed.data_ptr(), self.embed.data_ptr(), c["vocab"], Hd, -1, 0.0,
                                  self.lm_ws.data_ptr(), self.token.data_ptr(), out_index, logits_ptr))

    def _enqueue_layers(self, pos, device_kv_len):
        L, c, ck = self.L, self.cfg, capi.check
        Hd, I = c["hidden"], c["inter"]
        x, x2 = self.x, self.x2
        for li, d in enumerate(self.layers):
            if self.fuse_norm:
                ck(L.dh_q4k_matmul_rmsnorm(x.data_ptr(), d["input_norm"].data_ptr(), c["eps"], 0,
                                           d["wqkv"].data_ptr(), self.qkv.data_ptr(), capi.F32, 1,
                                           self.qs + 2 * self.ks, Hd, 1.0, None))
            else:
                ck(L.dh_rmsnorm(x.data_ptr(), d["input_norm"].data_ptr(), capi.F32, self.normed.data_ptr(), 1, Hd,
                                c["eps"], 0, None, None, None, 1.0))
                ck(L.dh_q4k_matmul(self.normed.data_ptr(), capi.F32, d["wqkv"].data_ptr(), self.qkv.data_ptr(),
                                   capi.F32, 1, self.qs + 2 * self.ks, Hd, 1.0, None))
            self._enqueue_attention(d, pos, device_kv_len)
            ck(L.dh_q4k_matmul(self.attn.data_ptr(), capi.F32, d["wo"].data_ptr(), x2.data_ptr(), capi.F32, 1, Hd,
                               self.qs, 1.0, x.data_ptr()))
            if self.fuse_norm:
                ck(L.dh_q4k_ffn_gate_up_rmsnorm(x2.data_ptr(), d["post_attn_norm"].data_ptr(), c["eps"], 0,
                                                d["wgate"].data_ptr(), d["wup"].data_ptr(), self.act.data_ptr(),
                                                1, Hd, I, capi.ACT_SILU, 1.0, 0.0))
            else:
                ck(L.dh_rmsnorm(x2.data_ptr(), d["post_attn_norm"].data_ptr(), capi.F32, self.normed.data_ptr(), 1,
                                Hd, c["eps"], 0, None, None, None, 1.0))
                ck(L.dh_q4k_ffn_gate_up(self.normed.data_ptr(), d["wgate"].data_ptr(), d["wup"].data_ptr(),
                                        self.act.data_ptr(), 1, Hd, I, capi.ACT_SILU, 1.0, 0.0))
            ck(L.dh_q4k_matmul(self.act.data_ptr(), capi.F32, d["wdown"].data_ptr(), x.data_ptr(), capi.F32, 1, Hd, I,
                               1.0, x2.data_ptr()))
            if self.finiteness_guard:
                ck(L.dh_check_finiteness(x.data_ptr(), capi.F32, Hd, self.token.data_ptr() + 4 * self.TOKEN_RING, li,
                                         pos, self.finiteness_abs_threshold))

    def _chain_phases(self, li):
        """o-projection, gate/up, down-projection of layer li and the q/k/v projection of layer li + 1 as
        the products of one dh_q4k_gemv_chain launch (built once per layer and kept)."""
        if li not in self._chains:
            c, d = self.cfg, self.layers[li]
            Hd, I = c["hidden"], c["inter"]
            ph = [dict(W=d["wo"].data_ptr(), C=self.x2.data_ptr(), residual=self.x.data_ptr(), N=Hd, K=self.qs),
                  dict(W=d["wgate"].data_ptr(), W2=d["wup"].data_ptr(), C=self.act.data_ptr(),
                       norm_weight=d["post_attn_norm"].data_ptr(), N=I, K=Hd, activation=capi.ACT_SILU, norm_eps=c["eps"]),
                  dict(W=d["wdown"].data_ptr(), C=self.x.data_ptr(), residual=self.x2.data_ptr(), N=Hd, K=I)]
            if li + 1 < len(self.layers):
                n = self.layers[li + 1]
                ph.append(dict(W=n["wqkv"].data_ptr(), C=self.qkv.data_ptr(), norm_weight=n["input_norm"].data_ptr(),
                               N=self.qs + 2 * self.ks, K=Hd, norm_eps=c["eps"]))
            self._chains[li] = (capi.chain_phases(ph), len(ph))
        return self._chains[li]

    def _enqueue_layers_chained(self, pos, device_kv_len):
        L, c, ck = self.L, self.cfg, capi.check
        H, Hkv, D = c["heads"], c["kv_heads"], c["head_dim"]
        use_norm = int(c.get("qk_norm", 1))
        d0 = self.layers[0]
        ck(L.dh_q4k_matmul_rmsnorm(self.x.data_ptr(), d0["input_norm"].data_ptr(), c["eps"], 0, d0["wqkv"].data_ptr(),
                                   self.qkv.data_ptr(), capi.F32, 1, self.qs + 2 * self.ks, c["hidden"], 1.0, None))
        for li, d in enumerate(self.layers):
            arr, n = self._chain_phases(li)
            # (a captured step with the position in the launch arguments keeps the attention's own merge:
            # the library moves that launch with the position, a split count handed to the chain it could not)
            if not self.chain_merges_attention or (getattr(self, "_capturing", False) and not device_kv_len):
                self._enqueue_attention(d, pos, device_kv_len)
                ck(L.dh_q4k_gemv_chain(self.attn.data_ptr(), arr, n))
                continue
            # the key splits' partial results stay in the workspace; the chain's first waves merge them
            src = capi.ChainAttnSource(self.attn_ws.data_ptr(), H, Hkv, D, 0, None, 0, 0, 0)
            if device_kv_len:
                ck(L.dh_attn_decode_qkv_kvlen_partials(
                    self.qkv.data_ptr(), d["q_norm"].data_ptr(), d["k_norm"].data_ptr(), self.cos.data_ptr(),
                    self.sin.data_ptr(), d["cache_k"].data_ptr(), d["cache_v"].data_ptr(), H, Hkv, D,
                    self.ids.data_ptr() + 4, self.max_seq, D, 0, c["eps"], 0, use_norm, self.scale, 0.0, 0, 0,
                    capi.KV_CONTIGUOUS, self.attn_ws.data_ptr()))
                src.d_kv_len = self.ids.data_ptr() + 4
                src.max_kv_len = self.max_seq
            else:
                nsplit = ctypes.c_int(0)
                ck(L.dh_attn_decode_qkv_partials(
                    self.qkv.data_ptr(), d["q_norm"].data_ptr(), d["k_norm"].data_ptr(), self.cos.data_ptr(),
                    self.sin.data_ptr(), d["cache_k"].data_ptr(), d["cache_v"].data_ptr(), H, Hkv, D, pos, D, 0, c["eps"],
                    0, use_norm, self.scale, 0.0, 0, 0, capi.KV_CONTIGUOUS, self.attn_ws.data_ptr(), ctypes.byref(nsplit)))
                src.nsplit = nsplit.value
            ck(L.dh_q4k_gemv_chain_attn(ctypes.byref(src), arr, n))

    def _enqueue_attention(self, d, pos, device_kv_len=False):
        """self.qkv (raw stacked projection of the step's token) -> self.attn, appending the
        token's key/value to the layer's cache."""
        L, c, ck = self.L, self.cfg, capi.check
        H, Hkv, D = c["heads"], c["kv_heads"], c["head_dim"]
        use_norm = int(c.get("qk_norm", 1))
        if device_kv_len:
            if not self.fuse_qkv_attention:
                raise ValueError("the device-side key count serves the fused attention kernel")
            ck(L.dh_attn_decode_qkv_kvlen(self.qkv.data_ptr(), d["q_norm"].data_ptr(), d["k_norm"].data_ptr(),
                                          self.cos.data_ptr(), self.sin.data_ptr(), d["cache_k"].data_ptr(),
                                          d["cache_v"].data_ptr(), self.attn.data_ptr(), H, Hkv, D,
                                          self.ids.data_ptr() + 4, self.max_seq, D, 0, c["eps"], 0, use_norm, self.scale,
                                          0.0, 0, 0, capi.KV_CONTIGUOUS, self.attn_ws.data_ptr()))
            return
        if self.fuse_qkv_attention:
            ck(L.dh_attn_decode_qkv(self.qkv.data_ptr(), d["q_norm"].data_ptr(), d["k_norm"].data_ptr(),
                                    self.cos.data_ptr(), self.sin.data_ptr(), d["cache_k"].data_ptr(),
                                    d["cache_v"].data_ptr(), self.attn.data_ptr(), H, Hkv, D, pos, D, 0, c["eps"], 0,
                                    use_norm, self.scale, 0.0, 0, 0, capi.KV_CONTIGUOUS, self.attn_ws.data_ptr()))
            return
        ck(L.dh_qkv_norm_rope_kvwrite(self.qkv.data_ptr(), d["q_norm"].data_ptr(), d["k_norm"].data_ptr(),
                                      self.cos.data_ptr(), self.sin.data_ptr(), self.q.data_ptr(),
                                      d["cache_k"].data_ptr(), d["cache_v"].data_ptr(), 1, H, Hkv, D, pos, D, 0,
                                      c["eps"], 0, pos * self.ks, use_norm))
        ck(L.dh_attn_decode(self.q.data_ptr(), d["cache_k"].data_ptr(), d["cache_v"].data_ptr(),
                            self.attn.data_ptr(), H, Hkv, D, pos + 1, self.scale, 1, pos, 0.0, 0, 0,
                            capi.KV_CONTIGUOUS, self.attn_ws.data_ptr()))

    def set_token(self, token, kv_len=None):
        """Token id of the step (and, for a captured step, its key count beside it: one upload)."""
        self._host_ids[0] = token
        self._host_ids[1] = 0 if kv_len is None else kv_len
        capi.check(self.L.dh_upload(self.ids.data_ptr(), 0, self._host_ids.ctypes.data, 4 if kv_len is None else 8))

    def read_token(self):
        capi.check(self.L.dh_download(self._host_token.ctypes.data, self.token.data_ptr(), 0, 4))
        return int(self._host_token[0])

    def _reset_finiteness(self):
        capi.check(self.L.dh_fill_zero(self.token.data_ptr(), 4 * self.TOKEN_RING, 16))

    def _raise_if_triggered(self, words, offset, what):
        from . import ops
        st = ops.parseFinitenessStatusWords(words, offset)
        if st["triggered"]:
            raise FinitenessError("F16 bounds exceeded during %s%s" % (what, st["metadata"]))

    def step(self, token, pos, want_logits=False, sampling=None):
        """One full step with the reference's single device->host crossing (the token id, with
        the finiteness status beside it when the guard is on).
        sampling = dict(temperature, topK, randomSeed): top-k temperature sampling from the
        step's logits instead of the fused greedy argmax."""
        self.set_token(token)
        out_index = 0
        if self.finiteness_guard:
            self._reset_finiteness()
            out_index = self.TOKEN_RING - 1
        self.enqueue_step(pos, want_logits or sampling is not None, out_index=out_index)
        if sampling is not None:
            self._enqueue_sample(sampling, out_index)
        if not self.finiteness_guard:
            return self.read_token()
        # staging layout of the reference: [token, status, layer, step, pad]
        words = np.empty(5, np.uint32)
        capi.check(self.L.dh_download(words.ctypes.data, self.token.data_ptr(), 4 * out_index, 20))
        self._raise_if_triggered(words, 1, "generation")
        return int(words[0])

    def decode_greedy(self, token, pos, n):
        """n greedy steps starting with `token` at position `pos`; returns the n new token ids.  Every
        step's token is read back (4 bytes per step, as in step()), but one step late: step k + 1 takes its
        input token from device memory and is enqueued before the host waits for token k, whose copy into
        pinned memory was enqueued behind step k, so the GPU never waits for the host between steps (the
        reference stages its token readbacks through a ring the same way, src/inference/decode-ring.js:141-177).
        A caller with a stop condition checks the tokens as they come and drops the one step in flight."""
        if n <= 0:
            return []
        if self.finiteness_guard:
            out = []
            for k in range(n):
                token = self.step(token, pos + k)
                out.append(token)
            return out
        L, ck, R, E = self.L, capi.check, self.TOKEN_RING, 4
        if getattr(self, "_pinned", None) is None:
            p = ctypes.c_void_p()
            ck(L.dh_host_alloc(4 * R, ctypes.byref(p)))
            self._pinned = p
            self._pinned_tokens = (ctypes.c_uint32 * R).from_address(p.value)
            self._read_events = []
            for _ in range(E):
                e = ctypes.c_void_p()
                ck(L.dh_event_create(ctypes.byref(e)))
                self._read_events.append(e)

        def enqueue_read(k):
            slot = k % R
            ck(L.dh_download_async(self._pinned.value + 4 * slot, self.token.data_ptr(), 4 * slot, 4))
            ck(L.dh_event_record(self._read_events[k % E]))

        def wait_read(k):
            ck(L.dh_event_synchronize(self._read_events[k % E]))
            return int(self._pinned_tokens[k % R])

        self.set_token(token)
        self.enqueue_step(pos, out_index=0)
        enqueue_read(0)
        out = []
        for k in range(1, n):
            self.enqueue_step(pos + k, from_device_token=True, in_index=(k - 1) % R, out_index=k % R)
            enqueue_read(k)
            out.append(wait_read(k - 1))
        out.append(wait_read(n - 1))
        return out

    def release_readback(self):
        """Frees the pinned staging memory and the events decode_greedy() made."""
        if getattr(self, "_pinned", None) is not None:
            for e in self._read_events:
                capi.check(self.L.dh_event_destroy(e))
            self._pinned_tokens = None
            capi.check(self.L.dh_host_free(self._pinned))
            self._pinned = None

    def capture_step(self, pos, want_logits=False, device_kv_len=True):
        """Captures one decode step (enqueued for position `pos`) into a HIP graph, the
        counterpart of the reference's one-submit-per-step recorder
        (src/inference/pipelines/text/generator-steps.js:605,814).  The step is run once
        normally first so that every kernel's one-time set-up is done outside the capture.
        device_kv_len: the captured attention launches read the key count from the word beside the
        token id (the reference's kvLenBuffer), so a replay patches nothing; False keeps the
        position in the launch arguments, which the library then moves before every replay."""
        if not self.fuse_qkv_attention:
            raise ValueError("capture_step serves the step with the fused attention kernel")
        # with the guard on the captured step also clears the status words and leaves its token next
        # to them (the library moves the checks' step number with the position at every replay)
        out_index = self.TOKEN_RING - 1 if self.finiteness_guard else 0
        self.enqueue_step(pos, want_logits, out_index=out_index)
        capi.check(self.L.dh_sync())
        self._graph_device_kv_len = bool(device_kv_len)
        capi.check(self.L.dh_graph_begin())
        g = ctypes.c_void_p()
        self._capturing = True
        try:
            if self.finiteness_guard:
                self._reset_finiteness()
            self.enqueue_step(pos, want_logits, out_index=out_index, device_kv_len=device_kv_len)
        except BaseException:
            # the capture must be closed either way; a graph that came out of it is not kept
            if self.L.dh_graph_end(pos, ctypes.byref(g)) == 0 and g.value:
                self.L.dh_graph_destroy(g)
            raise
        finally:
            self._capturing = False
        capi.check(self.L.dh_graph_end(pos, ctypes.byref(g)))
        capi.check(self.L.dh_graph_set_max_position(g, self.max_seq - 1))
        self._graph = g
        return g

    def step_graph(self, token, pos):
        """One decode step by replaying the captured graph at position `pos`: one graph launch
        and the 4-byte token readback (20 bytes with the finiteness guard on)."""
        if not 0 <= pos < self.max_seq:
            raise ValueError("decode position %d is outside the KV cache (max_seq=%d)" % (pos, self.max_seq))
        if getattr(self, "_graph", None) is None:
            self.capture_step(pos)
        self.set_token(token, pos + 1)
        capi.check(self.L.dh_graph_launch(self._graph, pos))
        if pos + 1 < self.max_seq and not self._graph_device_kv_len:
            # the next position's node parameters are set while the GPU runs this one
            capi.check(self.L.dh_graph_prepare(self._graph, pos + 1))
        if not self.finiteness_guard:
            return self.read_token()
        words = np.empty(5, np.uint32)
        capi.check(self.L.dh_download(words.ctypes.data, self.token.data_ptr(), 4 * (self.TOKEN_RING - 1), 20))
        self._raise_if_triggered(words, 1, "generation")
        return int(words[0])

    def release_graph(self):
        if getattr(self, "_graph", None) is not None:
            capi.check(self.L.dh_graph_destroy(self._graph))
            self._graph = None

    def _enqueue_sample(self, sampling, out_index=0):
        from . import ops
        L, c = self.L, self.cfg
        k = int(sampling["topK"])
        if float(sampling["temperature"]) < sampling.get("greedyThreshold", 0.01) or k <= 1:
            return                                  # the fused argmax already left the greedy token
        r = sampling["randomValue"] if "randomValue" in sampling else ops.seededRandom(sampling["randomSeed"])
        need = int(L.dh_sample_topk_workspace_bytes(c["vocab"], k))
        if getattr(self, "_sample_ws", None) is None or self._sample_ws.numel() < need:
            self._sample_ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
        capi.check(L.dh_sample_topk(self.logits.data_ptr(), c["vocab"], float(sampling["temperature"]), k, float(r), -1, 0.0,
                                    self._sample_ws.data_ptr(), self.token.data_ptr(), out_index))

    def generate(self, prompt, max_tokens, sampling=None, chunk=2048):
        """prefill + decode loop; sampling = dict(temperature, topK, seed) draws token i with
        randomSeed seed + i (greedy when None)."""
        draw = (lambda i: dict(temperature=sampling["temperature"], topK=sampling["topK"], randomSeed=sampling["seed"] + i)) \
            if sampling else (lambda i: None)
        if len(prompt) + max_tokens - 1 > self.max_seq:
            raise ValueError("prompt of %d tokens plus %d generated does not fit max_seq=%d" %
                             (len(prompt), max_tokens, self.max_seq))
        tok = self.prefill(prompt, chunk=chunk, sampling=draw(0))
        out = [tok]
        for i in range(1, max_tokens):
            tok = self.step(tok, len(prompt) + i - 1, sampling=draw(i))
            out.append(tok)
        return out

    def prefill(self, tokens, start_pos=0, chunk=2048, want_logits=False, sampling=None):
        """Pushes a prompt through the batched path, `chunk` tokens at a time: Q4_K prefill GEMMs,
        the T-token fused QKV-norm-RoPE-KV-write, matrix-core prefill attention.  KV rows
        start_pos .. start_pos + len(tokens) - 1 are written; returns the greedy token after the
        last prompt token (the reference's prefill, src/inference/pipelines/text/generator.js)."""
        L, c, ck = self.L, self.cfg, capi.check
        H, Hkv, D, Hd, I = c["heads"], c["kv_heads"], c["head_dim"], c["hidden"], c["inter"]
        tokens = np.asarray(tokens, np.uint32).reshape(-1)
        if tokens.size == 0 or start_pos + tokens.size > self.max_seq:
            raise ValueError("prefill of %d tokens at %d does not fit max_seq=%d" % (tokens.size, start_pos, self.max_seq))
        chunk = max(1, min(chunk, tokens.size))
        if getattr(self, "_pf_rows", 0) < chunk:
            f32 = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")
            self._pf = dict(x=f32(chunk * Hd), x2=f32(chunk * Hd), normed=f32(chunk * Hd),
                            qkv=f32(chunk * (self.qs + 2 * self.ks)), q=f32(chunk * self.qs), attn=f32(chunk * self.qs),
                            act=f32(chunk * I), ids=torch.zeros(chunk, dtype=torch.int32, device="cuda"))
            self._pf_rows = chunk
        b = self._pf
        qkv_n = self.qs + 2 * self.ks
        for c0 in range(0, tokens.size, chunk):
            ids = np.ascontiguousarray(tokens[c0:c0 + chunk])
            T, pos = ids.size, start_pos + c0
            ck(L.dh_upload(b["ids"].data_ptr(), 0, ids.ctypes.data, 4 * T))
            ck(L.dh_gather_f16(b["ids"].data_ptr(), self.embed.data_ptr(), b["x"].data_ptr(), T, Hd, c["vocab"], 0))
            x, x2 = b["x"], b["x2"]
            for d in self.layers:
                # the input RMSNorm runs inside the product (GEMV prologue below 16 tokens, the GEMM's
                # activation packing from 16 on)
                fused_norm = self.fuse_norm
                if fused_norm:
                    ck(L.dh_q4k_matmul_rmsnorm(x.data_ptr(), d["input_norm"].data_ptr(), c["eps"], 0,
                                               d["wqkv"].data_ptr(), b["qkv"].data_ptr(), capi.F32, T, qkv_n, Hd, 1.0,
                                               None))
                else:
                    ck(L.dh_rmsnorm(x.data_ptr(), d["input_norm"].data_ptr(), capi.F32, b["normed"].data_ptr(), T, Hd,
                                    c["eps"], 0, None, None, None, 1.0))
                    ck(L.dh_q4k_matmul(b["normed"].data_ptr(), capi.F32, d["wqkv"].data_ptr(), b["qkv"].data_ptr(),
                                       capi.F32, T, qkv_n, Hd, 1.0, None))
                ck(L.dh_qkv_norm_rope_kvwrite(b["qkv"].data_ptr(), d["q_norm"].data_ptr(), d["k_norm"].data_ptr(),
                                              self.cos.data_ptr(), self.sin.data_ptr(), b["q"].data_ptr(),
                                              d["cache_k"].data_ptr(), d["cache_v"].data_ptr(), T, H, Hkv, D, pos, D, 0,
                                              c["eps"], 0, pos * self.ks, int(c.get("qk_norm", 1))))
                if T == 1:
                    ck(L.dh_attn_decode(b["q"].data_ptr(), d["cache_k"].data_ptr(), d["cache_v"].data_ptr(),
                                        b["attn"].data_ptr(), H, Hkv, D, pos + 1, self.scale, 1, pos, 0.0, 0, 0,
                                        capi.KV_CONTIGUOUS, self.attn_ws.data_ptr()))
                else:
                    ck(L.dh_attn_prefill(b["q"].data_ptr(), d["cache_k"].data_ptr(), d["cache_v"].data_ptr(),
                                         b["attn"].data_ptr(), T, H, Hkv, D, pos + T, self.scale, 1, pos, 0.0, 0))
                ck(L.dh_q4k_matmul(b["attn"].data_ptr(), capi.F32, d["wo"].data_ptr(), x2.data_ptr(), capi.F32, T, Hd,
                                   self.qs, 1.0, x.data_ptr()))
                if fused_norm:
                    ck(L.dh_q4k_ffn_gate_up_rmsnorm(x2.data_ptr(), d["post_attn_norm"].data_ptr(), c["eps"], 0,
                                                    d["wgate"].data_ptr(), d["wup"].data_ptr(), b["act"].data_ptr(), T,
                                                    Hd, I, capi.ACT_SILU, 1.0, 0.0))
                else:
                    ck(L.dh_rmsnorm(x2.data_ptr(), d["post_attn_norm"].data_ptr(), capi.F32, b["normed"].data_ptr(), T,
                                    Hd, c["eps"], 0, None, None, None, 1.0))
                    ck(L.dh_q4k_ffn_gate_up(b["normed"].data_ptr(), d["wgate"].data_ptr(), d["wup"].data_ptr(),
                                            b["act"].data_ptr(), T, Hd, I, capi.ACT_SILU, 1.0, 0.0))
                ck(L.dh_q4k_matmul(b["act"].data_ptr(), capi.F32, d["wdown"].data_ptr(), x.data_ptr(), capi.F32, T, Hd, I,
                                   1.0, x2.data_ptr()))
        # logits of the last prompt token only
        last = b["x"].data_ptr() + (T - 1) * Hd * 4
        self._enqueue_head(last, 0, self.logits.data_ptr() if (want_logits or sampling is not None) else None)
        if sampling is not None:
            self._enqueue_sample(sampling)
        return self.read_token()

    def decode_batch(self, token, pos, n):
        """n greedy steps per submit, as the reference's batched decode does
        (src/inference/pipelines/text/generator-steps.js `shouldUseBatchDecode`, decode ring):
        step i reads its input token from the device buffer step i-1 wrote, nothing crosses to
        the host until all n steps are enqueued, then n token ids come back in one read."""
        if not 1 <= n <= self.TOKEN_RING:
            raise ValueError("decode_batch serves 1..%d tokens per submit, got %d" % (self.TOKEN_RING, n))
        self.set_token(token)
        if self.finiteness_guard:
            self._reset_finiteness()
        for i in range(n):
            self.enqueue_step(pos + i, from_device_token=i > 0, in_index=i - 1, out_index=i)
        if self.finiteness_guard:
            # ring and status in one read (src/inference/pipelines/text/generator-steps.js:1734-1740)
            words = np.empty(self.TOKEN_RING + 4, np.uint32)
            capi.check(self.L.dh_download(words.ctypes.data, self.token.data_ptr(), 0, words.nbytes))
            self._raise_if_triggered(words, self.TOKEN_RING, "batch generation")
            return [int(t) for t in words[:n]]
        out = np.empty(n, np.uint32)
        capi.check(self.L.dh_download(out.ctypes.data, self.token.data_ptr(), 0, 4 * n))
        return [int(t) for t in out]

    def read_logits(self):
        out = np.empty(self.cfg["vocab"], np.float32)
        capi.check(self.L.dh_download(out.ctypes.data, self.logits.data_ptr(), 0, out.nbytes))
        return out

    def read_kv(self, layer, rows):
        n = rows * self.ks
        k = np.empty(n, np.uint16)
        v = np.empty(n, np.uint16)
        d = self.layers[layer]
        capi.check(self.L.dh_download(k.ctypes.data, d["cache_k"].data_ptr(), 0, n * 2))
        capi.check(self.L.dh_download(v.ctypes.data, d["cache_v"].data_ptr(), 0, n * 2))
        return k, v


def random_model(cfg, seed=0, max_seq=None):
    """Random-init weights of a Q4_K decoder (config-4 recipe): Q4_K linears with the synthetic
    block distribution, norm weights N(1, 0.02), tied f16 embedding N(0, 0.02)."""
    H, Hkv, D, Hd, I = cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["hidden"], cfg["inter"]
    qs, ks = H * D, Hkv * D
    layers = []
    for i in range(cfg["layers"]):
        s = seed + 100 * (i + 1)
        layers.append(dict(
            wq=synth.q4k_tensor(qs, Hd, s + 1), wk=synth.q4k_tensor(ks, Hd, s + 2), wv=synth.q4k_tensor(ks, Hd, s + 3),
            wo=synth.q4k_tensor(Hd, qs, s + 4), wgate=synth.q4k_tensor(I, Hd, s + 5),
            wup=synth.q4k_tensor(I, Hd, s + 6), wdown=synth.q4k_tensor(Hd, I, s + 7),
            input_norm=1 + synth.normal_f32(Hd, s + 8, 0.02), post_attn_norm=1 + synth.normal_f32(Hd, s + 9, 0.02),
            q_norm=1 + synth.normal_f32(D, s + 10, 0.02), k_norm=1 + synth.normal_f32(D, s + 11, 0.02)))
    big = cfg["vocab"] * Hd >= 50_000_000
    embed = (synth.normal_f16_bits_large if big else synth.normal_f16_bits)((cfg["vocab"], Hd), seed + 7, 0.02)
    final_norm = 1 + synth.normal_f32(Hd, seed + 8, 0.02)
    cos, sin = synth.rope_tables(D, max_seq or cfg.get("max_seq", 4096), cfg.get("theta", 1e6))
    return layers, embed, final_norm, cos, sin
