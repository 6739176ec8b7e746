"""RDRR artifacts (manifest.json + shard_NNNNN.bin) -> device buffers of the HIP decode path.

Mirrors what the reference's loader does for the tensors this path consumes:
  * manifest normalisation and checks   src/formats/rdrr/parsing.js:28-76 (shards: filename |
    fileName, running offset when absent), :78-160 (tensor locations: shard | shardIndex,
    offset, size, shape, optional spans across shards; the same error texts)
  * shard file names                    src/formats/rdrr/manifest.js:5-7
  * Q4_K_M tensors go to the device verbatim, layout 'row'
                                        src/loader/tensors/tensor-loader.js:540-555
  * F16 norm weights are widened to f32 on the host (tensor-loader.js:520-533)

Q4_K bytes are never repacked: a tensor's bytes in the shard are exactly what the GEMV kernels
read.  Anything this path cannot run (MoE, non-row Q4_K layout, other weight dtypes, sliding
windows, soft caps, per-layer patterns) fails closed with an error that names the field.
A shard that carries a sha256 hash is checked against it when first opened; a mismatch is an error.

write_artifact() produces the same on-disk format from arrays; tests and examples use it to make
synthetic artifacts (the reference ships manifests, not shards).
"""
import hashlib
import json
import mmap
import os

import numpy as np

from . import synth

RDRR_VERSION = 1
DTYPE_BYTES = {"F32": 4, "F16": 2, "BF16": 2}


class RdrrError(ValueError):
    pass


def shard_filename(index):
    return "shard_%05d.bin" % index


def expected_tensor_bytes(name, loc):
    """Byte size a tensor's shape and dtype imply (None when the dtype is not one this path reads)."""
    shape, dtype = loc["shape"], loc.get("dtype")
    if dtype == "Q4_K_M":
        if len(shape) != 2:
            raise RdrrError("Tensor '%s' is Q4_K_M but not 2-D (shape %r)" % (name, shape))
        return synth.q4k_nbytes(int(shape[0]), int(shape[1]))
    if dtype in DTYPE_BYTES:
        return int(np.prod(shape, dtype=np.int64)) * DTYPE_BYTES[dtype]
    return None


def normalize_manifest(manifest):
    """Checks and normalises a parsed manifest in place; returns it."""
    if not isinstance(manifest, dict):
        raise RdrrError("Invalid manifest: not a JSON object")
    errors = []
    shards = manifest.get("shards")
    if not isinstance(shards, list) or not shards:
        errors.append("Missing or empty shards array")
        shards = []
    offset, norm = 0, []
    for i, s in enumerate(shards):
        if not isinstance(s, dict) or not isinstance(s.get("size"), int) or s["size"] <= 0:
            errors.append("Shard %d has invalid size" % i)
            continue
        fn = s.get("filename") or s.get("fileName") or ""
        if os.path.basename(fn) != fn or fn in (".", ".."):
            errors.append("Shard %d filename %r must be a plain file name inside the artifact directory" % (i, fn))
        if not fn:
            errors.append("Shard %d missing filename" % i)
        norm.append({"index": s.get("index", i), "filename": fn, "size": s["size"],
                     "hash": s.get("hash") or s.get("blake3") or "",
                     "offset": s.get("offset", offset)})
        offset += s["size"]
    manifest["shards"] = norm
    tensors = manifest.get("tensors")
    if not isinstance(tensors, dict) and not isinstance(manifest.get("tensorsFile"), str):
        errors.append("Missing tensorsFile and tensors - one is required")
    if errors:
        raise RdrrError("Invalid manifest:\n  - " + "\n  - ".join(errors))
    if isinstance(tensors, dict):
        manifest["tensors"] = normalize_tensor_map(tensors, norm)
    return manifest


def normalize_tensor_map(tensors, shards):
    out = {}
    for name, loc in tensors.items():
        if not isinstance(loc, dict):
            raise RdrrError("Tensor '%s' has an invalid location" % name)
        if not isinstance(loc.get("shape"), list):
            raise RdrrError("Tensor '%s' missing shape" % name)
        spans = loc.get("spans")
        if spans is not None:
            if not isinstance(spans, list):
                raise RdrrError("Tensor '%s' has invalid spans array" % name)
            ns = []
            for j, sp in enumerate(spans):
                sp = sp if isinstance(sp, dict) else {}
                idx = sp.get("shardIndex", sp.get("shard"))
                if not isinstance(idx, int):
                    raise RdrrError("Tensor '%s' span[%d] missing shard index" % (name, j))
                if not isinstance(sp.get("offset"), int):
                    raise RdrrError("Tensor '%s' span[%d] missing offset" % (name, j))
                if not isinstance(sp.get("size"), int):
                    raise RdrrError("Tensor '%s' span[%d] missing size" % (name, j))
                ns.append({"shardIndex": idx, "offset": sp["offset"], "size": sp["size"]})
            spans = ns
        else:
            idx = loc.get("shardIndex", loc.get("shard"))
            if not isinstance(idx, int):
                raise RdrrError("Tensor '%s' missing shard index" % name)
            if not isinstance(loc.get("offset"), int):
                raise RdrrError("Tensor '%s' missing offset" % name)
            if not isinstance(loc.get("size"), int):
                raise RdrrError("Tensor '%s' missing size" % name)
            spans = [{"shardIndex": idx, "offset": loc["offset"], "size": loc["size"]}]
        size = loc.get("size", sum(s["size"] for s in spans))
        if sum(s["size"] for s in spans) != size:
            raise RdrrError("Tensor '%s' spans cover %d bytes, size says %d" % (name, sum(s["size"] for s in spans), size))
        for sp in spans:
            if not 0 <= sp["shardIndex"] < len(shards):
                raise RdrrError("Tensor '%s' names shard %d of %d" % (name, sp["shardIndex"], len(shards)))
            if sp["offset"] < 0 or sp["offset"] + sp["size"] > shards[sp["shardIndex"]]["size"]:
                raise RdrrError("Tensor '%s' reaches past the end of shard %d" % (name, sp["shardIndex"]))
        n = dict(loc, size=size, spans=spans)
        want = expected_tensor_bytes(name, n)
        if want is not None and want != size:
            raise RdrrError("Tensor '%s' (%s %r) should hold %d bytes, manifest says %d" %
                            (name, loc.get("dtype"), loc["shape"], want, size))
        out[name] = n
    return out


def parse_manifest(text):
    try:
        manifest = json.loads(text)
    except ValueError as e:
        raise RdrrError("Failed to parse manifest JSON: %s" % e)
    return normalize_manifest(manifest)


class Artifact:
    """A directory with manifest.json (+ optional tensors file) and its shards, memory-mapped."""

    def __init__(self, directory, verify_hashes=True):
        """`verify_hashes`: check each shard that carries a hash against it when the shard is first
        opened (sha256 only; a hashed shard under another algorithm is refused unless this is off)."""
        self.dir = directory
        self.verify_hashes = verify_hashes
        with open(os.path.join(directory, "manifest.json"), "r") as f:
            self.manifest = parse_manifest(f.read())
        if "tensors" not in self.manifest or not isinstance(self.manifest["tensors"], dict):
            with open(os.path.join(directory, self.manifest["tensorsFile"]), "r") as f:
                try:
                    raw = json.loads(f.read())
                except ValueError as e:
                    raise RdrrError("Failed to parse tensors.json: %s" % e)
            self.manifest["tensors"] = normalize_tensor_map(raw, self.manifest["shards"])
        self.tensors = self.manifest["tensors"]
        self._maps = {}

    def _shard(self, index):
        m = self._maps.get(index)
        if m is None:
            info = self.manifest["shards"][index]
            path = os.path.join(self.dir, info["filename"] or shard_filename(index))
            if not os.path.exists(path):
                raise RdrrError("Shard file %s is missing" % path)
            if os.path.getsize(path) != info["size"]:
                raise RdrrError("Shard %d is %d bytes on disk, manifest says %d" %
                                (index, os.path.getsize(path), info["size"]))
            f = open(path, "rb")
            m = (f, mmap.mmap(f.fileno(), 0, access=mmap.ACCESS_READ))
            try:
                if self.verify_hashes and info["hash"]:
                    algorithm = self.manifest.get("hashAlgorithm")
                    if algorithm != "sha256":
                        raise RdrrError("Shard %d carries a %r hash, which this loader cannot check "
                                        "(pass verify_hashes=False to load it unchecked)" % (index, algorithm))
                    h = hashlib.sha256()
                    for at in range(0, info["size"], 64 << 20):
                        h.update(m[1][at:at + (64 << 20)])
                    if h.hexdigest() != info["hash"].lower():
                        raise RdrrError("Shard %d fails its sha256 check (manifest %s, file %s)" %
                                        (index, info["hash"], h.hexdigest()))
            except BaseException:
                # a shard that is refused is not kept open
                m[1].close()
                f.close()
                raise
            self._maps[index] = m
        return m[1]

    def tensor_bytes(self, name):
        """The tensor's bytes as a uint8 array (a copy when it spans shards, else a view)."""
        loc = self.tensors.get(name)
        if loc is None:
            raise RdrrError("Tensor '%s' is not in the manifest" % name)
        parts = [np.frombuffer(self._shard(s["shardIndex"]), np.uint8, s["size"], s["offset"]) for s in loc["spans"]]
        return parts[0] if len(parts) == 1 else np.concatenate(parts)

    def tensor_f32(self, name):
        loc = self.tensors[name] if name in self.tensors else None
        raw = self.tensor_bytes(name)
        if loc["dtype"] == "F32":
            return raw.view(np.float32).copy()
        if loc["dtype"] == "F16":
            return raw.view(np.float16).astype(np.float32)
        raise RdrrError("Tensor '%s' has dtype %s where f16/f32 is expected" % (name, loc["dtype"]))

    def close(self):
        for f, m in self._maps.values():
            try:
                m.close()
            except BufferError:      # arrays handed out still view the mapping; it goes with them
                pass
            f.close()
        self._maps = {}


def _require(cond, what):
    if not cond:
        raise RdrrError("[rdrr] unsupported by the HIP decode path: " + what)


def decoder_config(manifest):
    """cfg dict of doppler_amd.decoder.HipDecoder from a manifest; fails closed on features the
    path does not implement."""
    a = manifest.get("architecture") or {}
    inf = manifest.get("inference") or {}
    for k in ("numLayers", "hiddenSize", "intermediateSize", "numAttentionHeads", "numKeyValueHeads", "headDim",
              "vocabSize"):
        if not isinstance(a.get(k), int):
            raise RdrrError("Invalid manifest:\n  - architecture.%s is missing" % k)
    att, nrm, ffn, rope, outp = (inf.get(k) or {} for k in ("attention", "normalization", "ffn", "rope", "output"))
    _require(manifest.get("moeConfig") in (None, {}), "moeConfig (mixture of experts)")
    _require((manifest.get("quantizationInfo") or {}).get("layout", "row") == "row", "quantizationInfo.layout != 'row'")
    _require(not att.get("slidingWindow"), "inference.attention.slidingWindow")
    _require(not att.get("attnLogitSoftcapping"), "inference.attention.attnLogitSoftcapping")
    _require(not att.get("attentionBias") and not att.get("attentionOutputGate") and not att.get("valueNorm"),
             "attention bias / output gate / value norm")
    _require(not nrm.get("preFeedforwardNorm") and not nrm.get("postFeedforwardNorm"), "pre/post feed-forward norms")
    _require(ffn.get("gatedActivation", True) and ffn.get("branchMode", "dense") == "dense", "non-gated or non-dense FFN")
    _require(ffn.get("activation", "silu") in ("silu", "gelu"), "ffn.activation %r" % ffn.get("activation"))
    _require(not rope.get("partialRotaryFactor") and not rope.get("ropeScalingType") and not rope.get("mropeSection"),
             "partial / scaled / multi-axis RoPE")
    _require(outp.get("tieWordEmbeddings", True), "untied LM head")
    _require(not outp.get("finalLogitSoftcapping") and not outp.get("scaleEmbeddings"), "logit soft cap / embedding scale")
    _require((inf.get("layerPattern") or {}).get("type", "uniform") == "uniform", "non-uniform layer pattern")
    # scalars the decoder hard-wires: attention scale 1/sqrt(headDim), no logit or residual-branch scale
    qpas = att.get("queryPreAttnScalar")
    _require(qpas in (None, a["headDim"]), "inference.attention.queryPreAttnScalar %r != headDim %d" % (qpas, a["headDim"]))
    _require(outp.get("logitInputScale") in (None, 1, 1.0), "inference.output.logitInputScale %r" % outp.get("logitInputScale"))
    rbs = (inf.get("layerPattern") or {}).get("residualBranchScale")
    _require(rbs in (None, 1, 1.0), "inference.layerPattern.residualBranchScale %r" % rbs)
    return dict(layers=a["numLayers"], hidden=a["hiddenSize"], inter=a["intermediateSize"],
                heads=a["numAttentionHeads"], kv_heads=a["numKeyValueHeads"], head_dim=a["headDim"],
                vocab=a["vocabSize"], eps=float(nrm.get("rmsNormEps", 1e-6)),
                qk_norm=1 if att.get("queryKeyNorm") else 0,
                theta=float(rope.get("ropeTheta") or a.get("ropeTheta") or 10000.0),
                norm_offset=bool(nrm.get("rmsNormWeightOffset")), activation=ffn.get("activation", "silu"),
                swiglu_limit=ffn.get("swigluLimit"))


LAYER_TENSORS = {
    "wq": "self_attn.q_proj.weight", "wk": "self_attn.k_proj.weight", "wv": "self_attn.v_proj.weight",
    "wo": "self_attn.o_proj.weight", "wgate": "mlp.gate_proj.weight", "wup": "mlp.up_proj.weight",
    "wdown": "mlp.down_proj.weight",
}
LAYER_NORMS = {"input_norm": "input_layernorm.weight", "post_attn_norm": "post_attention_layernorm.weight",
               "q_norm": "self_attn.q_norm.weight", "k_norm": "self_attn.k_norm.weight"}


def _find(art, *candidates):
    for c in candidates:
        for prefix in ("", "model."):
            if prefix + c in art.tensors:
                return prefix + c
    raise RdrrError("Tensor '%s' is not in the manifest" % candidates[0])


def load_model_arrays(art):
    """(cfg, layers, embed_bits, final_norm) in the form HipDecoder and the CPU checker take.
    Every linear weight must be Q4_K_M in row layout with the shape the architecture implies."""
    cfg = decoder_config(art.manifest)
    _require(not cfg["norm_offset"] and cfg["activation"] == "silu" and not cfg["swiglu_limit"],
             "the decoder host wires SiLU, plain RMSNorm weights and no clamp (the ops themselves take the options)")
    H, Hkv, D, Hd, I = cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["hidden"], cfg["inter"]
    shapes = {"wq": [H * D, Hd], "wk": [Hkv * D, Hd], "wv": [Hkv * D, Hd], "wo": [Hd, H * D],
              "wgate": [I, Hd], "wup": [I, Hd], "wdown": [Hd, I]}
    layers = []
    for i in range(cfg["layers"]):
        d = {}
        for key, suffix in LAYER_TENSORS.items():
            name = _find(art, "layers.%d.%s" % (i, suffix))
            loc = art.tensors[name]
            if loc.get("dtype") != "Q4_K_M" or loc.get("layout", "row") != "row":
                raise RdrrError("Tensor '%s' must be Q4_K_M in row layout (dtype %s, layout %s)" %
                                (name, loc.get("dtype"), loc.get("layout")))
            if list(loc["shape"]) != shapes[key]:
                raise RdrrError("Tensor '%s' has shape %r, architecture implies %r" % (name, loc["shape"], shapes[key]))
            d[key] = art.tensor_bytes(name)
        for key, suffix in LAYER_NORMS.items():
            if key in ("q_norm", "k_norm") and not cfg["qk_norm"]:
                d[key] = np.ones(D, np.float32)
                continue
            d[key] = art.tensor_f32(_find(art, "layers.%d.%s" % (i, suffix)))
        layers.append(d)
    ename = _find(art, "embed_tokens.weight")
    eloc = art.tensors[ename]
    if eloc.get("dtype") != "F16" or list(eloc["shape"]) != [cfg["vocab"], Hd]:
        raise RdrrError("Tensor '%s' must be F16 [%d, %d] (dtype %s, shape %r)" %
                        (ename, cfg["vocab"], Hd, eloc.get("dtype"), eloc["shape"]))
    embed = art.tensor_bytes(ename).view(np.uint16).reshape(cfg["vocab"], Hd)
    final_norm = art.tensor_f32(_find(art, "norm.weight"))
    return cfg, layers, embed, final_norm


def load_decoder(directory, max_seq, verify_hashes=True, **decoder_kwargs):
    """Open an RDRR directory and return a ready HipDecoder (weights resident in HBM).
    `verify_hashes` as in Artifact."""
    from . import decoder
    art = Artifact(directory, verify_hashes=verify_hashes)
    try:
        cfg, layers, embed, final_norm = load_model_arrays(art)
        cos, sin = synth.rope_tables(cfg["head_dim"], max_seq, cfg["theta"])
        return decoder.HipDecoder(dict(cfg, max_seq=max_seq), layers, embed, final_norm, cos, sin, max_seq,
                                  **decoder_kwargs)
    finally:
        art.close()


def write_artifact(directory, cfg, layers, embed_bits, final_norm, shard_bytes=64 << 20, model_id="synthetic-q4k",
                   layout=None, hash_shards=None):
    """Writes manifest.json and shards for a dense Q4_K decoder.  Tensors are laid out in name
    order into shards of `shard_bytes`; a tensor that does not fit the rest of a shard is split
    into spans, as the reference's converter does for large embeddings.  `layout`, if given,
    maps tensor name -> spans to write at (used to reproduce an existing manifest's placement).
    `hash_shards`: record each shard's sha256 (default: only when the artifact is under 1 GiB)."""
    os.makedirs(directory, exist_ok=True)
    items = {"embed_tokens.weight": (np.ascontiguousarray(embed_bits).view(np.uint8).reshape(-1),
                                     [cfg["vocab"], cfg["hidden"]], "F16", "embedding", "embed"),
             "norm.weight": (final_norm.astype(np.float16).view(np.uint8).reshape(-1), [cfg["hidden"]], "F16", "norm", "head")}
    H, Hkv, D, Hd, I = cfg["heads"], cfg["kv_heads"], cfg["head_dim"], cfg["hidden"], cfg["inter"]
    shapes = {"wq": [H * D, Hd], "wk": [Hkv * D, Hd], "wv": [Hkv * D, Hd], "wo": [Hd, H * D],
              "wgate": [I, Hd], "wup": [I, Hd], "wdown": [Hd, I]}
    for i, l in enumerate(layers):
        for key, suffix in LAYER_TENSORS.items():
            items["layers.%d.%s" % (i, suffix)] = (np.ascontiguousarray(l[key]).reshape(-1), shapes[key], "Q4_K_M",
                                                   "matmul", "layer.%d" % i)
        for key, suffix in LAYER_NORMS.items():
            if key in ("q_norm", "k_norm") and not cfg.get("qk_norm"):
                continue
            w = l[key].astype(np.float16)
            items["layers.%d.%s" % (i, suffix)] = (w.view(np.uint8).reshape(-1), [int(w.size)], "F16", "norm", "layer.%d" % i)
    tensors, shard_sizes = {}, []
    files = {}

    def shard_file(idx):
        if idx not in files:
            files[idx] = open(os.path.join(directory, shard_filename(idx)), "wb+")
        return files[idx]

    cur, used = 0, 0
    for name in sorted(items):
        data, shape, dtype, role, group = items[name]
        spans = []
        if layout is not None:
            spans = [dict(s) for s in layout[name]]
        else:
            left, at = data.size, 0
            while left > 0:
                if used == shard_bytes:
                    cur, used = cur + 1, 0
                n = min(left, shard_bytes - used)
                spans.append({"shardIndex": cur, "offset": used, "size": int(n)})
                used += n
                left -= n
                at += n
        at = 0
        for sp in spans:
            f = shard_file(sp["shardIndex"])
            f.seek(sp["offset"])
            f.write(data[at:at + sp["size"]].tobytes())
            at += sp["size"]
            while len(shard_sizes) <= sp["shardIndex"]:
                shard_sizes.append(0)
            shard_sizes[sp["shardIndex"]] = max(shard_sizes[sp["shardIndex"]], sp["offset"] + sp["size"])
        loc = {"size": int(data.size), "shape": shape, "dtype": dtype, "role": role, "group": group}
        if dtype == "Q4_K_M":
            loc["layout"] = "row"
        if len(spans) == 1:
            loc.update(shard=spans[0]["shardIndex"], offset=spans[0]["offset"])
        else:
            loc["spans"] = spans
        tensors[name] = loc
    for f in files.values():
        f.close()
    offset, shards = 0, []
    if hash_shards is None:
        hash_shards = sum(shard_sizes) < (1 << 30)
    for i, size in enumerate(shard_sizes):
        digest = ""
        if hash_shards:
            h = hashlib.sha256()
            with open(os.path.join(directory, shard_filename(i)), "rb") as f:
                for chunk in iter(lambda: f.read(64 << 20), b""):
                    h.update(chunk)
            digest = h.hexdigest()
        shards.append({"index": i, "filename": shard_filename(i), "size": int(size), "hash": digest, "offset": offset})
        offset += size
    manifest = {
        "version": RDRR_VERSION, "modelId": model_id, "modelType": "transformer", "quantization": "Q4_K_M",
        "quantizationInfo": {"weights": "q4k", "embeddings": "f16", "compute": "f32", "layout": "row"},
        "architecture": {"numLayers": cfg["layers"], "hiddenSize": Hd, "intermediateSize": I, "numAttentionHeads": H,
                         "numKeyValueHeads": Hkv, "headDim": D, "vocabSize": cfg["vocab"],
                         "maxSeqLen": cfg.get("max_seq", 4096), "ropeTheta": cfg.get("theta", 1e6)},
        "moeConfig": None,
        "inference": {"attention": {"queryKeyNorm": bool(cfg.get("qk_norm")), "causal": True, "slidingWindow": None,
                                    "attnLogitSoftcapping": None},
                      "normalization": {"rmsNormEps": cfg.get("eps", 1e-6), "rmsNormWeightOffset": False},
                      "ffn": {"activation": "silu", "gatedActivation": True, "branchMode": "dense", "swigluLimit": None},
                      "rope": {"ropeTheta": cfg.get("theta", 1e6)},
                      "output": {"tieWordEmbeddings": True, "finalLogitSoftcapping": None},
                      "layerPattern": {"type": "uniform"}},
        "shards": shards, "tensors": tensors, "totalSize": int(offset), "hashAlgorithm": "sha256",
    }
    with open(os.path.join(directory, "manifest.json"), "w") as f:
        json.dump(manifest, f)
    return manifest
