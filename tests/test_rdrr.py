"""RDRR artifact reader (doppler_amd.rdrr): manifest checks against a manifest the reference
ships, write -> read round trip, fail-closed errors.  CPU only.

tests/golden/qwen3_0_6b_q4k_rdrr_manifest.json is the reference's
models/local/qwen-3-embedding-0-6b-q4k-ehf16-af32/manifest.json, a data file (the reference
ships manifests without shards): 310 tensors of a 28-layer hidden-1024 Qwen3 block stack, the
shapes of benchmark config 1.
"""
import json
import os

import numpy as np
import pytest

from doppler_amd import rdrr, synth

HERE = os.path.dirname(os.path.abspath(__file__))
REAL = os.path.join(HERE, "golden", "qwen3_0_6b_q4k_rdrr_manifest.json")

TINY = dict(layers=2, hidden=256, inter=512, heads=4, kv_heads=2, head_dim=64, vocab=300, eps=1e-6, qk_norm=1,
            theta=1e6, max_seq=64)


def tiny_model(seed=5):
    from doppler_amd import decoder
    layers, embed, final_norm, _, _ = decoder.random_model(TINY, seed=seed, max_seq=64)
    return layers, embed, final_norm


def test_real_manifest_sizes_follow_the_q4k_row_layout_rule():
    m = rdrr.parse_manifest(open(REAL).read())
    t = m["tensors"]
    assert len(t) == 310 and len(m["shards"]) == 9
    q4 = [(n, v) for n, v in t.items() if v["dtype"] == "Q4_K_M"]
    assert len(q4) == 28 * 7
    for n, v in q4:
        N, K = v["shape"]
        assert v["size"] == N * ((K + 255) // 256) * 144, n      # rows of ceil(K/256) super-blocks of 144 bytes
        assert v["layout"] == "row"
    # block total of one layer = the figure the GEMV benchmark uses for this block
    layer0 = sum(v["size"] for n, v in q4 if n.startswith("layers.0."))
    assert layer0 == 8847360
    emb = t["embed_tokens.weight"]
    assert len(emb["spans"]) == 5 and sum(s["size"] for s in emb["spans"]) == emb["size"] == 151669 * 1024 * 2
    # tensors tile the shards without overlap
    cover = {}
    for v in t.values():
        for s in v["spans"]:
            cover.setdefault(s["shardIndex"], []).append((s["offset"], s["offset"] + s["size"]))
    for idx, spans in cover.items():
        spans.sort()
        assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
        assert spans[-1][1] <= m["shards"][idx]["size"]
    assert sum(s["size"] for s in m["shards"]) == m["totalSize"]


def test_real_manifest_maps_to_the_decoder_config():
    m = rdrr.parse_manifest(open(REAL).read())
    cfg = rdrr.decoder_config(m)
    assert cfg == dict(layers=28, hidden=1024, inter=3072, heads=16, kv_heads=8, head_dim=128, vocab=151669, eps=1e-6,
                       qk_norm=1, theta=1e6, norm_offset=False, activation="silu", swiglu_limit=None)
    shapes = {(tuple(v["shape"])) for n, v in m["tensors"].items() if v["dtype"] == "Q4_K_M"}
    assert shapes == {(N, K) for (N, K) in synth.CFG1_SHAPES.values()}


def test_write_then_read_round_trip_with_spans(tmp_path):
    layers, embed, final_norm = tiny_model()
    man = rdrr.write_artifact(str(tmp_path), TINY, layers, embed, final_norm, shard_bytes=100_000)
    assert len(man["shards"]) > 3
    assert any("spans" in v for v in man["tensors"].values())
    art = rdrr.Artifact(str(tmp_path))
    cfg, l2, e2, fn2 = rdrr.load_model_arrays(art)
    assert cfg["layers"] == 2 and cfg["qk_norm"] == 1
    for a, b in zip(layers, l2):
        for k in rdrr.LAYER_TENSORS:
            assert np.array_equal(a[k], b[k]), k
        for k in rdrr.LAYER_NORMS:
            assert np.array_equal(a[k].astype(np.float16).astype(np.float32), b[k]), k
    assert np.array_equal(embed, e2)
    assert np.array_equal(final_norm.astype(np.float16).astype(np.float32), fn2)
    art.close()


def _manifest_with(tmp_path, mutate):
    layers, embed, final_norm = tiny_model()
    rdrr.write_artifact(str(tmp_path), TINY, layers, embed, final_norm, shard_bytes=1 << 20)
    p = os.path.join(str(tmp_path), "manifest.json")
    m = json.load(open(p))
    mutate(m)
    json.dump(m, open(p, "w"))


@pytest.mark.parametrize("mutate,match", [
    (lambda m: m["tensors"]["layers.0.mlp.up_proj.weight"].pop("shard"), "missing shard index"),
    (lambda m: m["tensors"]["layers.0.mlp.up_proj.weight"].pop("offset"), "missing offset"),
    (lambda m: m["tensors"]["layers.0.mlp.up_proj.weight"].pop("shape"), "missing shape"),
    (lambda m: m["tensors"]["layers.0.mlp.up_proj.weight"].update(size=1000), "should hold"),
    (lambda m: m["tensors"]["layers.0.mlp.up_proj.weight"].update(offset=10 ** 9), "past the end of shard"),
    (lambda m: m.pop("shards"), "Missing or empty shards"),
    (lambda m: m.pop("tensors"), "Missing tensorsFile and tensors"),
    (lambda m: m["shards"][0].update(filename="../shard_00000.bin"), "plain file name"),
    (lambda m: m["shards"][0].update(filename="/etc/passwd"), "plain file name"),
])
def test_manifest_errors_fail_closed(tmp_path, mutate, match):
    _manifest_with(tmp_path, mutate)
    with pytest.raises(rdrr.RdrrError, match=match):
        rdrr.Artifact(str(tmp_path))


@pytest.mark.parametrize("mutate,match", [
    (lambda m: m["inference"]["attention"].update(slidingWindow=512), "slidingWindow"),
    (lambda m: m.update(moeConfig={"numExperts": 8}), "moeConfig"),
    (lambda m: m["inference"]["output"].update(tieWordEmbeddings=False), "untied LM head"),
    (lambda m: m["tensors"]["layers.1.self_attn.q_proj.weight"].update(dtype="F16", shape=[18432]), "must be Q4_K_M"),
    (lambda m: m["tensors"]["layers.1.self_attn.q_proj.weight"].update(layout="column"), "row layout"),
    (lambda m: m["tensors"].pop("layers.1.mlp.down_proj.weight"), "is not in the manifest"),
    (lambda m: m["architecture"].pop("headDim"), "architecture.headDim"),
    (lambda m: m["inference"]["attention"].update(queryPreAttnScalar=256), "queryPreAttnScalar"),
    (lambda m: m["inference"]["output"].update(logitInputScale=0.5), "logitInputScale"),
    (lambda m: m["inference"].setdefault("layerPattern", {}).update(residualBranchScale=0.22), "residualBranchScale"),
])
def test_unsupported_models_fail_closed(tmp_path, mutate, match):
    _manifest_with(tmp_path, mutate)
    art = rdrr.Artifact(str(tmp_path))
    with pytest.raises(rdrr.RdrrError, match=match):
        rdrr.load_model_arrays(art)
    art.close()


def test_truncated_shard_is_detected(tmp_path):
    layers, embed, final_norm = tiny_model()
    rdrr.write_artifact(str(tmp_path), TINY, layers, embed, final_norm, shard_bytes=1 << 20)
    p = os.path.join(str(tmp_path), rdrr.shard_filename(0))
    with open(p, "r+b") as f:
        f.truncate(os.path.getsize(p) - 1)
    art = rdrr.Artifact(str(tmp_path))
    with pytest.raises(rdrr.RdrrError, match="bytes on disk"):
        rdrr.load_model_arrays(art)
    art.close()


def test_corrupted_shard_fails_its_hash_check(tmp_path):
    layers, embed, final_norm = tiny_model()
    man = rdrr.write_artifact(str(tmp_path), TINY, layers, embed, final_norm, shard_bytes=1 << 20)
    import hashlib
    for s in man["shards"]:
        with open(os.path.join(str(tmp_path), s["filename"]), "rb") as f:
            assert hashlib.sha256(f.read()).hexdigest() == s["hash"]
    p = os.path.join(str(tmp_path), rdrr.shard_filename(0))
    with open(p, "r+b") as f:
        f.seek(1000)
        b = f.read(1)
        f.seek(1000)
        f.write(bytes([b[0] ^ 0x10]))
    art = rdrr.Artifact(str(tmp_path))
    with pytest.raises(rdrr.RdrrError, match="fails its sha256 check"):
        rdrr.load_model_arrays(art)
    art.close()
    art = rdrr.Artifact(str(tmp_path), verify_hashes=False)
    rdrr.load_model_arrays(art)
    art.close()


def test_a_hash_this_loader_cannot_check_is_refused(tmp_path):
    _manifest_with(tmp_path, lambda m: m.update(hashAlgorithm="blake3"))
    art = rdrr.Artifact(str(tmp_path))
    with pytest.raises(rdrr.RdrrError, match="cannot check"):
        rdrr.load_model_arrays(art)
    art.close()


@pytest.mark.skipif(__import__("shutil").which("node") is None, reason="node is not installed")
def test_js_loader_checks_hashes_and_shard_names(tmp_path):
    import subprocess
    layers, embed, final_norm = tiny_model()
    rdrr.write_artifact(str(tmp_path), TINY, layers, embed, final_norm, shard_bytes=1 << 20)
    loader = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                          "doppler_amd", "js", "loader", "rdrr-loader.js")
    script = """
import fs from 'fs';
import { RdrrArtifact, parseManifest } from %r;
const dir = %r;
const name = Object.keys(new RdrrArtifact(dir).tensors)[0];
new RdrrArtifact(dir).tensorBytes(name);
const text = fs.readFileSync(dir + '/manifest.json', 'utf8');
const m = JSON.parse(text);
m.shards[0].filename = '../x.bin';
let caught = '';
try { parseManifest(JSON.stringify(m)); } catch (e) { caught = e.message; }
if (!/plain file name/.test(caught)) throw new Error('path component accepted: ' + caught);
const p = dir + '/shard_00000.bin';
const bytes = fs.readFileSync(p);
bytes[1000] ^= 0x10;
fs.writeFileSync(p, bytes);
caught = '';
try { const a = new RdrrArtifact(dir); for (const n of Object.keys(a.tensors)) a.tensorBytes(n); } catch (e) { caught = e.message; }
if (!/fails its sha256 check/.test(caught)) throw new Error('corruption accepted: ' + caught);
const a = new RdrrArtifact(dir, { verifyHashes: false });
for (const n of Object.keys(a.tensors)) a.tensorBytes(n);
console.log('ok');
""" % (loader, str(tmp_path))
    src = tmp_path / "check.mjs"
    src.write_text(script)
    out = subprocess.run(["node", str(src)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stderr
    assert out.stdout.strip() == "ok"
