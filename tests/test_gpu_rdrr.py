"""RDRR artifact -> HBM -> greedy decode.  The artifact has the exact tensor placement (shards,
offsets, a five-span embedding) of a manifest the reference ships for Qwen3-0.6B-shaped weights
(tests/golden/qwen3_0_6b_q4k_rdrr_manifest.json); the reference ships no shards, so their bytes
are seeded random weights written at those offsets.  The decoder built by rdrr.load_decoder must
produce the CPU oracle's greedy tokens and logits (relative L2 <= 1e-3) from the same bytes."""
import json
import os

import numpy as np
import pytest

import oracle
from doppler_amd import decoder, rdrr, synth

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
REAL = os.path.join(HERE, "golden", "qwen3_0_6b_q4k_rdrr_manifest.json")


def rel_l2(a, b):
    a, b = np.asarray(a, np.float64), np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


@pytest.mark.timeout(900)
def test_real_manifest_placement_loads_and_decodes(tmp_path):
    real = rdrr.parse_manifest(open(REAL).read())
    cfg = dict(rdrr.decoder_config(real), max_seq=48)
    layers, embed, final_norm, _, _ = decoder.random_model(cfg, seed=21, max_seq=48)
    layout = {n: v["spans"] for n, v in real["tensors"].items()}
    written = rdrr.write_artifact(str(tmp_path), cfg, layers, embed, final_norm, layout=layout)
    assert [s["size"] for s in written["shards"]] == [s["size"] for s in real["shards"]]
    # keep the reference manifest itself (its inference block and all) as the one that is loaded
    m = json.load(open(REAL))
    with open(os.path.join(str(tmp_path), "manifest.json"), "w") as f:
        json.dump(m, f)

    max_seq = 48
    # the manifest's blake3 hashes belong to the real model's shards; these shards hold random weights
    # at the same placement, so the loader must refuse them checked and load them unchecked
    with pytest.raises(rdrr.RdrrError, match="blake3"):
        rdrr.load_decoder(str(tmp_path), max_seq)
    gpu = rdrr.load_decoder(str(tmp_path), max_seq, verify_hashes=False)
    art = rdrr.Artifact(str(tmp_path), verify_hashes=False)
    c2, l2, e2, fn2 = rdrr.load_model_arrays(art)
    for a, b in zip(layers, l2):
        for k in rdrr.LAYER_TENSORS:
            assert np.array_equal(a[k], b[k])
    cos, sin = synth.rope_tables(c2["head_dim"], max_seq, c2["theta"])
    ol = []
    for l in l2:
        d = dict(l)
        d["cache_k"] = np.zeros((max_seq, c2["kv_heads"], c2["head_dim"]), np.uint16)
        d["cache_v"] = np.zeros_like(d["cache_k"])
        ol.append(d)
    cpu = oracle.DecoderOracle(dict(c2, max_seq=max_seq), ol, e2, fn2, cos, sin)
    prompt = synth.rng(3).integers(0, c2["vocab"], 6)
    tok = None
    for pos in range(14):
        inp = int(prompt[pos]) if pos < len(prompt) else tok
        want_logits = pos in (0, 13)
        g = gpu.step(inp, pos, want_logits=want_logits)
        if want_logits:
            c, want = cpu.step(inp, pos, want_logits=True)
            assert rel_l2(gpu.read_logits(), want) <= 1e-3, pos
        else:
            c = cpu.step(inp, pos)
        assert g == c, (pos, g, c)
        tok = g
    art.close()
