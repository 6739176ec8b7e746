"""Builds tests/golden/qwen35_9b_gate_proj_receipt.npz from DATA files of the reference.

The reference keeps a receipt of one real Qwen3.5-9B Q4_K tensor (gate_proj of layer 0,
[12288, 4096], 196,608 super-blocks) under
reports/qwen-3-5-9b-metal/2026-07-12/layer0-ffn-gate-oracle/ with the per-block d/dmin,
the 6-bit scale/min values of every sub-block, and sha256 digests of the decoded scale and
minimum arrays (layer0-ffn-gate-oracle.json: artifactFiles).  The packed tensor itself is
not in the checkout.  This script copies those data files (no reference code is imported
or run) into one compressed archive:

  d_bits, dmin_bits  uint16[196608]   f16 bit patterns (the f32 files are exact widenings)
  scale_bits, min_bits uint8[1572864] index block*8 + sub
  sha256             JSON string: the digests recorded in the receipt

Run from the repo root in the build container: python tests/golden/make_receipt_fixture.py
"""
import hashlib
import json
import os

import numpy as np

REF = "/root/reference/reports/qwen-3-5-9b-metal/2026-07-12"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "qwen35_9b_gate_proj_receipt.npz")


def main():
    receipt = json.load(open(os.path.join(REF, "layer0-ffn-gate-oracle.json")))
    files = receipt["artifactFiles"]
    d = np.fromfile(os.path.join(REF, "layer0-ffn-gate-oracle/block-d.f32"), np.float32)
    dmin = np.fromfile(os.path.join(REF, "layer0-ffn-gate-oracle/block-dmin.f32"), np.float32)
    sc = np.fromfile(os.path.join(REF, "layer0-ffn-gate-oracle/packed-scale-bits.u8"), np.uint8)
    mn = np.fromfile(os.path.join(REF, "layer0-ffn-gate-oracle/packed-min-bits.u8"), np.uint8)
    for arr, key in ((d, "blockD"), (dmin, "blockDmin"), (sc, "packedScaleBits"), (mn, "packedMinBits")):
        assert hashlib.sha256(arr.tobytes()).hexdigest() == files[key]["sha256"], key
    d16 = d.astype(np.float16)
    dmin16 = dmin.astype(np.float16)
    assert np.array_equal(d16.astype(np.float32), d) and np.array_equal(dmin16.astype(np.float32), dmin)
    digests = {k: files[k]["sha256"] for k in ("decodedScales", "decodedMinima", "packedScaleBits",
                                                "packedMinBits", "blockD", "blockDmin")}
    digests["shape"] = receipt["projection"]["shape"]
    digests["blockCount"] = receipt["decodedQ4"]["blockCount"]
    np.savez_compressed(OUT, d_bits=d16.view(np.uint16), dmin_bits=dmin16.view(np.uint16),
                        scale_bits=sc, min_bits=mn, sha256=np.array(json.dumps(digests)))
    print(OUT, os.path.getsize(OUT))


if __name__ == "__main__":
    main()
