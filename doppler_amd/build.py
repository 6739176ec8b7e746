"""Builds the in-tree native pieces: libdopplerhip.so (HIP kernels + C ABI, gfx950) and the
Node-API addon that binds it for the JavaScript host code.

    python -m doppler_amd.build            # everything
    python -m doppler_amd.build --hip-only

hipcc cross-compiles for gfx950 without a GPU present.  The flag pair
`-Xclang -target-feature -Xclang -packed-fp32-ops` keeps the compiler from forming packed
FP32 instructions (the host pass prints a harmless "not a recognized feature" note).
"""
import argparse
import glob
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIB_DIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIB_DIR, "libdopplerhip.so")
ADDON = os.path.join(HERE, "js", "doppler_hip.node")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# Per-file additions.  -amdgpu-mfma-vgpr-form: matrix-core results stay in ordinary vector
# registers.  The prefill attention rescales its accumulators between products; in accumulation
# registers every key tile paid a copy of all of them out and back (217 against 275 us at
# T = 4096).  The decode attention measured the same or slightly slower with it and stays as is.
FILE_FLAGS = {"attention_prefill.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    if out.strip():
        print(out)


def build_hip(jobs=4):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = [os.path.join(OBJ, os.path.basename(s)[:-4] + ".o") for s in srcs]
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        list(ex.map(lambda so: _run([HIPCC] + HIP_FLAGS + FILE_FLAGS.get(os.path.basename(so[0]), []) +
                                    ["-c", so[0], "-o", so[1]]), zip(srcs, objs)))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    return LIB


def build_addon():
    src = os.path.join(CSRC, "napi", "doppler_hip_napi.c")
    if not os.path.exists(src):
        return None
    inc = "/usr/include/node"
    if not os.path.exists(os.path.join(inc, "node_api.h")):
        raise RuntimeError("node_api.h not found under /usr/include/node")
    _run(["gcc", "-O2", "-fPIC", "-shared", "-std=c11", "-Wall", "-DNAPI_VERSION=6",
          "-DNODE_GYP_MODULE_NAME=doppler_hip", "-I", inc, "-I", os.path.join(HERE, "..", "include"),
          "-o", ADDON, src, "-L", LIB_DIR, "-ldopplerhip", "-Wl,-rpath,$ORIGIN/../lib"])
    return ADDON


def build_all(hip_only=False):
    lib = build_hip()
    addon = None if hip_only else build_addon()
    return lib, addon


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--hip-only", action="store_true")
    args = ap.parse_args()
    print(build_all(args.hip_only))
    sys.exit(0)
