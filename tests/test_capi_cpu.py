"""No-GPU checks of the C ABI: the library loads and exports exactly what the header declares,
and calls fail loudly (not silently) when no device has been initialised."""
import os
import re

import pytest

from doppler_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "doppler_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dh_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_what_python_binds():
    assert header_symbols() == sorted(capi.SIGNATURES)


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    for name in header_symbols():
        assert hasattr(lib, name), name


def test_ops_fail_loudly_without_init():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present: covered by the GPU error tests")
    lib = capi.load()
    assert lib.dh_sync() != 0
    assert b"dh_init" in lib.dh_last_error()
    assert lib.dh_q4k_matmul(None, 0, None, None, 0, 1, 1, 256, 1.0, None) != 0
    from doppler_amd import ops
    with pytest.raises(capi.DopplerHipError):
        ops.acquireBuffer(16)


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "doppler_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".js", ".mjs", ".hip", ".h", ".c")):
                src = open(os.path.join(dirpath, f), errors="replace").read()
                assert "import oracle" not in src and "from oracle" not in src and "doppler_oracle" not in src, f
