import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def receipt():
    """Real Qwen3.5-9B gate_proj scale data copied from the reference's receipt."""
    import json
    import numpy as np
    z = np.load(os.path.join(ROOT, "tests", "golden", "qwen35_9b_gate_proj_receipt.npz"))
    return dict(d_bits=z["d_bits"], dmin_bits=z["dmin_bits"], scale_bits=z["scale_bits"],
                min_bits=z["min_bits"], sha256=json.loads(str(z["sha256"])))
