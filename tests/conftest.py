import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    # GPU tests must never silently pass on a machine without a GPU
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import q4_oracle
    return q4_oracle


def to_cuda_layer(layer):
    """numpy layer dict (oracle.make_layer) -> dict of CUDA tensors."""
    import torch
    return dict(
        qweight=torch.from_numpy(layer["qweight"]).cuda(),
        qzeros=torch.from_numpy(layer["qzeros"]).cuda(),
        scales=torch.from_numpy(layer["scales"]).cuda(),
        g_idx=torch.from_numpy(layer["g_idx"]).cuda(),
        groupsize=layer["groupsize"],
    )


def rel_err(got, ref):
    """max |got - ref| / max |ref|  (the tolerance form used throughout: <= 1e-2)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.max(np.abs(got - ref)) / max(np.max(np.abs(ref)), 1e-30))
