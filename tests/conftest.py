import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    # GPU tests are selected with -m gpu; without a GPU they are skipped, never silently passed
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    import oracle as orc
    orc.oracle_lib()
    return orc


def to_device(nb, dtype, device="cuda:0"):
    """7-tensor NumPy batch -> torch tensors on the device."""
    import torch
    out = {}
    for k in ("binum", "bilist", "bnumneigh", "bfirstneigh", "btypes"):
        out[k] = torch.from_numpy(np.ascontiguousarray(nb[k], np.int32)).to(device)
    out["brcs"] = torch.from_numpy(np.ascontiguousarray(nb["brcs"])).to(dtype).to(device)
    out["nghost"] = int(nb.get("nghost", 0))
    return out
