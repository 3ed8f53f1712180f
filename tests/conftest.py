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
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def to_dev(layer, device="cuda"):
    """numpy layer dict (oracle.make_layer) -> dict of torch tensors on the device."""
    import torch
    out = {}
    for k, v in layer.items():
        out[k] = torch.from_numpy(np.ascontiguousarray(v)).to(device) if isinstance(v, np.ndarray) else v
    return out


def bits(a):
    return np.asarray(a, dtype=np.float16).view(np.uint16)


@pytest.fixture(autouse=True)
def _automatic_launch_plans_after_every_test():
    """The library's tuning hooks are process-wide: whatever a test forced - also one that failed before its own
    clean-up ran - is back to automatic before the next test starts.  (Only if the library is loaded already.)"""
    yield
    mod = sys.modules.get("gptq_triton_amd._lib")
    lib = getattr(mod, "_lib", None) if mod is not None else None
    if lib is None:
        return
    lib.gptq4_set_tuning(0, 0, 0)
    lib.gptq4_set_gemv_tuning(1, 0, 0, 0)
    lib.gptq4_set_midm_tuning(1, 0, 0)
    lib.gptq4_set_gemm_tuning(0, 0)
    lib.gptq4_set_exchange_spin_limit(0)
    lib.gptq4_set_chain_tuning(0, 0, 0, -1)
    lib.gptq4_set_stream_tuning(0, 0)
