import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Parity bars: fp32 paths rtol=1e-4 / atol=1e-5; 16-bit outputs and gradients against an fp32/fp64
# reference on identical inputs rtol=2e-2 / atol=2e-2.
TOL = {"float32": dict(rtol=1e-4, atol=1e-5), "bfloat16": dict(rtol=2e-2, atol=2e-2), "float16": dict(rtol=2e-2, atol=2e-2)}


def tol_for(dtype):
    return TOL[str(dtype).replace("torch.", "")]
