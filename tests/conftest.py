import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as graft  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    mod = graft.load_oracle()
    mod.build()
    return mod


@pytest.fixture(scope="session")
def pkg():
    return graft.load_package()


@pytest.fixture(scope="session")
def aclnn(pkg):
    if not os.path.exists(pkg.library_path()):
        pytest.fail("libcust_opapi.so is not built; run `python ops-transformer_amd/build.py`")
    pkg.aclnn.lib()
    return pkg.aclnn


@pytest.fixture(scope="session")
def dev():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test selected but no GPU is visible")
    return torch.device("cuda:0")


def bf16_round(a):
    """fp32 numpy -> fp32 numpy holding bf16-representable values (torch's round-to-nearest-even)."""
    import torch
    return torch.from_numpy(np.ascontiguousarray(a, np.float32)).to(torch.bfloat16).to(torch.float32).numpy()
