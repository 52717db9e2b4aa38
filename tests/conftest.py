import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP kernels through the C ABI)")


@pytest.fixture(scope="session", autouse=True)
def built_artifacts():
    """Load what is built; build only if nothing is (hipcc cross-compiles without a GPU)."""
    from tritonformer_amd import _build, _lib

    if not (os.path.exists(_lib.LIB_PATH) and os.path.exists(_lib.DIAG_LIB_PATH)):
        _build.build_library(verbose=False)
    _lib.load()   # refuses a library built from other sources than the ones in the tree
    ref_so = os.path.join(ROOT, "oracle", "libref_ops.so")
    if not os.path.exists(ref_so):
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle")], check=True, capture_output=True)
    return _lib.LIB_PATH


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
