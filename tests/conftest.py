import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle.oracle import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def reference():
    """The reference's own ggml code (oracle/_ref), present only where it was built."""
    from oracle.oracle import Reference
    if not Reference.available():
        pytest.skip("oracle/_ref/libggml_ref.so not built (reference checkout absent)")
    return Reference()


@pytest.fixture(scope="session")
def golden():
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "golden.npz")
    return np.load(path, allow_pickle=False)


@pytest.fixture(scope="session")
def hip():
    """The HIP backend facade; fails loudly if the library is missing or no GPU answers."""
    from tensorsharp_amd import HipBasicOps, hip_native
    hip_native.lib()
    assert HipBasicOps.IsAvailable(), hip_native.get_last_error()
    return HipBasicOps
