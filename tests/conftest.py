import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# fp32 tolerance stated by the task for hidden states, attention weights and log-probs
RTOL = 1e-4
ATOL = 1e-5


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def assert_close(a, b, what="", rtol=RTOL, atol=ATOL):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    assert a.shape == b.shape, f"{what}: shape {a.shape} vs {b.shape}"
    err = np.abs(a - b)
    lim = atol + rtol * np.abs(b)
    if not np.all(err <= lim):
        i = np.unravel_index(np.argmax(err - lim), err.shape)
        raise AssertionError(f"{what}: max violation at {i}: got {a[i]!r} want {b[i]!r} "
                             f"(|err|={err[i]:.3e}, limit={lim[i]:.3e}); "
                             f"{int(np.sum(err > lim))} of {err.size} elements out of tolerance")


@pytest.fixture(scope="session")
def orc():
    from oracle import orc as _orc
    _orc.lib()
    return _orc


@pytest.fixture(scope="session")
def lh():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from linmt_amd import lib
    lib.load()
    return lib
