import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(params=["deterministic", "streamed"])
def sharing_mode(request, monkeypatch):
    """Runs a GPU test twice: with the library's default (fixed work geometry, bit-reproducible
    results) and with the `streamed_sharing` option of the attention call, under which the KV
    iterations of shared query tiles may go to whichever workgroup is free (results reproducible
    to rounding)."""
    from xdit_amd import ops
    monkeypatch.setitem(ops.TUNING, "streamed", 0 if request.param == "deterministic" else 1)
    return request.param
