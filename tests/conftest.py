import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def ops():
    """The drop-in operator module with the HIP library loaded.  GPU tests fail
    (not skip) when the library is missing: there is no fallback to test."""
    import torch
    from arcticinference_amd import py_custom_ops

    assert torch.cuda.is_available(), "GPU test selected but no GPU is visible"
    assert py_custom_ops.try_load_torch_library(), (
        "libarctic_mi355x.so is not built / not loadable; run `make -C arcticinference_amd/csrc`")
    return py_custom_ops
