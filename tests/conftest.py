import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # ARCTIC_TEST_SEED_SHIFT=k moves every `random.Random(seed)` of the tests to seed + k, so that the seeded sweeps
    # (`-k random_configurations`) can be run over other configurations than the committed ones
    shift = int(os.environ.get("ARCTIC_TEST_SEED_SHIFT", "0"))
    if shift:
        import random
        base = random.Random

        class Shifted(base):
            def __init__(self, seed=None):
                super().__init__(None if seed is None else seed + shift)

        random.Random = Shifted


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
