"""MI355X (gfx950) implementation of ArcticInference's ``csrc/custom_ops`` hot path.

``arcticinference_amd.py_custom_ops`` is the drop-in counterpart of the
reference's ``arctic_inference/py_custom_ops.py``: it loads the HIP library
through its C ABI and registers the ``torch.ops.arctic_inference`` operators.
"""
__version__ = "0.1.0"

from . import py_custom_ops  # noqa: F401
from .py_custom_ops import (  # noqa: F401
    gather_rows,
    reshape_and_cache_flash_bulk,
    reshape_and_cache_flash_bulk_select,
    reshape_and_cache_flash_fp4,
    scatter_rows,
    speculator_add_ln_gelu,
    speculator_argmax,
    speculator_embed_add_ln_gelu,
    speculator_ln,
    speculator_ln_scaled,
    sum_lstm,
    sum_lstm_embedded,
    sum_lstm_shared_z,
    try_load_jit_library,
    try_load_torch_library,
)
