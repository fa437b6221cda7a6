"""ctypes binding of ``libarctic_mi355x.so`` (the C ABI in ``include/arctic_mi355x.h``).

The library is the only implementation: there is no CPU or PyTorch fallback in
this package.  ``load()`` raises if the shared object is missing or cannot be
loaded, and every operator raises if it is called before a successful load.
"""
from __future__ import annotations

import ctypes
import os
import shutil
import subprocess
from typing import Optional

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_CSRC_DIR = os.path.join(_PKG_DIR, "csrc")
LIB_BASENAME = "libarctic_mi355x"
ABI_VERSION = 2

DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
KV_AUTO, KV_FP8_E4M3, KV_FP8_E5M2 = 0, 1, 2

# every symbol include/arctic_mi355x.h declares
EXPORTED_SYMBOLS = (
    "arctic_abi_version",
    "arctic_last_error",
    "arctic_reshape_and_cache_flash_bulk",
    "arctic_reshape_and_cache_flash_bulk_select",
    "arctic_reshape_and_cache_flash_bulk_select_static",
    "arctic_build_row_map",
    "arctic_reshape_and_cache_flash_fp4",
    "arctic_speculator_ln",
    "arctic_speculator_add_ln_act",
    "arctic_speculator_embed_add_ln_act",
    "arctic_sum_lstm",
    "arctic_sum_lstm_shared_z",
    "arctic_sum_lstm_embedded",
    "arctic_gather_rows",
    "arctic_argmax_clamp",
)

_lib: Optional[ctypes.CDLL] = None


def library_path() -> Optional[str]:
    """Path of the built shared object inside the package directory, or None."""
    for name in sorted(os.listdir(_PKG_DIR)):
        if name.startswith(LIB_BASENAME) and name.endswith(".so"):
            return os.path.join(_PKG_DIR, name)
    return None


def build(force: bool = True, verbose: bool = False) -> str:
    """Compile the HIP sources for gfx950 with hipcc (``make`` in ``csrc/``)."""
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        raise RuntimeError("arcticinference_amd: hipcc not found; cannot build " + LIB_BASENAME)
    cmd = ["make", "-C", _CSRC_DIR, "-j8", f"HIPCC={hipcc}", "all"]
    if force:
        cmd.append("-B")
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if verbose or proc.returncode != 0:
        print(proc.stdout)
        print(proc.stderr)
    if proc.returncode != 0:
        raise RuntimeError(f"arcticinference_amd: build failed (exit {proc.returncode})")
    path = library_path()
    if path is None:
        raise RuntimeError("arcticinference_amd: build produced no " + LIB_BASENAME + ".so")
    return path


def _declare(lib: ctypes.CDLL) -> None:
    vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
    lib.arctic_abi_version.argtypes = []
    lib.arctic_abi_version.restype = i32
    lib.arctic_last_error.argtypes = []
    lib.arctic_last_error.restype = ctypes.c_char_p
    lib.arctic_reshape_and_cache_flash_bulk.argtypes = [
        vp, vp, i64, i64,      # keys, values, key_stride, value_stride
        vp, vp, vp, vp,        # host tables: key caches, value caches, k scales, v scales
        vp, i64,               # slot_mapping, num_tokens
        i32, i32, i32, i32,    # num_layers, num_heads, head_size, block_size
        i64, i64, i32, i32, vp]  # block_stride, num_blocks, src_dtype, kv_cache_dtype, stream
    lib.arctic_reshape_and_cache_flash_bulk.restype = i32
    lib.arctic_reshape_and_cache_flash_bulk_select.argtypes = lib.arctic_reshape_and_cache_flash_bulk.argtypes[:-1] + [
        vp, vp, i32, i64, i64,   # row_map, indices, index_bytes, num_indices, num_src_rows
        vp, vp, i64, i64, vp]    # keys_out, values_out, their row strides, stream
    lib.arctic_reshape_and_cache_flash_bulk_select.restype = i32
    lib.arctic_reshape_and_cache_flash_bulk_select_static.argtypes = (
        lib.arctic_reshape_and_cache_flash_bulk.argtypes[:-1] + [
            vp, i32, i64, i64,       # indices, index_bytes, num_indices, num_src_rows
            vp, vp, i64, i64, vp])   # keys_out, values_out, their row strides, stream
    lib.arctic_reshape_and_cache_flash_bulk_select_static.restype = i32
    lib.arctic_build_row_map.argtypes = [vp, i64, vp, i32, i64, vp]
    lib.arctic_build_row_map.restype = i32
    lib.arctic_reshape_and_cache_flash_fp4.argtypes = [
        vp, vp, i64, i64, vp, vp, vp, vp, vp, i64, i32, i32, i32, i64, i64, i64, i64, i32, vp]
    lib.arctic_reshape_and_cache_flash_fp4.restype = i32
    lib.arctic_speculator_ln.argtypes = [vp, vp, vp, vp, i64, i32, i64, f32, i32, vp]
    lib.arctic_speculator_ln.restype = i32
    lib.arctic_speculator_add_ln_act.argtypes = [vp, vp, vp, vp, vp, i64, i32, i64, i64, f32, f32, i32, f32, i32, vp]
    lib.arctic_speculator_add_ln_act.restype = i32
    lib.arctic_sum_lstm.argtypes = [vp] * 9 + [i64, i32, i64, i64, i64, i64, f32, f32, f32, i32, i32, vp]
    lib.arctic_sum_lstm.restype = i32
    lib.arctic_sum_lstm_shared_z.argtypes = lib.arctic_sum_lstm.argtypes
    lib.arctic_sum_lstm_shared_z.restype = i32
    lib.arctic_sum_lstm_embedded.argtypes = [vp] * 10 + [i64, i32, i64, i64, i64, i64, i64, f32, f32, f32, i32, i32, vp]
    lib.arctic_sum_lstm_embedded.restype = i32
    lib.arctic_speculator_embed_add_ln_act.argtypes = [vp, vp, vp, vp, vp, vp, i64, i32, i64, i64, i64, f32, f32, i32,
                                                       f32, i32, vp]
    lib.arctic_speculator_embed_add_ln_act.restype = i32
    lib.arctic_gather_rows.argtypes = [i32, vp, vp, vp, vp, vp, vp, i32, i64, i64, i32, vp]
    lib.arctic_gather_rows.restype = i32
    lib.arctic_argmax_clamp.argtypes = [vp, vp, i64, i32, i64, i64, i32, vp]
    lib.arctic_argmax_clamp.restype = i32


def load() -> ctypes.CDLL:
    """Load the shared object (once) and declare its prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if path is None:
        raise RuntimeError(
            f"arcticinference_amd: {LIB_BASENAME}.so not found in {_PKG_DIR}; "
            "build it with `make -C arcticinference_amd/csrc` (needs hipcc)")
    lib = ctypes.CDLL(path)
    for sym in EXPORTED_SYMBOLS:
        if not hasattr(lib, sym):
            raise RuntimeError(f"arcticinference_amd: {path} does not export {sym}")
    _declare(lib)
    got = lib.arctic_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"arcticinference_amd: ABI version {got} != expected {ABI_VERSION}")
    _lib = lib
    return lib


def is_loaded() -> bool:
    return _lib is not None


def loaded_path() -> Optional[str]:
    return library_path() if _lib is not None else None


def last_error() -> str:
    if _lib is None:
        return ""
    msg = _lib.arctic_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(rc: int) -> None:
    """Raise RuntimeError (what TORCH_CHECK surfaces as in Python) on failure."""
    if rc != 0:
        raise RuntimeError(last_error() or f"arcticinference_amd: native call failed with code {rc}")
