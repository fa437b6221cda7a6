"""ctypes binding of ``libarctic_suffix.so`` (the C ABI in ``include/arctic_suffix.h``).

``SuffixTree`` and ``Draft`` have the methods and attributes of the classes the reference binds with
nanobind (csrc/suffix_decoding/bindings.cc:79-102).  There is no Python fallback: without the shared
object this module raises on import.
"""
from __future__ import annotations

import ctypes
import os
from typing import List, Sequence

import numpy as np

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_BASENAME = "libarctic_suffix"
ABI_VERSION = 1

# every symbol include/arctic_suffix.h declares
EXPORTED_SYMBOLS = (
    "arctic_suffix_abi_version",
    "arctic_suffix_tree_create",
    "arctic_suffix_tree_destroy",
    "arctic_suffix_tree_num_seqs",
    "arctic_suffix_tree_append",
    "arctic_suffix_tree_extend",
    "arctic_suffix_tree_remove",
    "arctic_suffix_tree_speculate",
    "arctic_suffix_tree_check_integrity",
    "arctic_suffix_tree_estimate_memory",
)


def library_path() -> str:
    path = os.path.join(_PKG_DIR, LIB_BASENAME + ".so")
    if not os.path.exists(path):
        raise ImportError(f"arcticinference_amd: {LIB_BASENAME}.so not found in {_PKG_DIR}; "
                          "build it with `make -C arcticinference_amd/csrc`")
    return path


def _load() -> ctypes.CDLL:
    lib = ctypes.CDLL(library_path())
    for sym in EXPORTED_SYMBOLS:
        if not hasattr(lib, sym):
            raise ImportError(f"arcticinference_amd: {LIB_BASENAME}.so does not export {sym}")
    vp, i32, i64, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
    lib.arctic_suffix_abi_version.restype = i32
    lib.arctic_suffix_tree_create.argtypes = [i32]
    lib.arctic_suffix_tree_create.restype = vp
    lib.arctic_suffix_tree_destroy.argtypes = [vp]
    lib.arctic_suffix_tree_destroy.restype = None
    lib.arctic_suffix_tree_num_seqs.argtypes = [vp]
    lib.arctic_suffix_tree_append.argtypes = [vp, i32, ctypes.c_int32]
    lib.arctic_suffix_tree_extend.argtypes = [vp, i32, vp, i64]
    lib.arctic_suffix_tree_remove.argtypes = [vp, i32]
    lib.arctic_suffix_tree_speculate.argtypes = [vp, vp, i64, i32, f32, f32, f32, i32, vp, vp, vp,
                                                 ctypes.POINTER(f32), ctypes.POINTER(i32)]
    lib.arctic_suffix_tree_check_integrity.argtypes = [vp, ctypes.c_char_p, i32]
    lib.arctic_suffix_tree_estimate_memory.argtypes = [vp]
    lib.arctic_suffix_tree_estimate_memory.restype = ctypes.c_size_t
    if lib.arctic_suffix_abi_version() != ABI_VERSION:
        raise ImportError(f"arcticinference_amd: {LIB_BASENAME}.so has ABI version "
                          f"{lib.arctic_suffix_abi_version()}, expected {ABI_VERSION}")
    return lib


_lib = _load()


class Draft:
    """Result of one speculation (the reference's Draft, csrc/suffix_decoding/suffix_tree.h:101-117)."""
    __slots__ = ("token_ids", "parents", "probs", "score", "match_len")

    def __init__(self, token_ids=None, parents=None, probs=None, score: float = 0.0, match_len: int = 0):
        self.token_ids: List[int] = token_ids if token_ids is not None else []
        self.parents: List[int] = parents if parents is not None else []
        self.probs: List[float] = probs if probs is not None else []
        self.score = score
        self.match_len = match_len


def _as_int32(tokens) -> np.ndarray:
    return np.ascontiguousarray(tokens, dtype=np.int32)


def _require_int32_vector(tokens, what: str) -> None:
    """The reference's binding takes nb::ndarray<int32_t, nb::ndim<1>, nb::c_contig> (csrc/suffix_decoding/bindings.cc:79-102)
    and turns anything else away; here the array's memory is handed to C as it is, so the same must hold."""
    if not (isinstance(tokens, np.ndarray) and tokens.dtype == np.int32 and tokens.ndim == 1
            and tokens.flags["C_CONTIGUOUS"]):
        raise TypeError(f"{what}: expected a C-contiguous 1-D numpy array of int32")


def _check(rc: int, what: str) -> int:
    if rc < 0:
        raise MemoryError(f"{what}: out of memory") if rc == -2 else ValueError(f"{what}: invalid argument")
    return rc


class SuffixTree:
    """A suffix tree over token sequences, depth-limited, with speculation of likely continuations."""

    def __init__(self, max_depth: int):
        self._handle = _lib.arctic_suffix_tree_create(int(max_depth))
        if not self._handle:
            raise ValueError("SuffixTree: max_depth must be a positive integer")
        self._score, self._match_len = ctypes.c_float(0.0), ctypes.c_int(0)
        self._score_ref, self._match_len_ref = ctypes.byref(self._score), ctypes.byref(self._match_len)
        self._reserve(64)

    def _reserve(self, capacity: int) -> None:
        # output arrays of speculate, kept between calls
        self._capacity = capacity
        self._token_ids = np.empty(capacity, dtype=np.int32)
        self._parents = np.empty(capacity, dtype=np.int32)
        self._probs = np.empty(capacity, dtype=np.float32)
        self._out = (self._token_ids.ctypes.data, self._parents.ctypes.data, self._probs.ctypes.data)

    def __del__(self):
        handle, self._handle = getattr(self, "_handle", None), None
        if handle:
            _lib.arctic_suffix_tree_destroy(handle)

    def num_seqs(self) -> int:
        return _lib.arctic_suffix_tree_num_seqs(self._handle)

    def append(self, seq_id: int, token: int) -> None:
        _check(_lib.arctic_suffix_tree_append(self._handle, seq_id, token), "append")

    def extend(self, seq_id: int, tokens: Sequence[int]) -> None:
        self.extend_ndarray(seq_id, _as_int32(tokens))

    def extend_ndarray(self, seq_id: int, tokens: np.ndarray) -> None:
        _require_int32_vector(tokens, "extend_ndarray")
        _check(_lib.arctic_suffix_tree_extend(self._handle, seq_id, tokens.ctypes.data, tokens.size), "extend")

    def remove(self, seq_id: int) -> None:
        _check(_lib.arctic_suffix_tree_remove(self._handle, seq_id), "remove")

    def speculate(self, context: Sequence[int], max_spec_tokens: int, max_spec_factor: float,
                  max_spec_offset: float, min_token_prob: float, use_tree_spec: bool) -> Draft:
        return self.speculate_ndarray(_as_int32(context), max_spec_tokens, max_spec_factor, max_spec_offset,
                                      min_token_prob, use_tree_spec)

    def speculate_ndarray(self, context: np.ndarray, max_spec_tokens: int, max_spec_factor: float,
                          max_spec_offset: float, min_token_prob: float, use_tree_spec: bool) -> Draft:
        _require_int32_vector(context, "speculate_ndarray")
        max_spec_tokens = int(max_spec_tokens)
        if max_spec_tokens > self._capacity:
            self._reserve(max_spec_tokens)
        n = _lib.arctic_suffix_tree_speculate(
            self._handle, context.ctypes.data, context.size, max_spec_tokens, max_spec_factor, max_spec_offset,
            min_token_prob, 1 if use_tree_spec else 0, *self._out, self._score_ref, self._match_len_ref)
        if n < 0:
            _check(n, "speculate")
        return Draft(self._token_ids[:n].tolist(), self._parents[:n].tolist(), self._probs[:n].tolist(),
                     self._score.value, self._match_len.value)

    def check_integrity(self) -> str:
        """Empty string if every invariant of the tree holds, else a description of the first broken one."""
        buf = ctypes.create_string_buffer(512)
        _check(_lib.arctic_suffix_tree_check_integrity(self._handle, buf, len(buf)), "check_integrity")
        return buf.value.decode()

    def estimate_memory(self) -> int:
        return _lib.arctic_suffix_tree_estimate_memory(self._handle)
