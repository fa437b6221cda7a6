"""The reference's own SuffixTree behind ctypes - TEST INFRASTRUCTURE ONLY.

`make -C oracle ref` compiles the reference's csrc/suffix_decoding/suffix_tree.cc, from where it lies, with
the C shim oracle/suffix_ref_shim.cc into oracle/_ref/libsuffix_ref.so.  Used by the tests (as the checker),
by tests/golden/make_suffix_golden.py (to write fixtures) and by bench.py's CPU-baseline leg (timed beside
the library).  Absent where the reference's sources are not available and the library was not shipped.
"""
import ctypes
import os

import numpy as np

REF_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "_ref", "libsuffix_ref.so")


class RefTree:
    """The reference's SuffixTree, compiled from its own sources by `make -C oracle ref`."""

    _lib = None

    @classmethod
    def available(cls) -> bool:
        return os.path.exists(REF_LIB)

    @classmethod
    def lib(cls):
        if cls._lib is None:
            lib = ctypes.CDLL(REF_LIB)
            vp, i32, i64, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
            lib.ref_suffix_tree_create.restype = vp
            lib.ref_suffix_tree_create.argtypes = [i32]
            lib.ref_suffix_tree_destroy.argtypes = [vp]
            lib.ref_suffix_tree_num_seqs.argtypes = [vp]
            lib.ref_suffix_tree_extend.argtypes = [vp, i32, vp, i64]
            lib.ref_suffix_tree_remove.argtypes = [vp, i32]
            lib.ref_suffix_tree_speculate.argtypes = [vp, vp, i64, i32, f32, f32, f32, i32, vp, vp, vp,
                                                      ctypes.POINTER(f32), ctypes.POINTER(i32)]
            lib.ref_suffix_tree_check_integrity.argtypes = [vp, ctypes.c_char_p, i32]
            cls._lib = lib
        return cls._lib

    def __init__(self, max_depth: int):
        self._h = self.lib().ref_suffix_tree_create(max_depth)

    def __del__(self):
        if getattr(self, "_h", None):
            self.lib().ref_suffix_tree_destroy(self._h)
            self._h = None

    def num_seqs(self):
        return self.lib().ref_suffix_tree_num_seqs(self._h)

    def extend(self, seq_id, tokens):
        a = np.ascontiguousarray(tokens, dtype=np.int32)
        self.lib().ref_suffix_tree_extend(self._h, seq_id, a.ctypes.data, a.size)

    def remove(self, seq_id):
        self.lib().ref_suffix_tree_remove(self._h, seq_id)

    def speculate(self, context, k, factor, offset, min_prob, use_tree):
        ctx = np.ascontiguousarray(context, dtype=np.int32)
        cap = max(k, 0)
        a, b, c = np.empty(cap, np.int32), np.empty(cap, np.int32), np.empty(cap, np.float32)
        s, m = ctypes.c_float(), ctypes.c_int()
        n = self.lib().ref_suffix_tree_speculate(self._h, ctx.ctypes.data, ctx.size, k, factor, offset, min_prob,
                                                 int(use_tree), a.ctypes.data, b.ctypes.data, c.ctypes.data,
                                                 ctypes.byref(s), ctypes.byref(m))
        return a[:n].tolist(), b[:n].tolist(), c[:n].tolist(), s.value, m.value

    def check_integrity(self):
        buf = ctypes.create_string_buffer(512)
        self.lib().ref_suffix_tree_check_integrity(self._h, buf, len(buf))
        return buf.value.decode()
