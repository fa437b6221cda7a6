"""CPU oracle for the custom_ops hot path: TEST INFRASTRUCTURE ONLY.

Python face of ``arctic_oracle.c`` (loaded with ctypes).  The wrappers take CPU
torch tensors and have the same signatures as the ``torch.ops.arctic_inference``
operators they check (csrc/custom_ops/torch_bindings.cpp:7-49 in the reference).

Only tests, the smoke test and the benchmark's CPU-baseline leg may import this
package.  The shipped package ``arcticinference_amd`` never does.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import List, Optional, Sequence, Tuple

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libarctic_oracle.so")

F32, F16, BF16 = 0, 1, 2
KV_AUTO, KV_FP8_E4M3, KV_FP8_E5M2 = 0, 1, 2

_SRC_DTYPE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}
_KV_DTYPE = {"auto": KV_AUTO, "fp8": KV_FP8_E4M3, "fp8_e4m3": KV_FP8_E4M3,
             "fp8_e5m2": KV_FP8_E5M2}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make`` in this directory)."""
    if force or not os.path.exists(_LIB_PATH) or (
            os.path.getmtime(_LIB_PATH)
            < os.path.getmtime(os.path.join(_HERE, "arctic_oracle.c"))):
        args = ["make", "-C", _HERE] + (["-B"] if force else [])
        subprocess.run(args, check=True, capture_output=True)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, i32, f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
        L.ao_f32_to_e4m3fn.argtypes = [f32]
        L.ao_f32_to_e4m3fn.restype = ctypes.c_uint8
        L.ao_f32_to_e5m2.argtypes = [f32]
        L.ao_f32_to_e5m2.restype = ctypes.c_uint8
        L.ao_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
        L.ao_e4m3fn_to_f32.restype = f32
        L.ao_e5m2_to_f32.argtypes = [ctypes.c_uint8]
        L.ao_e5m2_to_f32.restype = f32
        L.ao_f32_to_bf16.argtypes = [f32]
        L.ao_f32_to_bf16.restype = ctypes.c_uint16
        L.ao_f32_to_f16.argtypes = [f32]
        L.ao_f32_to_f16.restype = ctypes.c_uint16
        L.ao_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.ao_f16_to_f32.restype = f32
        L.ao_scaled_convert.argtypes = [vp, vp, i64, f32, i32, i32]
        L.ao_scaled_convert.restype = None
        L.ao_reshape_and_cache_flash_bulk.argtypes = [
            vp, vp, i64, i64, vp, vp, vp, vp, vp, i64, i32, i32, i32, i32, i64,
            i32, i32]
        L.ao_reshape_and_cache_flash_bulk.restype = i32
        L.ao_f32_to_e2m1.argtypes = [f32]
        L.ao_f32_to_e2m1.restype = ctypes.c_uint8
        L.ao_e2m1_to_f32.argtypes = [ctypes.c_uint8]
        L.ao_e2m1_to_f32.restype = f32
        L.ao_reshape_and_cache_flash_fp4.argtypes = [vp, vp, i64, i64, vp, vp, vp, vp, vp, i64, i32, i32, i32,
                                                     i64, i64, i64, i32]
        L.ao_reshape_and_cache_flash_fp4.restype = i32
        L.ao_speculator_ln.argtypes = [vp, vp, vp, vp, i64, i32, i64, f32, i32]
        L.ao_speculator_ln.restype = i32
        L.ao_speculator_add_ln_act.argtypes = [vp, vp, vp, vp, vp, i64, i32, i64, i64, f32, f32, i32, f32, i32]
        L.ao_speculator_add_ln_act.restype = i32
        L.ao_sum_lstm.argtypes = [vp] * 9 + [i64, i32, i64, i64, i64, i64, f32,
                                             f32, f32, i32, i32]
        L.ao_sum_lstm.restype = i32
        L.ao_num_threads.restype = i32
        L.ao_set_num_threads.argtypes = [i32]
        _lib = L
    return _lib


def num_threads() -> int:
    return int(lib().ao_num_threads())


def set_num_threads(n: int) -> None:
    lib().ao_set_num_threads(int(n))


def _cpu(t: torch.Tensor, name: str) -> torch.Tensor:
    if t.device.type != "cpu":
        raise ValueError(f"oracle: {name} must be a CPU tensor")
    return t


def scaled_convert(x: torch.Tensor, scale: float, kv_cache_dtype: str = "fp8") -> torch.Tensor:
    """uint8 fp8 codes of ``x / scale`` (quant_utils.cuh:456-489,515-526)."""
    x = _cpu(x, "x").contiguous()
    out = torch.empty(x.shape, dtype=torch.uint8)
    lib().ao_scaled_convert(x.data_ptr(), out.data_ptr(), x.numel(), float(scale),
                            _SRC_DTYPE[x.dtype], _KV_DTYPE[kv_cache_dtype])
    return out


def e4m3fn_decode(codes: torch.Tensor) -> torch.Tensor:
    L = lib()
    table = torch.tensor([L.ao_e4m3fn_to_f32(c) for c in range(256)], dtype=torch.float32)
    return table[codes.to(torch.int64)]


def e5m2_decode(codes: torch.Tensor) -> torch.Tensor:
    L = lib()
    table = torch.tensor([L.ao_e5m2_to_f32(c) for c in range(256)], dtype=torch.float32)
    return table[codes.to(torch.int64)]


def _ptr_array(tensors: Sequence[torch.Tensor]):
    arr = (ctypes.c_void_p * len(tensors))()
    for i, t in enumerate(tensors):
        arr[i] = t.data_ptr()
    return arr


def reshape_and_cache_flash_bulk(
    keys: torch.Tensor,
    values: torch.Tensor,
    key_caches: List[torch.Tensor],
    value_caches: List[torch.Tensor],
    slot_mapping: torch.Tensor,
    kv_cache_dtype: str,
    k_scales: List[torch.Tensor],
    v_scales: List[torch.Tensor],
    num_heads: int,
    head_size: int,
) -> None:
    """In-place bulk KV write on CPU tensors; argument meaning as in
    csrc/custom_ops/reshape_and_cache_flash_bulk.cu:77-102."""
    L = len(key_caches)
    if L == 0:
        return
    assert len(value_caches) == L and len(k_scales) == L and len(v_scales) == L
    for t in (keys, values, slot_mapping, *key_caches, *value_caches, *k_scales, *v_scales):
        _cpu(t, "tensor")
    assert slot_mapping.dtype == torch.int64 and slot_mapping.is_contiguous()
    assert keys.stride(-1) == 1 and values.stride(-1) == 1
    block_size = key_caches[0].size(1)
    block_stride = key_caches[0].stride(0)
    assert block_stride == value_caches[0].stride(0)
    k_scales = [s.to(torch.float32) for s in k_scales]
    v_scales = [s.to(torch.float32) for s in v_scales]
    rc = lib().ao_reshape_and_cache_flash_bulk(
        keys.data_ptr(), values.data_ptr(), keys.stride(0), values.stride(0),
        _ptr_array(key_caches), _ptr_array(value_caches), _ptr_array(k_scales),
        _ptr_array(v_scales), slot_mapping.data_ptr(), slot_mapping.size(0), L,
        int(num_heads), int(head_size), int(block_size), int(block_stride),
        _SRC_DTYPE[keys.dtype], _KV_DTYPE[kv_cache_dtype])
    if rc != 0:
        raise RuntimeError("oracle: unsupported dtype combination")


def fp4_layout(key: torch.Tensor, key_cache: torch.Tensor):
    """(is_nhd, block_size, block_stride, page_stride, head_stride) exactly as the reference's
    host code derives them (csrc/custom_ops/reshape_and_cache_flash_fp4.cu:266-280)."""
    num_heads = key.size(1)
    is_nhd = key_cache.size(2) == num_heads
    block_stride = key_cache.stride(0)
    page_stride = key_cache.stride(1) if is_nhd else key_cache.stride(2)
    head_stride = key_cache.stride(2) if is_nhd else key_cache.stride(1)
    block_size = key_cache.size(1) if is_nhd else key_cache.size(2)
    return is_nhd, block_size, block_stride, page_stride, head_stride


def reshape_and_cache_flash_fp4(keys: torch.Tensor, values: torch.Tensor, key_cache: torch.Tensor,
                                value_cache: torch.Tensor, key_cache_scales: torch.Tensor,
                                value_cache_scales: torch.Tensor, slot_mapping: torch.Tensor,
                                kv_cache_dtype: str, k_scale: torch.Tensor, v_scale: torch.Tensor) -> None:
    """In-place NVFP4-style cache write on CPU tensors; argument order of the reference's Python
    wrapper (arctic_inference/py_custom_ops.py:76-90)."""
    for t in (keys, values, key_cache, value_cache, key_cache_scales, value_cache_scales, slot_mapping):
        _cpu(t, "tensor")
    assert key_cache.dim() == 4 and value_cache.dim() == 4
    _, block_size, block_stride, page_stride, head_stride = fp4_layout(keys, key_cache)
    rc = lib().ao_reshape_and_cache_flash_fp4(
        keys.data_ptr(), values.data_ptr(), keys.stride(0), values.stride(0), key_cache.data_ptr(),
        value_cache.data_ptr(), key_cache_scales.data_ptr(), value_cache_scales.data_ptr(),
        slot_mapping.data_ptr(), slot_mapping.size(0), keys.size(1), keys.size(2), block_size, block_stride,
        page_stride, head_stride, _SRC_DTYPE[keys.dtype])
    if rc != 0:
        raise RuntimeError("oracle: fp4 cache write needs fp16/bf16 input and head_size % 16 == 0")


def e2m1_decode(nibbles: torch.Tensor) -> torch.Tensor:
    L = lib()
    table = torch.tensor([L.ao_e2m1_to_f32(c) for c in range(16)], dtype=torch.float32)
    return table[nibbles.to(torch.int64)]


def speculator_ln(input: torch.Tensor, weight: Optional[torch.Tensor],
                  bias: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """RMS-style norm; output is dense like ``empty_like(input)``
    (csrc/custom_ops/speculator_ln.cu:152-201)."""
    _cpu(input, "input")
    hidden = input.size(-1)
    assert input.stride(-1) == 1
    in2 = input.view(-1, hidden)
    out = torch.empty(input.shape, dtype=input.dtype)
    w = weight.contiguous() if weight is not None else None
    b = bias.contiguous() if bias is not None else None
    rc = lib().ao_speculator_ln(
        out.data_ptr(), in2.data_ptr(), w.data_ptr() if w is not None else None,
        b.data_ptr() if b is not None else None, in2.size(0), hidden,
        in2.stride(0) if in2.size(0) > 1 else hidden, float(eps), _SRC_DTYPE[input.dtype])
    if rc != 0:
        raise RuntimeError("oracle: speculator_ln supports fp16/bf16 only")
    return out


_ACTIVATION = {"none": 0, "gelu": 1, "gelu_tanh": 2}


def speculator_add_ln_act(input: torch.Tensor, z: Optional[torch.Tensor], weight: Optional[torch.Tensor],
                          bias: Optional[torch.Tensor], alpha: float, eps: float, activation: str,
                          out_scale: float) -> torch.Tensor:
    """``act(ln(input + alpha * z)) * out_scale`` with the roundings of the separate PyTorch ops
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:296-307, 733-734, 809-816)."""
    _cpu(input, "input")
    hidden = input.size(-1)
    assert input.stride(-1) == 1
    in2 = input.view(-1, hidden)
    z2 = None
    if z is not None:
        _cpu(z, "z")
        assert z.shape == input.shape and z.dtype == input.dtype and z.stride(-1) == 1
        z2 = z.view(-1, hidden)
    out = torch.empty(input.shape, dtype=input.dtype)
    w = weight.contiguous() if weight is not None else None
    b = bias.contiguous() if bias is not None else None
    rows = in2.size(0)
    rc = lib().ao_speculator_add_ln_act(
        out.data_ptr(), in2.data_ptr(), z2.data_ptr() if z2 is not None else None,
        w.data_ptr() if w is not None else None, b.data_ptr() if b is not None else None, rows, hidden,
        in2.stride(0) if rows > 1 else hidden, (z2.stride(0) if rows > 1 else hidden) if z2 is not None else 0,
        float(alpha), float(eps), _ACTIVATION[activation], float(out_scale), _SRC_DTYPE[input.dtype])
    if rc != 0:
        raise RuntimeError("oracle: speculator_add_ln_act supports fp16/bf16 and activations none/gelu/gelu_tanh")
    return out


def sum_lstm(states_4d: torch.Tensor, z4_4d: torch.Tensor, prev_cell_d: torch.Tensor,
             w_cell: Optional[torch.Tensor], b_cell: Optional[torch.Tensor],
             w_state: Optional[torch.Tensor], b_state: Optional[torch.Tensor],
             alpha: float, eps_cell: float, eps_state: float,
             use_fast_gelu: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """(state, cell); outputs inherit prev_cell's 2-D strides
    (csrc/custom_ops/sum_lstm.cu:346-365)."""
    for t in (states_4d, z4_4d, prev_cell_d):
        _cpu(t, "input")
    D = prev_cell_d.size(-1)
    s2 = states_4d.view(-1, 4 * D)
    z2 = z4_4d.view(-1, 4 * D)
    p2 = prev_cell_d.view(-1, D)
    out_cell = torch.empty_strided(p2.shape, p2.stride(), dtype=p2.dtype)
    out_state = torch.empty_strided(p2.shape, p2.stride(), dtype=p2.dtype)
    rows = s2.size(0)

    def st(t):
        return t.stride(0) if rows > 1 else t.size(1)

    def p(t):
        return t.data_ptr() if t is not None else None

    rc = lib().ao_sum_lstm(
        out_state.data_ptr(), out_cell.data_ptr(), s2.data_ptr(), z2.data_ptr(),
        p2.data_ptr(), p(w_cell), p(b_cell), p(w_state), p(b_state), rows, D,
        st(s2), st(z2), st(p2), st(out_cell), float(alpha), float(eps_cell),
        float(eps_state), int(bool(use_fast_gelu)), _SRC_DTYPE[states_4d.dtype])
    if rc != 0:
        raise RuntimeError("oracle: sum_lstm supports fp16/bf16 only")
    return out_state.view(prev_cell_d.shape), out_cell.view(prev_cell_d.shape)


def gather_rows(sources, indices: torch.Tensor, outs=None):
    """The reference's own expression on the CPU: ``torch.index_select(t, 0, indices, out=buf[:n])`` per
    tensor (arctic_inference/vllm/swiftkv/llama_swiftkv.py:663-679).  Rows whose index is out of range
    are left as they are (torch raises there; the kernel skips)."""
    n = indices.numel()
    idx = indices.to(torch.int64)
    result = []
    for k, src in enumerate(sources):
        _cpu(src, "source")
        out = outs[k] if outs is not None and outs[k] is not None else torch.zeros(
            (n,) + tuple(src.shape[1:]), dtype=src.dtype)
        ok = (idx >= 0) & (idx < src.size(0))
        rows = torch.nonzero(ok).flatten()
        out[rows] = src.index_select(0, idx[rows])
        result.append(out)
    return result


def scatter_rows(sources, indices: torch.Tensor, outs) -> None:
    """``out[indices] = src[:n]`` per tensor (arctic_inference/vllm/swiftkv/llama_swiftkv.py:733-742);
    out-of-range indices are skipped."""
    n = indices.numel()
    idx = indices.to(torch.int64)
    for src, out in zip(sources, outs):
        _cpu(src, "source")
        ok = (idx >= 0) & (idx < out.size(0))
        rows = torch.nonzero(ok).flatten()
        out[idx[rows]] = src[:n][rows]
