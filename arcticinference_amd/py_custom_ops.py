"""Drop-in ``torch.ops.arctic_inference.*`` surface backed by gfx950 HIP kernels.

Mirrors the operator boundary of the reference
(``arctic_inference/py_custom_ops.py:9-118`` and the schemas in
``csrc/custom_ops/torch_bindings.cpp:6-51``): same namespace, same schema
strings, same wrapper names and argument meaning, the same argument checks with
the same message prefixes.  The reference registers compiled C++ functions from
a pybind extension; here the schemas are defined from Python and the ``CUDA``
dispatch key (HIP tensors under PyTorch-ROCm) is bound to thin shims that unwrap
tensors into pointers, sizes and strides and call the C ABI of
``libarctic_mi355x.so`` on the current stream.

There is no fallback: without the shared object ``try_load_torch_library()``
returns ``False`` (as the reference does) and every operator raises.
"""
from __future__ import annotations

import ctypes
import logging
from typing import List, Optional, Tuple

import torch

from . import _native

logger = logging.getLogger(__name__)

_NAMESPACE = "arctic_inference"

# Schemas as registered by the reference (csrc/custom_ops/torch_bindings.cpp:7-49).
_SCHEMAS = {
    "reshape_and_cache_flash_bulk":
        "reshape_and_cache_flash_bulk(Tensor keys, Tensor values, Tensor(c!)[] key_caches, "
        "Tensor(d!)[] value_caches, Tensor slot_mapping, str kv_cache_dtype, Tensor(e)[] k_scales, "
        "Tensor(f)[] v_scales, int num_heads, int head_size) -> ()",
    "reshape_and_cache_flash_fp4":
        "reshape_and_cache_flash_fp4(Tensor key, Tensor value, Tensor(c!) key_cache, "
        "Tensor(d!) value_cache, Tensor slot_mapping, str kv_cache_dtype, Tensor k_scale, "
        "Tensor v_scale, Tensor(e!) key_scale_cache, Tensor(f!) value_scale_cache) -> ()",
    "speculator_ln_cuda":
        "speculator_ln_cuda(Tensor input, Tensor? weight, Tensor? bias, float eps) -> Tensor",
    "sum_lstm_cuda":
        "sum_lstm_cuda(Tensor states_4d, Tensor z4_4d, Tensor prev_cell_d, Tensor? w_cell, "
        "Tensor? b_cell, Tensor? w_state, Tensor? b_state, float alpha, float eps_cell, "
        "float eps_state, bool use_fast_gelu) -> (Tensor, Tensor)",
}

# Operators that fuse a caller-side step into one of the above; the reference has no such schema.
_EXTRA_SCHEMAS = {
    "sum_lstm_shared_z_cuda":
        "sum_lstm_shared_z_cuda(Tensor states_4d, Tensor z_d, Tensor? prev_cell_d, Tensor? w_cell, "
        "Tensor? b_cell, Tensor? w_state, Tensor? b_state, float alpha, float eps_cell, "
        "float eps_state, bool use_fast_gelu) -> (Tensor, Tensor)",
    "sum_lstm_zero_cell_cuda":
        "sum_lstm_zero_cell_cuda(Tensor states_4d, Tensor z4_4d, Tensor? w_cell, Tensor? b_cell, Tensor? w_state, "
        "Tensor? b_state, float alpha, float eps_cell, float eps_state, bool use_fast_gelu) -> (Tensor, Tensor)",
    "speculator_add_ln_act_cuda":
        "speculator_add_ln_act_cuda(Tensor input, Tensor? z, Tensor? weight, Tensor? bias, float alpha, "
        "float eps, str activation, float out_scale) -> Tensor",
    "sum_lstm_embedded_cuda":
        "sum_lstm_embedded_cuda(Tensor states_4d, Tensor emb_weight, Tensor token_ids, Tensor? prev_cell_d, "
        "Tensor? w_cell, Tensor? b_cell, Tensor? w_state, Tensor? b_state, float alpha, float eps_cell, "
        "float eps_state, bool use_fast_gelu) -> (Tensor, Tensor)",
    "speculator_embed_add_ln_act_cuda":
        "speculator_embed_add_ln_act_cuda(Tensor input, Tensor emb_weight, Tensor token_ids, Tensor? weight, "
        "Tensor? bias, float alpha, float eps, str activation, float out_scale) -> Tensor",
    "speculator_argmax_cuda": "speculator_argmax_cuda(Tensor logits, int max_index) -> Tensor",
    "reshape_and_cache_flash_bulk_select":
        "reshape_and_cache_flash_bulk_select(Tensor keys, Tensor values, Tensor(c!)[] key_caches, "
        "Tensor(d!)[] value_caches, Tensor slot_mapping, str kv_cache_dtype, Tensor(e)[] k_scales, "
        "Tensor(f)[] v_scales, int num_heads, int head_size, Tensor logits_indices, Tensor(g!) k_out, "
        "Tensor(h!) v_out) -> ()",
    "gather_rows": "gather_rows(Tensor[] sources, Tensor indices, Tensor(a!)[] outs) -> ()",
    "scatter_rows": "scatter_rows(Tensor[] sources, Tensor indices, Tensor(a!)[] outs) -> ()",
}

_SRC_DTYPES = {
    torch.float32: _native.DTYPE_F32,
    torch.float16: _native.DTYPE_F16,
    torch.bfloat16: _native.DTYPE_BF16,
}
_HALF_DTYPES = {torch.float16: _native.DTYPE_F16, torch.bfloat16: _native.DTYPE_BF16}
_SELECT_SCAN_MAX_INDICES = 2048   # ARCTIC_SELECT_SCAN_MAX_INDICES of the C ABI

_torch_lib: Optional[torch.library.Library] = None
_registered = False


def _check(cond: bool, msg: str) -> None:
    # TORCH_CHECK raises c10::Error, which Python sees as RuntimeError.  Checks whose message has to be
    # formatted are written out as `if not (...): raise RuntimeError(f"...")` instead, so that the call
    # path that succeeds formats nothing: these shims run once per operator call.
    if not cond:
        raise RuntimeError(msg)


def _lib() -> ctypes.CDLL:
    if not _native.is_loaded():
        raise RuntimeError(
            "arctic_inference custom ops are not loaded: call try_load_torch_library() "
            "and check that it returned True (libarctic_mi355x.so must be built)")
    return _native.load()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_of(t: torch.Tensor) -> int:
    """hipStream_t of torch's current stream on the tensor's device (what
    at::cuda::getCurrentCUDAStream() is to the reference)."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index if t.device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(t.device).cuda_stream


def _rows_of(t: torch.Tensor, cols: int) -> torch.Tensor:
    """``t.view(-1, cols)``; a tensor that is 2-D already is passed through (a view costs a microsecond of
    host time, and the speculator hands over 2-D tensors).  A single row still goes through view(), which
    sets its row stride to ``cols`` as the reference's view() does."""
    return t if t.dim() == 2 and t.size(0) != 1 else t.view(-1, cols)


class _on_device_of:
    """OptionalCUDAGuard: make the tensor's device current for the launch."""

    def __init__(self, t: torch.Tensor):
        self.idx = t.device.index
        self.prev = None

    def __enter__(self):
        cur = torch.cuda.current_device()
        if self.idx is not None and self.idx != cur:
            self.prev = cur
            torch.cuda.set_device(self.idx)

    def __exit__(self, *exc):
        if self.prev is not None:
            torch.cuda.set_device(self.prev)
        return False


# --------------------------------------------------------------------------- #
# operator implementations (CUDA dispatch key)
# --------------------------------------------------------------------------- #
def _kv_dtype_code(src_dtype: torch.dtype, kv_cache_dtype: str) -> Tuple[int, int]:
    # DISPATCH_BY_KV_CACHE_DTYPE, csrc/custom_ops/quant_utils.cuh:532-567
    if kv_cache_dtype == "auto":
        kv = _native.KV_AUTO
    elif kv_cache_dtype in ("fp8", "fp8_e4m3"):
        kv = _native.KV_FP8_E4M3
    elif kv_cache_dtype == "fp8_e5m2":
        kv = _native.KV_FP8_E5M2
    else:
        raise RuntimeError(f"Unsupported data type of kv cache: {kv_cache_dtype}")
    if src_dtype not in _SRC_DTYPES:
        raise RuntimeError(f"Unsupported input type of kv cache: {src_dtype}")
    return _SRC_DTYPES[src_dtype], kv


_data_ptr = torch.Tensor.data_ptr


def _ptr_table(tensors: List[torch.Tensor]):
    return (ctypes.c_void_p * len(tensors))(*map(_data_ptr, tensors))


# sets of per-layer cache / scale tensors (by address) whose layers have been compared with layer 0 already
_validated_layer_sets: dict = {}


def _reshape_and_cache_flash_bulk_impl(
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
    _select: Optional[Tuple[Optional[torch.Tensor], torch.Tensor, torch.Tensor, torch.Tensor]] = None,
) -> None:
    """Host side of the bulk KV write; follows the reference's launcher
    (csrc/custom_ops/reshape_and_cache_flash_bulk.cu:77-144) up to the point
    where it would copy four pointer tables to the device: here the tables ride
    in the kernel arguments instead."""
    lib = _lib()
    num_layers = len(key_caches)
    if num_layers == 0:
        return
    _check(num_layers == len(value_caches), "Expected num_layers == value_caches.size() to be true")
    _check(num_layers == len(k_scales), "Expected num_layers == k_scales.size() to be true")
    _check(num_layers == len(v_scales), "Expected num_layers == v_scales.size() to be true")
    src_code, kv_code = _kv_dtype_code(keys.dtype, kv_cache_dtype)

    num_tokens = slot_mapping.size(0)
    block_size = key_caches[0].size(1)
    key_stride = keys.stride(0)
    value_stride = values.stride(0)
    block_stride = key_caches[0].stride(0)
    _check(block_stride == value_caches[0].stride(0),
           "Expected block_stride == value_caches[0].stride(0) to be true")
    if not (slot_mapping.dtype == torch.int64):
        raise RuntimeError(f"expected scalar type Long but found {slot_mapping.dtype}")
    # Not checked by the reference (it reinterprets the pointers); a mismatch
    # there corrupts memory, here it is an error.
    _check(values.dtype == keys.dtype, "reshape_and_cache_flash_bulk: keys and values dtype differ")
    _check(keys.stride(-1) == 1 and values.stride(-1) == 1,
           "reshape_and_cache_flash_bulk: last dimension of keys/values must be contiguous")
    _check(slot_mapping.dim() == 1 and (num_tokens <= 1 or slot_mapping.stride(0) == 1),
           "reshape_and_cache_flash_bulk: slot_mapping must be 1-D and contiguous")
    cache_elem = key_caches[0].element_size()
    want_elem = keys.element_size() if kv_code == _native.KV_AUTO else 1
    if not (cache_elem == want_elem and value_caches[0].element_size() == want_elem):
        raise RuntimeError(f"reshape_and_cache_flash_bulk: cache element size {cache_elem} does not match "
                           f"kv_cache_dtype '{kv_cache_dtype}' (expected {want_elem})")
    first = key_caches[0]
    _check(first.device == keys.device and values.device == keys.device and slot_mapping.device == keys.device,
           "reshape_and_cache_flash_bulk: all tensors must be on the same device")
    width = num_layers * int(num_heads) * int(head_size)
    if not (keys.dim() == 2 and values.dim() == 2 and keys.size(0) >= num_tokens and values.size(0) >= num_tokens
            and keys.size(1) >= width and values.size(1) >= width):
        raise RuntimeError(f"reshape_and_cache_flash_bulk: keys and values must be 2-D with at least {num_tokens} rows "
                           f"(one per slot) and {width} columns (layers x heads x head_size)")
    tables = (_ptr_table(key_caches), _ptr_table(value_caches), _ptr_table(k_scales), _ptr_table(v_scales))
    # Every layer's K and V view must look like layer 0's (the kernel takes one block stride, block size and number
    # of blocks for all of them), and the scales must be fp32 on the device.  Looking at 4 x num_layers tensors costs
    # more host time than the rest of the call, and a serving process passes the same tensors every step, so a set of
    # per-layer tensors, identified by its addresses, is looked at once; after that only layer 0 is compared with
    # what was seen then.
    seen_key = tuple(map(bytes, tables))
    geometry0 = (first.dtype, block_stride, first.size(0), block_size, first.device, kv_code)
    if _validated_layer_sets.get(seen_key) != geometry0:
        geometry = {(t.dtype, t.stride(0), t.size(0), t.size(1), t.device) for t in key_caches}
        geometry.update((t.dtype, t.stride(0), t.size(0), t.size(1), t.device) for t in value_caches)
        if not (len(geometry) == 1):
            raise RuntimeError("reshape_and_cache_flash_bulk: key and value caches of all layers must share dtype, "
                               "block stride, number of blocks, block size and device")
        if kv_code != _native.KV_AUTO:
            _check({s.dtype for s in k_scales} == {torch.float32} and {s.dtype for s in v_scales} == {torch.float32},
                   "reshape_and_cache_flash_bulk: k_scales / v_scales must be float32")
            _check({s.device for s in k_scales} | {s.device for s in v_scales} == {first.device},
                   "reshape_and_cache_flash_bulk: all tensors must be on the same device")
        if len(_validated_layer_sets) >= 64:
            _validated_layer_sets.clear()
        _validated_layer_sets[seen_key] = geometry0

    common = (keys.data_ptr(), values.data_ptr(), key_stride, value_stride, *tables,
              slot_mapping.data_ptr(), num_tokens, num_layers, int(num_heads), int(head_size),
              int(block_size), int(block_stride), int(first.size(0)), src_code, kv_code)
    with _on_device_of(keys):
        if _select is None:
            rc = lib.arctic_reshape_and_cache_flash_bulk(*common, _stream_of(keys))
        else:
            row_map, idx, k_out, v_out = _select
            rc = lib.arctic_reshape_and_cache_flash_bulk_select(
                *common, row_map.data_ptr() if row_map is not None else None, idx.data_ptr(), idx.element_size(),
                idx.numel(), keys.size(0),
                k_out.data_ptr(), v_out.data_ptr(), k_out.stride(0), v_out.stride(0), _stream_of(keys))
    _native.check(rc)


def _reshape_and_cache_flash_bulk_select_impl(
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
    logits_indices: torch.Tensor,
    k_out: torch.Tensor,
    v_out: torch.Tensor,
) -> None:
    """The bulk KV write and, in the same pass over keys / values, ``k_out[j] = keys[logits_indices[j]]`` and
    ``v_out[j] = values[logits_indices[j]]``: the two largest index_select calls of swiftkv_select
    (arctic_inference/vllm/swiftkv/llama_swiftkv.py:663-679) without a second read of k_states / v_states.
    The selected rows equal ``torch.index_select`` for every index in ``[0, keys.size(0))``, repeated ones
    included (SwiftKV's never repeat: one per request); a row whose index lies outside that range is left as it
    was, where index_select would raise."""
    fn = "reshape_and_cache_flash_bulk_select"
    num_layers = len(key_caches)
    n_sel = logits_indices.numel()
    if not (
            logits_indices.is_cuda and logits_indices.dim() == 1 and logits_indices.dtype in (torch.int32, torch.int64)
    ):
        raise RuntimeError(f"{fn}: logits_indices must be a 1-D int32 or int64 CUDA tensor")
    for name, src, out in (("k_out", keys, k_out), ("v_out", values, v_out)):
        if not (out.is_cuda and out.device == src.device and out.dtype == src.dtype):
            raise RuntimeError(f"{fn}: {name} must be on the device of keys / values and of their type")
        if not (out.dim() == 2 and out.size(0) >= n_sel):
            raise RuntimeError(f"{fn}: {name} must be 2-D with at least {n_sel} rows")
        if not (out.stride(1) == 1):
            raise RuntimeError(f"{fn}: rows of {name} must be contiguous")
    if num_layers == 0:
        return  # no layer, so no column to write or to select (reshape_and_cache_flash_bulk.cu:87-89)
    width = num_layers * int(num_heads) * int(head_size)
    if not (k_out.size(1) == width and v_out.size(1) == width and keys.size(1) >= width and values.size(1) >= width):
        raise RuntimeError(f"{fn}: k_out and v_out must have {width} columns (layers x heads x head_size)")
    if not (keys.size(0) == values.size(0)):
        raise RuntimeError(f"{fn}: keys and values differ in their number of rows")
    idx = logits_indices if logits_indices.is_contiguous() else logits_indices.contiguous()
    num_tokens = slot_mapping.size(0)
    if num_tokens == 0:
        # nothing is written to a cache, but the selected rows (of the first `width` columns) are still wanted
        if n_sel:
            _move_rows_impl("gather_rows", [keys[:, :width], values[:, :width]], idx, [k_out, v_out], False)
        return
    row_map = None
    if n_sel > _SELECT_SCAN_MAX_INDICES:
        # a long list: the inverse of logits_indices (which output row, if any, a token goes to) is built first;
        # up to that length every token's workgroup scans the list itself and nothing is allocated or launched here
        row_map = torch.empty(num_tokens, dtype=torch.int64, device=keys.device)
        with _on_device_of(keys):
            rc = _lib().arctic_build_row_map(row_map.data_ptr(), num_tokens, idx.data_ptr(), idx.element_size(), n_sel,
                                             _stream_of(keys))
        _native.check(rc)
    _reshape_and_cache_flash_bulk_impl(keys, values, key_caches, value_caches, slot_mapping, kv_cache_dtype, k_scales,
                                       v_scales, num_heads, head_size, _select=(row_map, idx, k_out, v_out))


def _reshape_and_cache_flash_fp4_impl(
    key: torch.Tensor,
    value: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
    kv_cache_dtype: str,
    k_scale: torch.Tensor,
    v_scale: torch.Tensor,
    key_scale_cache: torch.Tensor,
    value_scale_cache: torch.Tensor,
) -> None:
    """Host side of the NVFP4-style cache write; layout detection and checks follow the
    reference's launcher (csrc/custom_ops/reshape_and_cache_flash_fp4.cu:256-337).
    kv_cache_dtype, k_scale and v_scale are accepted and unused, as in the reference."""
    lib = _lib()
    _check(key.dtype in _HALF_DTYPES,
           "Unsupported input dtype for reshape_and_cache_fp4. Must be half or bfloat16.")
    _check(key.dim() == 3 and value.dim() == 3, "reshape_and_cache_flash_fp4: key/value must be [tokens, heads, head_size]")
    num_tokens = slot_mapping.size(0)
    num_heads, head_size = key.size(1), key.size(2)
    _check(key_cache.dim() == 4 and value_cache.dim() == 4, "KV cache must be rank-4")
    is_nhd = key_cache.size(2) == num_heads
    block_stride = key_cache.stride(0)
    page_stride = key_cache.stride(1) if is_nhd else key_cache.stride(2)
    head_stride = key_cache.stride(2) if is_nhd else key_cache.stride(1)
    block_size = key_cache.size(1) if is_nhd else key_cache.size(2)
    _check(value_cache.stride(0) == block_stride, "block_stride mismatch")
    _check((value_cache.stride(1) if is_nhd else value_cache.stride(2)) == page_stride, "page_stride mismatch")
    _check((value_cache.stride(2) if is_nhd else value_cache.stride(1)) == head_stride, "head_stride mismatch")
    _check((value_cache.size(1) if is_nhd else value_cache.size(2)) == block_size,
           "block_size mismatch between key_cache and value_cache")
    # assumed, not checked, by the reference (it would write out of bounds instead)
    _check(value.dtype == key.dtype and value.shape == key.shape, "reshape_and_cache_flash_fp4: key/value mismatch")
    _check(key.stride(2) == 1 and key.stride(1) == head_size and value.stride(2) == 1 and
           value.stride(1) == head_size, "reshape_and_cache_flash_fp4: heads of a token must be dense")
    if not (slot_mapping.dtype == torch.int64):
        raise RuntimeError(f"expected scalar type Long but found {slot_mapping.dtype}")
    _check(all(t.element_size() == 1 for t in (key_cache, value_cache, key_scale_cache, value_scale_cache)),
           "reshape_and_cache_flash_fp4: caches and scale caches must be byte tensors")
    _check(key_cache.size(3) * 2 == head_size and key_cache.stride(3) == 1,
           "reshape_and_cache_flash_fp4: cache last dim must be head_size / 2 packed bytes")
    _check(key_scale_cache.numel() * 8 >= key_cache.numel() and value_scale_cache.numel() * 8 >= value_cache.numel(),
           "reshape_and_cache_flash_fp4: scale cache too small (one byte per 16 elements)")
    with _on_device_of(key):
        rc = lib.arctic_reshape_and_cache_flash_fp4(
            key.data_ptr(), value.data_ptr(), key.stride(0), value.stride(0), key_cache.data_ptr(),
            value_cache.data_ptr(), key_scale_cache.data_ptr(), value_scale_cache.data_ptr(),
            slot_mapping.data_ptr(), num_tokens, num_heads, head_size, int(block_size), int(block_stride),
            int(page_stride), int(head_stride), int(key_cache.size(0)), _HALF_DTYPES[key.dtype], _stream_of(key))
    _native.check(rc)


_ACTIVATIONS = {"none": 0, "gelu": 1, "gelu_tanh": 2}


def _check_embedding(fn: str, emb_weight: torch.Tensor, token_ids: torch.Tensor, like: torch.Tensor, width: int,
                     rows: int) -> None:
    """An embedding table [V, width] in the activations' type and one int64 token id per row."""
    if not (
            emb_weight.is_cuda and token_ids.is_cuda and emb_weight.device == like.device
            and token_ids.device == like.device
    ):
        raise RuntimeError(f"{fn}: embedding table and token ids must be on the input's device")
    if not (emb_weight.dtype == like.dtype):
        raise RuntimeError(f"{fn}: embedding table dtype must match input dtype")
    if not (emb_weight.dim() == 2 and emb_weight.size(1) == width and emb_weight.stride(1) == 1):
        raise RuntimeError(f"{fn}: embedding table must be [num_embeddings, {width}] with contiguous rows")
    if not (emb_weight.size(0) > 0):
        raise RuntimeError(f"{fn}: the embedding table has no rows")
    if not (token_ids.dtype == torch.int64):
        raise RuntimeError(f"{fn}: token ids must be int64")
    if not (token_ids.numel() == rows and token_ids.is_contiguous()):
        raise RuntimeError(f"{fn}: one contiguous token id per row is needed ({token_ids.numel()} ids, {rows} rows)")


def _ln_common(fn: str, input: torch.Tensor, z: Optional[torch.Tensor], weight: Optional[torch.Tensor],
               bias: Optional[torch.Tensor], alpha: float, eps: float, activation: str,
               out_scale: float, token_ids: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Argument checks and launch shared by speculator_ln_cuda and speculator_add_ln_act_cuda
    (the checks are those of csrc/custom_ops/speculator_ln.cu:152-201)."""
    lib = _lib()
    if not (input.dtype in _HALF_DTYPES):
        raise RuntimeError(f"{fn}: only fp16 and bf16 are supported.")
    if not (input.is_cuda):
        raise RuntimeError(f"{fn}: input must be CUDA")
    dtype = input.dtype
    hidden = input.size(-1)
    if not (hidden > 0):
        raise RuntimeError(f"{fn}: hidden size must be > 0")
    if not (input.stride(-1) == 1):
        raise RuntimeError(f"{fn}: last dimension must be contiguous (stride -1 == 1)")
    if weight is not None:
        _check(weight.is_cuda, "weight must be CUDA")
        _check(weight.dtype == dtype, "weight dtype must match input dtype")
        _check(weight.dim() == 1 and weight.numel() == hidden, "weight must be 1D of size hidden")
        _check(weight.is_contiguous(), "weight must be contiguous")
    if bias is not None:
        _check(bias.is_cuda, "bias must be CUDA")
        _check(bias.dtype == dtype, "bias dtype must match input dtype")
        _check(bias.dim() == 1 and bias.numel() == hidden, "bias must be 1D of size hidden")
        _check(bias.is_contiguous(), "bias must be contiguous")
    if not (activation in _ACTIVATIONS):
        raise RuntimeError(f"{fn}: activation must be one of {sorted(_ACTIVATIONS)}")

    in_2d = _rows_of(input, hidden)
    rows = in_2d.size(0)
    row_stride = in_2d.stride(0)
    z_2d = None
    if token_ids is not None:
        _check_embedding(fn, z, token_ids, input, hidden, rows)
    elif z is not None:
        _check(z.is_cuda and z.device == input.device, "z must be CUDA, on the input's device")
        _check(z.dtype == dtype, "z dtype must match input dtype")
        _check(z.shape == input.shape, "z must have the input's shape")
        if not (z.stride(-1) == 1):
            raise RuntimeError(f"{fn}: last dimension of z must be contiguous")
        z_2d = _rows_of(z, hidden)
    out = torch.empty_like(input)
    out_2d = _rows_of(out, hidden)  # rows are written dense, `hidden` apart
    if rows == 0:
        return out
    if not (out_2d.stride(0) == hidden or rows == 1):
        raise RuntimeError(f"{fn}: internal - output rows must be dense")
    w_ptr = weight.data_ptr() if weight is not None else None
    b_ptr = bias.data_ptr() if bias is not None else None
    with _on_device_of(input):
        if token_ids is not None:
            rc = lib.arctic_speculator_embed_add_ln_act(
                out_2d.data_ptr(), in_2d.data_ptr(), z.data_ptr(), token_ids.data_ptr(), w_ptr, b_ptr, rows, hidden,
                row_stride, z.stride(0), z.size(0), float(alpha), float(eps), _ACTIVATIONS[activation],
                float(out_scale), _HALF_DTYPES[dtype], _stream_of(input))
        elif z is None and activation == "none" and out_scale == 1.0:
            rc = lib.arctic_speculator_ln(out_2d.data_ptr(), in_2d.data_ptr(), w_ptr, b_ptr, rows, hidden,
                                          row_stride, float(eps), _HALF_DTYPES[dtype], _stream_of(input))
        else:
            rc = lib.arctic_speculator_add_ln_act(
                out_2d.data_ptr(), in_2d.data_ptr(), z_2d.data_ptr() if z_2d is not None else None, w_ptr, b_ptr,
                rows, hidden, row_stride, z_2d.stride(0) if z_2d is not None else 0, float(alpha), float(eps),
                _ACTIVATIONS[activation], float(out_scale), _HALF_DTYPES[dtype], _stream_of(input))
    _native.check(rc)
    return out


def _speculator_ln_impl(input: torch.Tensor, weight: Optional[torch.Tensor],
                        bias: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """Host side of speculator_ln_cuda (csrc/custom_ops/speculator_ln.cu:152-252)."""
    return _ln_common("speculator_ln", input, None, weight, bias, 0.0, eps, "none", 1.0)


def _speculator_add_ln_act_impl(input: torch.Tensor, z: Optional[torch.Tensor], weight: Optional[torch.Tensor],
                                bias: Optional[torch.Tensor], alpha: float, eps: float, activation: str,
                                out_scale: float) -> torch.Tensor:
    """The norm with the speculator's element-wise steps around it in one launch
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:296-307, 733-734, 809-816)."""
    return _ln_common("speculator_add_ln_act", input, z, weight, bias, alpha, eps, activation, out_scale)


def _speculator_embed_add_ln_act_impl(input: torch.Tensor, emb_weight: torch.Tensor, token_ids: torch.Tensor,
                                      weight: Optional[torch.Tensor], bias: Optional[torch.Tensor], alpha: float,
                                      eps: float, activation: str, out_scale: float) -> torch.Tensor:
    """speculator_add_ln_act with z = emb_weight[clamp(token_ids)] looked up inside the launch
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:301-309, 845, 862)."""
    return _ln_common("speculator_embed_add_ln_act", input, emb_weight, weight, bias, alpha, eps, activation,
                      out_scale, token_ids=token_ids)


def _sum_lstm_impl(
    states_4d: torch.Tensor,
    z4_4d: torch.Tensor,
    prev_cell_d: torch.Tensor,
    w_cell: Optional[torch.Tensor],
    b_cell: Optional[torch.Tensor],
    w_state: Optional[torch.Tensor],
    b_state: Optional[torch.Tensor],
    alpha: float,
    eps_cell: float,
    eps_state: float,
    use_fast_gelu: bool,
    _shared_z: bool = False,
    _token_ids: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Host side of sum_lstm_cuda (csrc/custom_ops/sum_lstm.cu:293-473).  With _shared_z the
    second argument is the un-repeated [..., D] embedding row (see sum_lstm_shared_z)."""
    lib = _lib()
    dtype = states_4d.dtype
    _check(dtype in _HALF_DTYPES, "sum_lstm: only fp16 and bf16 are supported.")
    zero_cell = prev_cell_d is None     # not in the reference's schema: the cell of zeros a proposal round starts from
    _check(states_4d.is_cuda and z4_4d.is_cuda and (zero_cell or prev_cell_d.is_cuda),
           "sum_lstm: inputs must be CUDA tensors")
    _check(z4_4d.dtype == dtype and (zero_cell or prev_cell_d.dtype == dtype),
           "sum_lstm: all input dtypes must match")
    hidden4 = states_4d.size(-1)
    _check(hidden4 > 0 and hidden4 % 4 == 0, "sum_lstm: last dim of states must be 4*D_gate")
    d_gate = hidden4 // 4
    if _shared_z:
        _check(z4_4d.size(-1) == d_gate, "sum_lstm_shared_z: z must have last dim D_gate")
    else:
        _check(z4_4d.size(-1) == hidden4, "sum_lstm: z4 must have last dim 4*D_gate")
    d_cell = d_gate if zero_cell else prev_cell_d.size(-1)
    if not (d_cell == d_gate):
        raise RuntimeError(f"sum_lstm: prev_cell last dim must equal D_gate. Got {d_cell} vs expected {d_gate}.")
    _check(states_4d.stride(-1) == 1 and z4_4d.stride(-1) == 1 and (zero_cell or prev_cell_d.stride(-1) == 1),
           "sum_lstm: last dimension must be contiguous (stride -1 == 1)")
    for t, name in ((w_cell, "w_cell"), (b_cell, "b_cell"), (w_state, "w_state"), (b_state, "b_state")):
        if t is not None:
            if not (t.is_cuda):
                raise RuntimeError(f"sum_lstm: {name} must be CUDA")
            if not (t.dtype == dtype):
                raise RuntimeError(f"sum_lstm: {name} dtype mismatch")
            if not (t.numel() >= d_gate):
                raise RuntimeError(f"sum_lstm: {name} must have length >= D_eff")
            if not (t.is_contiguous()):
                raise RuntimeError(f"sum_lstm: {name} must be contiguous")

    s2 = _rows_of(states_4d, hidden4)
    z2 = _rows_of(z4_4d, d_gate if _shared_z else hidden4)
    rows = s2.size(0)
    p2 = None if zero_cell else _rows_of(prev_cell_d, d_cell)
    if _token_ids is not None:
        _check(zero_cell or p2.size(0) == rows, "sum_lstm: row counts of the inputs differ")
        _check_embedding("sum_lstm_embedded", z4_4d, _token_ids, states_4d, d_gate, rows)
    else:
        _check(z2.size(0) == rows and (zero_cell or p2.size(0) == rows), "sum_lstm: row counts of the inputs differ")
    if zero_cell:
        # dense outputs shaped like states_4d with its last dimension cut to D_gate
        out_cell = torch.empty((rows, d_gate), dtype=dtype, device=states_4d.device)
        out_state = torch.empty((rows, d_gate), dtype=dtype, device=states_4d.device)
        flat = states_4d.dim() == 2
        shape = states_4d.shape[:-1] + (d_gate,)
        out_cell_orig = out_cell if flat else out_cell.view(shape)
        out_state_orig = out_state if flat else out_state.view(shape)
    else:
        # outputs inherit prev_cell's row pitch (reference :356-365)
        out_cell = torch.empty_strided(p2.size(), p2.stride(), dtype=dtype, device=p2.device)
        out_state = torch.empty_strided(p2.size(), p2.stride(), dtype=dtype, device=p2.device)
        _check(out_cell.stride(0) == out_state.stride(0), "sum_lstm: internal - output strides mismatch")
        flat = prev_cell_d.dim() == 2
        out_cell_orig = out_cell if flat else out_cell.view(prev_cell_d.size())
        out_state_orig = out_state if flat else out_state.view(prev_cell_d.size())
    if rows == 0:
        return out_state_orig, out_cell_orig

    def ptr(t):
        return t.data_ptr() if t is not None else None

    pc_stride = 0 if zero_cell else p2.stride(0)
    entry = lib.arctic_sum_lstm_shared_z if _shared_z else lib.arctic_sum_lstm
    with _on_device_of(states_4d):
        if _token_ids is not None:
            rc = lib.arctic_sum_lstm_embedded(
                out_state.data_ptr(), out_cell.data_ptr(), s2.data_ptr(), z4_4d.data_ptr(), _token_ids.data_ptr(),
                ptr(p2), ptr(w_cell), ptr(b_cell), ptr(w_state), ptr(b_state),
                rows, d_gate, s2.stride(0), z4_4d.stride(0), pc_stride, out_cell.stride(0), z4_4d.size(0),
                float(alpha), float(eps_cell), float(eps_state), int(bool(use_fast_gelu)),
                _HALF_DTYPES[dtype], _stream_of(states_4d))
        else:
            rc = entry(
                out_state.data_ptr(), out_cell.data_ptr(), s2.data_ptr(), z2.data_ptr(), ptr(p2),
                ptr(w_cell), ptr(b_cell), ptr(w_state), ptr(b_state),
                rows, d_gate, s2.stride(0), z2.stride(0), pc_stride, out_cell.stride(0),
                float(alpha), float(eps_cell), float(eps_state), int(bool(use_fast_gelu)),
                _HALF_DTYPES[dtype], _stream_of(states_4d))
    _native.check(rc)
    return out_state_orig, out_cell_orig


def _sum_lstm_zero_cell_impl(states_4d, z4_4d, w_cell, b_cell, w_state, b_state, alpha, eps_cell, eps_state,
                             use_fast_gelu):
    """sum_lstm with the cell of zeros every proposal round starts from
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:899-903) implied instead of passed."""
    return _sum_lstm_impl(states_4d, z4_4d, None, w_cell, b_cell, w_state, b_state, alpha, eps_cell, eps_state,
                          use_fast_gelu)


def _sum_lstm_shared_z_impl(states_4d, z_d, prev_cell_d, w_cell, b_cell, w_state, b_state, alpha, eps_cell,
                            eps_state, use_fast_gelu):
    return _sum_lstm_impl(states_4d, z_d, prev_cell_d, w_cell, b_cell, w_state, b_state, alpha, eps_cell,
                          eps_state, use_fast_gelu, _shared_z=True)


def _sum_lstm_embedded_impl(states_4d, emb_weight, token_ids, prev_cell_d, w_cell, b_cell, w_state, b_state, alpha,
                            eps_cell, eps_state, use_fast_gelu):
    """sum_lstm_shared_z with z = emb_weight[clamp(token_ids)] looked up inside the launch
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:744, 845, 862)."""
    return _sum_lstm_impl(states_4d, emb_weight, prev_cell_d, w_cell, b_cell, w_state, b_state, alpha, eps_cell,
                          eps_state, use_fast_gelu, _shared_z=True, _token_ids=token_ids)


def _move_rows_impl(fn: str, sources: List[torch.Tensor], indices: torch.Tensor, outs: List[torch.Tensor],
                    scatter: bool) -> None:
    lib = _lib()
    if not (len(sources) == len(outs)):
        raise RuntimeError(f"{fn}: {len(sources)} sources but {len(outs)} outputs")
    if not (indices.is_cuda and indices.dim() == 1 and indices.is_contiguous()):
        raise RuntimeError(f"{fn}: indices must be a contiguous 1-D CUDA tensor")
    if not (indices.dtype in (torch.int32, torch.int64)):
        raise RuntimeError(f"{fn}: indices must be int32 or int64")
    n = indices.numel()
    if n == 0 or not sources:
        return
    indexed_rows = None
    row_bytes, src_stride, dst_stride = [], [], []
    for k, (src, dst) in enumerate(zip(sources, outs)):
        if not (src.is_cuda and dst.is_cuda and src.device == indices.device and dst.device == indices.device):
            raise RuntimeError(f"{fn}: tensor {k}: sources, outputs and indices must be on one CUDA device")
        if not (src.dtype == dst.dtype):
            raise RuntimeError(f"{fn}: tensor {k}: source and output dtypes differ")
        if not (src.dim() >= 1 and src.shape[1:] == dst.shape[1:]):
            raise RuntimeError(f"{fn}: tensor {k}: row shapes differ")
        if not (src.size(0) == 0 or src[0].is_contiguous()):
            raise RuntimeError(f"{fn}: tensor {k}: source rows must be contiguous")
        if not (dst.size(0) == 0 or dst[0].is_contiguous()):
            raise RuntimeError(f"{fn}: tensor {k}: output rows must be contiguous")
        indexed, linear = (dst, src) if scatter else (src, dst)
        if not (linear.size(0) >= n):
            raise RuntimeError(f"{fn}: tensor {k}: {n} indices but only {linear.size(0)} rows")
        if not (indexed_rows in (None, indexed.size(0))):
            raise RuntimeError(f"{fn}: indexed tensors differ in their number of rows")
        indexed_rows = indexed.size(0)
        es = src.element_size()
        row = 1
        for d in src.shape[1:]:
            row *= d
        row_bytes.append(row * es)
        src_stride.append(src.stride(0) * es)
        dst_stride.append(dst.stride(0) * es)
    i64s = lambda v: (ctypes.c_int64 * len(v))(*v)
    with _on_device_of(indices):
        rc = lib.arctic_gather_rows(len(sources), _ptr_table(sources), _ptr_table(outs), i64s(row_bytes),
                                    i64s(src_stride), i64s(dst_stride), indices.data_ptr(), indices.element_size(),
                                    n, indexed_rows, 1 if scatter else 0, _stream_of(indices))
    _native.check(rc)


def _gather_rows_impl(sources: List[torch.Tensor], indices: torch.Tensor, outs: List[torch.Tensor]) -> None:
    """outs[k][r] = sources[k][indices[r]]: the index_select calls of swiftkv_select
    (arctic_inference/vllm/swiftkv/llama_swiftkv.py:663-679) in one launch."""
    _move_rows_impl("gather_rows", sources, indices, outs, False)


def _scatter_rows_impl(sources: List[torch.Tensor], indices: torch.Tensor, outs: List[torch.Tensor]) -> None:
    """outs[k][indices[r]] = sources[k][r]: `orig_hidden_states[logits_indices] = hidden_states[:batch_size]`
    (arctic_inference/vllm/swiftkv/llama_swiftkv.py:733-742)."""
    _move_rows_impl("scatter_rows", sources, indices, outs, True)


def _speculator_argmax_impl(logits: torch.Tensor, max_index: int) -> torch.Tensor:
    """``torch.argmax(logits, dim=-1).clamp_(0, max_index)`` in one launch
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:846-848, 862)."""
    lib = _lib()
    _check(logits.is_cuda, "speculator_argmax: logits must be CUDA")
    _check(logits.dtype in _SRC_DTYPES, "speculator_argmax: logits must be fp32, fp16 or bf16")
    _check(logits.dim() >= 1 and logits.size(-1) > 0, "speculator_argmax: logits need a non-empty last dimension")
    _check(logits.stride(-1) == 1, "speculator_argmax: last dimension must be contiguous")
    _check(max_index >= 0, "speculator_argmax: max_index must not be negative")
    cols = logits.size(-1)
    in_2d = _rows_of(logits, cols)
    rows = in_2d.size(0)
    out = torch.empty(logits.shape[:-1], dtype=torch.int64, device=logits.device)
    if rows == 0:
        return out
    with _on_device_of(logits):
        rc = lib.arctic_argmax_clamp(out.data_ptr(), in_2d.data_ptr(), rows, cols, in_2d.stride(0), int(max_index),
                                     _SRC_DTYPES[logits.dtype], _stream_of(logits))
    _native.check(rc)
    return out


_IMPLS = {
    "speculator_argmax_cuda": _speculator_argmax_impl,
    "gather_rows": _gather_rows_impl,
    "scatter_rows": _scatter_rows_impl,
    "sum_lstm_shared_z_cuda": _sum_lstm_shared_z_impl,
    "sum_lstm_embedded_cuda": _sum_lstm_embedded_impl,
    "speculator_add_ln_act_cuda": _speculator_add_ln_act_impl,
    "speculator_embed_add_ln_act_cuda": _speculator_embed_add_ln_act_impl,
    "reshape_and_cache_flash_bulk": _reshape_and_cache_flash_bulk_impl,
    "reshape_and_cache_flash_bulk_select": _reshape_and_cache_flash_bulk_select_impl,
    "reshape_and_cache_flash_fp4": _reshape_and_cache_flash_fp4_impl,
    "speculator_ln_cuda": _speculator_ln_impl,
    "sum_lstm_cuda": _sum_lstm_impl,
    "sum_lstm_zero_cell_cuda": _sum_lstm_zero_cell_impl,
}


# Shape-only implementations for meta tensors (tracing under torch.compile): the same output shapes,
# strides and dtypes as the launches above, no data.  The reference binds the CUDA key only
# (torch_bindings.cpp:17,32,37,50), so its operators cannot be traced; these change nothing for real tensors.
def _meta_like_input(input, *args):
    return torch.empty_like(input)


def _meta_sum_lstm_embedded(states_4d, emb_weight, token_ids, prev_cell_d, *args):
    return _meta_sum_lstm(states_4d, emb_weight, prev_cell_d)


def _meta_sum_lstm_zero_cell(states_4d, z4_4d, *args):
    return _meta_sum_lstm(states_4d, z4_4d, None)


def _meta_sum_lstm(states_4d, z, prev_cell_d, *args):
    if prev_cell_d is None:
        shape = states_4d.shape[:-1] + (states_4d.size(-1) // 4,)
        return (torch.empty(shape, dtype=states_4d.dtype, device=states_4d.device),
                torch.empty(shape, dtype=states_4d.dtype, device=states_4d.device))
    p2 = prev_cell_d.view(-1, prev_cell_d.size(-1))
    make = lambda: torch.empty_strided(p2.size(), p2.stride(), dtype=p2.dtype, device=p2.device).view(prev_cell_d.size())
    return make(), make()


def _meta_argmax(logits, max_index):
    return torch.empty(logits.shape[:-1], dtype=torch.int64, device=logits.device)


def _meta_nothing(*args):
    return None


_META_IMPLS = {
    "speculator_ln_cuda": _meta_like_input,
    "sum_lstm_zero_cell_cuda": _meta_sum_lstm_zero_cell,
    "speculator_add_ln_act_cuda": _meta_like_input,
    "sum_lstm_cuda": _meta_sum_lstm,
    "sum_lstm_shared_z_cuda": _meta_sum_lstm,
    "sum_lstm_embedded_cuda": _meta_sum_lstm_embedded,
    "speculator_embed_add_ln_act_cuda": _meta_like_input,
    "speculator_argmax_cuda": _meta_argmax,
    "reshape_and_cache_flash_bulk": _meta_nothing,
    "reshape_and_cache_flash_bulk_select": _meta_nothing,
    "reshape_and_cache_flash_fp4": _meta_nothing,
    "gather_rows": _meta_nothing,
    "scatter_rows": _meta_nothing,
}


def _register_ops() -> None:
    """Define the four schemas and bind the CUDA key (the only key the reference
    binds, torch_bindings.cpp:17,32,37,50)."""
    global _torch_lib, _registered
    if _registered:
        return
    lib = torch.library.Library(_NAMESPACE, "DEF")
    for name, schema in {**_SCHEMAS, **_EXTRA_SCHEMAS}.items():
        lib.define(schema)
        lib.impl(name, _IMPLS[name], "CUDA")
        lib.impl(name, _META_IMPLS[name], "Meta")
    _torch_lib = lib  # keep alive: dropping the Library object unregisters the ops
    _registered = True


# --------------------------------------------------------------------------- #
# public surface (names and meaning as in arctic_inference/py_custom_ops.py)
# --------------------------------------------------------------------------- #
def try_load_torch_library() -> bool:
    """Load ``libarctic_mi355x*.so`` from the package directory and register the
    ``torch.ops.arctic_inference`` operators.  True iff the operators are usable
    (reference: arctic_inference/py_custom_ops.py:9-37)."""
    path = _native.library_path()
    if path is None:
        logger.info("Could not find compiled %s library in package.", _native.LIB_BASENAME)
        return False
    try:
        _native.load()
        _register_ops()
        logger.info("Successfully loaded custom ops from %s.", path)
        return True
    except Exception as e:  # missing ROCm runtime, ABI mismatch, duplicate registration ...
        logger.info("Unable to load custom library from %s. %s: %s.", path, type(e).__name__, e)
        return False


def try_load_jit_library() -> bool:
    """Build the library with hipcc on the spot, then load it.  Counterpart of the
    reference's JIT route (arctic_inference/py_custom_ops.py:40-56)."""
    try:
        _native.build(force=False)
    except Exception as e:
        logger.info("Unable to build %s. %s: %s.", _native.LIB_BASENAME, type(e).__name__, e)
        return False
    return try_load_torch_library()


def _ops():
    if not _registered:
        raise RuntimeError(
            "arctic_inference custom ops are not loaded: call try_load_torch_library() "
            "and check that it returned True (libarctic_mi355x.so must be built)")
    return torch.ops.arctic_inference


_is_compiling = getattr(getattr(torch, "compiler", None), "is_compiling", lambda: False)


def _call(name: str, *args):
    """``torch.ops.arctic_inference.<name>(*args)``.  The operators are implemented in Python on top of
    the C ABI, so outside ``torch.compile`` the implementation is called directly: the round trip through
    the dispatcher (boxing four lists of per-layer tensors and unboxing them again) is a third of the host
    time of a 40-layer bulk write.  Under ``torch.compile`` the registered operator is used, so that the
    call stays one opaque node of the traced graph."""
    ops = _ops()
    first = args[0][0] if isinstance(args[0], (list, tuple)) and args[0] else args[0]
    if _is_compiling() or not (isinstance(first, torch.Tensor) and first.is_cuda):
        return getattr(ops, name)(*args)   # also the path on which non-GPU tensors are turned away
    return _IMPLS[name](*args)


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
    _call("reshape_and_cache_flash_bulk", keys, values, key_caches, value_caches, slot_mapping,
                                        kv_cache_dtype, k_scales, v_scales, num_heads, head_size)


def reshape_and_cache_flash_bulk_select(
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
    logits_indices: torch.Tensor,
    k_out: torch.Tensor,
    v_out: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``reshape_and_cache_flash_bulk(...)`` followed by ``torch.index_select(keys, 0, logits_indices,
    out=k_out[:n])`` and the same for values (arctic_inference/vllm/swiftkv/llama_swiftkv.py:617-622, 663-679),
    with keys / values read once for both.  Returns ``(k_out[:n], v_out[:n])``.  Indices may repeat; a row whose
    index lies outside ``[0, keys.size(0))`` is left as it was (index_select would raise).  With no layers there is
    no column to select and the call does nothing."""
    _call("reshape_and_cache_flash_bulk_select", keys, values, key_caches, value_caches, slot_mapping, kv_cache_dtype,
          k_scales, v_scales, num_heads, head_size, logits_indices, k_out, v_out)
    n = logits_indices.numel()
    return k_out[:n], v_out[:n]


def reshape_and_cache_flash_fp4(
    keys: torch.Tensor,
    values: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    key_cache_scales: torch.Tensor,
    value_cache_scales: torch.Tensor,
    slot_mapping: torch.Tensor,
    kv_cache_dtype: str,
    k_scale: torch.Tensor,
    v_scale: torch.Tensor,
) -> None:
    _call("reshape_and_cache_flash_fp4", keys, values, key_cache, value_cache, slot_mapping,
                                       kv_cache_dtype, k_scale, v_scale, key_cache_scales,
                                       value_cache_scales)


def speculator_ln(
    input: torch.Tensor,
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    eps: float,
) -> torch.Tensor:
    return _call("speculator_ln_cuda", input, weight, bias, eps)


def sum_lstm(
    states_4d: torch.Tensor,
    z4_4d: torch.Tensor,
    prev_cell_d: Optional[torch.Tensor],
    w_cell: Optional[torch.Tensor],
    b_cell: Optional[torch.Tensor],
    w_state: Optional[torch.Tensor],
    b_state: Optional[torch.Tensor],
    alpha: float,
    eps_cell: float,
    eps_state: float,
    use_fast_gelu: bool,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """The reference's wrapper (arctic_inference/py_custom_ops.py:101-117).  Beyond it, ``prev_cell_d=None``
    stands for the cell of zeros a proposal round starts from (arctic_speculator.py:899-903): same result as
    a zero tensor bit for bit, but no tensor is made, cleared or read; the outputs are then dense and shaped
    like ``states_4d`` with its last dimension divided by four.  ``sum_lstm_shared_z`` and
    ``sum_lstm_embedded`` take None the same way."""
    if prev_cell_d is None:
        return _call("sum_lstm_zero_cell_cuda", states_4d, z4_4d, w_cell, b_cell, w_state, b_state, alpha, eps_cell,
                     eps_state, use_fast_gelu)
    return _call("sum_lstm_cuda", states_4d, z4_4d, prev_cell_d, w_cell, b_cell, w_state, b_state,
                                alpha, eps_cell, eps_state, use_fast_gelu)


def sum_lstm_shared_z(
    states_4d: torch.Tensor,
    z_d: torch.Tensor,
    prev_cell_d: Optional[torch.Tensor],
    w_cell: Optional[torch.Tensor],
    b_cell: Optional[torch.Tensor],
    w_state: Optional[torch.Tensor],
    b_state: Optional[torch.Tensor],
    alpha: float,
    eps_cell: float,
    eps_state: float,
    use_fast_gelu: bool,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``sum_lstm(states_4d, z_d.repeat(..., 4), ...)`` without building the repeated tensor:
    the speculator's ``z4 = forget_emb(tokens).repeat(1, 1, 4)``
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:744) folded into the operator.
    Bit-identical to the two-step form; reads 6*D fewer bytes per row."""
    return _call("sum_lstm_shared_z_cuda", states_4d, z_d, prev_cell_d, w_cell, b_cell, w_state, b_state,
                                         alpha, eps_cell, eps_state, use_fast_gelu)


def sum_lstm_embedded(
    states_4d: torch.Tensor,
    emb_weight: torch.Tensor,
    token_ids: torch.Tensor,
    prev_cell_d: Optional[torch.Tensor],
    w_cell: Optional[torch.Tensor],
    b_cell: Optional[torch.Tensor],
    w_state: Optional[torch.Tensor],
    b_state: Optional[torch.Tensor],
    alpha: float,
    eps_cell: float,
    eps_state: float,
    use_fast_gelu: bool,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """``sum_lstm_shared_z(states_4d, emb_weight[token_ids.clamp(0, V - 1)], ...)`` without the lookup as a
    launch of its own: the speculator's ``forget_emb[i](last_tokens)`` with the clamp of ``last_tokens``
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:744, 845, 862) folded into the operator.
    Bit-identical to the two-step form."""
    return _call("sum_lstm_embedded_cuda", states_4d, emb_weight, token_ids, prev_cell_d, w_cell, b_cell, w_state,
                 b_state, alpha, eps_cell, eps_state, use_fast_gelu)


def speculator_embed_add_ln_gelu(
    states: torch.Tensor,
    emb_weight: torch.Tensor,
    token_ids: torch.Tensor,
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    alpha: float,
    eps: float,
) -> torch.Tensor:
    """``speculator_add_ln_gelu(states, emb_weight[token_ids.clamp(0, V - 1)], ...)`` in one launch: the MLP
    speculator's ``z = emb[i](last_tokens); states.add_(z, alpha=...); activation(ln(states))``
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:301-309).  ``states`` is left unchanged."""
    return _call("speculator_embed_add_ln_act_cuda", states, emb_weight, token_ids, weight, bias, alpha, eps, "gelu",
                 1.0)


def speculator_add_ln_gelu(
    states: torch.Tensor,
    z: torch.Tensor,
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    alpha: float,
    eps: float,
) -> torch.Tensor:
    """``gelu(ln(states + alpha * z))`` in one launch: the MLP / sum_rnn speculator's
    ``states.add_(z, alpha=emb_weight / state_weight); activation(ln(states))``
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:300-307, 809-816), rounded after each
    step like the three separate ops.  ``states`` is left unchanged."""
    return _call("speculator_add_ln_act_cuda", states, z, weight, bias, alpha, eps, "gelu", 1.0)


def speculator_ln_scaled(
    input: torch.Tensor,
    weight: Optional[torch.Tensor],
    bias: Optional[torch.Tensor],
    eps: float,
    out_scale: float,
) -> torch.Tensor:
    """``speculator_ln(input, weight, bias, eps) * out_scale`` in one launch: the speculator's
    ``ln0(previous_hidden_states) / SQRT2`` with ``out_scale = 1 / SQRT2``
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:296-297, 733-734)."""
    return _call("speculator_add_ln_act_cuda", input, None, weight, bias, 0.0, eps, "none", out_scale)


def gather_rows(sources: List[torch.Tensor], indices: torch.Tensor,
                outs: Optional[List[Optional[torch.Tensor]]] = None) -> List[torch.Tensor]:
    """``torch.index_select(sources[k], 0, indices, out=outs[k][:indices.numel()])`` for every k in one
    launch: the five ``index_fn`` calls of ``swiftkv_select``
    (arctic_inference/vllm/swiftkv/llama_swiftkv.py:663-679).  A missing output is allocated, like
    ``tensor.index_select(0, indices)``.  Returns the outputs (whole buffers, as passed)."""
    n = indices.numel()
    outs = list(outs) if outs is not None else [None] * len(sources)
    for k, src in enumerate(sources):
        if outs[k] is None:
            outs[k] = torch.empty((n,) + tuple(src.shape[1:]), dtype=src.dtype, device=src.device)
    _call("gather_rows", list(sources), indices, outs)
    return outs


def scatter_rows(sources: List[torch.Tensor], indices: torch.Tensor, outs: List[torch.Tensor]) -> None:
    """``outs[k][indices] = sources[k][:indices.numel()]`` for every k in one launch: the write-back
    ``orig_hidden_states[logits_indices] = hidden_states[:batch_size]``
    (arctic_inference/vllm/swiftkv/llama_swiftkv.py:733-742)."""
    _call("scatter_rows", list(sources), indices, list(outs))


def speculator_argmax(logits: torch.Tensor, vocab_size: int) -> torch.Tensor:
    """``torch.argmax(logits, dim=-1)`` followed by ``.clamp_(0, vocab_size - 1)`` in one launch: the token
    selection at the end of a speculator step (arctic_inference/vllm/spec_dec/arctic_speculator.py:846-848,
    862).  Same winner as torch: lowest index among equal values, a NaN beats every number."""
    return _call("speculator_argmax_cuda", logits, int(vocab_size) - 1)
