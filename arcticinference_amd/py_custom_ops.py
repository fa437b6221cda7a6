"""Drop-in ``torch.ops.arctic_inference.*`` surface backed by gfx950 HIP kernels.

Mirrors the operator boundary of the reference
(``arctic_inference/py_custom_ops.py:9-118`` and the schemas in
``csrc/custom_ops/torch_bindings.cpp:6-51``): same namespace, same schema
strings, same wrapper names and argument meaning, the same argument checks with
the same message prefixes.  The reference registers compiled C++ functions from
a torch extension; here the schemas are defined from Python and the ``CUDA``
dispatch key (HIP tensors under PyTorch-ROCm) is bound to the functions of the
extension module ``_host_ext``: the host side in C++, which unwraps tensors
into pointers, sizes and strides and calls the C ABI of ``libarctic_mi355x.so``
on the current stream.

There is no fallback: without the two shared objects ``try_load_torch_library()``
returns ``False`` (as the reference does) and every operator raises.
"""
from __future__ import annotations

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

_torch_lib: Optional[torch.library.Library] = None
_registered = False
# operator name -> its host-side implementation (the functions of the _host_ext extension module)
_IMPLS: dict = {}


def _load_host_layer() -> None:
    """Import ``arcticinference_amd._host_ext`` (built from csrc/torch_forwards.cpp + csrc/host_ext.cpp): the
    operators' host side in C++ - the reference's argument checks with its messages, outputs allocated the way
    its launchers allocate them, pointers, sizes and strides handed to the C ABI on torch's current stream.
    The reference's host side is C++ as well (csrc/custom_ops/*.cu, the launcher below each kernel)."""
    if _IMPLS:
        return
    from . import _host_ext
    for name in {**_SCHEMAS, **_EXTRA_SCHEMAS}:
        _IMPLS[name] = getattr(_host_ext, name)


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
    _load_host_layer()
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
    """Load ``libarctic_mi355x*.so`` and the host layer ``_host_ext*.so`` from the package directory and
    register the ``torch.ops.arctic_inference`` operators.  True iff the operators are usable
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
    """``torch.ops.arctic_inference.<name>(*args)``.  Outside ``torch.compile`` the host-layer function is
    called directly for GPU tensors: the round trip through the dispatcher (boxing four lists of per-layer
    tensors and handing them back to Python) costs more host time than the whole call.  Under
    ``torch.compile`` the registered operator is used, so that the call stays one opaque node of the
    traced graph."""
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


def prepare_bulk_kv_layers(key_caches: List[torch.Tensor], value_caches: List[torch.Tensor],
                           k_scales: List[torch.Tensor], v_scales: List[torch.Tensor]):
    """The per-layer arguments of ``reshape_and_cache_flash_bulk``, checked once and held, for a caller that writes
    the same layers on every step.  The reference's caller rebuilds its four lists - two views of every layer's cache
    tensor and two attribute reads - on every engine step (arctic_inference/vllm/swiftkv/llama_swiftkv.py:594-615),
    which costs it several times the host time of the write itself; with the object returned here a step is
    ``layers.write(k_states, v_states, slot_mapping, kv_cache_dtype, num_heads, head_size)`` (or ``write_select`` with
    ``logits_indices, k_out, v_out`` behind), same checks of the per-call arguments, same launch.  The object keeps an
    alias of every tensor, so what it checked stays allocated and keeps its geometry; scales updated in place are seen.
    Make a new one whenever a cache or scale tensor is REPLACED (a pool rebuilt after sleep / wake, a scale
    re-assigned): it cannot notice that.  Not in the reference; not a registered operator (eager callers only)."""
    _ops()
    from . import _host_ext
    return _host_ext.BulkKVLayers(key_caches, value_caches, k_scales, v_scales)


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
