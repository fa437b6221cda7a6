"""Host side of the drop-in operator surface (runs without a GPU)."""
import re

import pytest
import torch

from arcticinference_amd import _native, py_custom_ops as ops

# The schemas the reference registers (csrc/custom_ops/torch_bindings.cpp:7-49), whitespace-normalised.
REFERENCE_SCHEMAS = {
    "reshape_and_cache_flash_bulk":
        "arctic_inference::reshape_and_cache_flash_bulk(Tensor keys, Tensor values, Tensor(c!)[] key_caches, "
        "Tensor(d!)[] value_caches, Tensor slot_mapping, str kv_cache_dtype, Tensor(e)[] k_scales, "
        "Tensor(f)[] v_scales, int num_heads, int head_size) -> ()",
    "reshape_and_cache_flash_fp4":
        "arctic_inference::reshape_and_cache_flash_fp4(Tensor key, Tensor value, Tensor(c!) key_cache, "
        "Tensor(d!) value_cache, Tensor slot_mapping, str kv_cache_dtype, Tensor k_scale, Tensor v_scale, "
        "Tensor(e!) key_scale_cache, Tensor(f!) value_scale_cache) -> ()",
    "speculator_ln_cuda":
        "arctic_inference::speculator_ln_cuda(Tensor input, Tensor? weight, Tensor? bias, float eps) -> Tensor",
    "sum_lstm_cuda":
        "arctic_inference::sum_lstm_cuda(Tensor states_4d, Tensor z4_4d, Tensor prev_cell_d, Tensor? w_cell, "
        "Tensor? b_cell, Tensor? w_state, Tensor? b_state, float alpha, float eps_cell, float eps_state, "
        "bool use_fast_gelu) -> (Tensor, Tensor)",
}


@pytest.fixture(scope="module")
def loaded():
    assert ops.try_load_torch_library(), "libarctic_mi355x.so is not built"
    return ops


def test_load_is_idempotent(loaded):
    assert ops.try_load_torch_library() and ops.try_load_torch_library()
    assert _native.is_loaded() and _native.loaded_path().endswith(".so")


def test_schemas_match_the_reference(loaded):
    for name, want in REFERENCE_SCHEMAS.items():
        got = str(getattr(torch.ops.arctic_inference, name).default._schema)
        assert re.sub(r"\s+", " ", got) == want


def test_no_cpu_backend_and_no_fallback(loaded):
    x = torch.randn(4, 64, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError, match="CPU"):
        ops.speculator_ln(x, None, None, 1e-6)
    with pytest.raises(NotImplementedError, match="CPU"):
        ops.sum_lstm(torch.randn(4, 256).bfloat16(), torch.randn(4, 256).bfloat16(), x, None, None, None, None, 1.0,
                     1e-6, 1e-6, False)
    with pytest.raises(NotImplementedError, match="CPU"):
        ops.reshape_and_cache_flash_bulk(x, x, [x], [x], torch.zeros(4, dtype=torch.int64), "auto", [x], [x], 1, 64)


def test_meta_tensors_trace_shapes_without_data(loaded):
    # shape-only implementations: output shapes, strides and dtypes of the real launches
    x = torch.empty(3, 5, 64, dtype=torch.bfloat16, device="meta")
    y = ops.speculator_ln(x, None, None, 1e-6)
    assert y.is_meta and y.shape == x.shape and y.dtype == x.dtype and y.is_contiguous()
    y = ops.speculator_add_ln_gelu(x, x, None, None, 0.5, 1e-6)
    assert y.is_meta and y.shape == x.shape
    pc = torch.empty(7, 100, dtype=torch.float16, device="meta")[:, :64]     # pitched rows
    s4 = torch.empty(7, 256, dtype=torch.float16, device="meta")
    state, cell = ops.sum_lstm(s4, s4, pc, None, None, None, None, 1.0, 1e-6, 1e-6, False)
    assert state.shape == cell.shape == (7, 64) and state.stride() == cell.stride() == (100, 1)
    state, cell = ops.sum_lstm_shared_z(s4, pc, pc, None, None, None, None, 1.0, 1e-6, 1e-6, False)
    assert state.shape == (7, 64) and state.dtype == torch.float16
    logits = torch.empty(4, 2, 1000, device="meta")
    t = ops.speculator_argmax(logits, 999)
    assert t.is_meta and t.shape == (4, 2) and t.dtype == torch.int64
    i = torch.empty(4, dtype=torch.int64, device="meta")
    assert ops.reshape_and_cache_flash_bulk(x, x, [x], [x], i, "auto", [x], [x], 1, 64) is None


def test_argument_checks_mirror_the_reference(loaded):
    # the host layer runs the reference's TORCH_CHECKs before touching the device, so the
    # ones that precede the device check can be exercised with CPU tensors
    ln, lstm, bulk = ops._IMPLS["speculator_ln_cuda"], ops._IMPLS["sum_lstm_cuda"], ops._IMPLS["reshape_and_cache_flash_bulk"]
    x32 = torch.randn(4, 64)
    slots = torch.zeros(4, dtype=torch.int64)
    with pytest.raises(RuntimeError, match="speculator_ln: only fp16 and bf16 are supported."):
        ln(x32, None, None, 1e-6)
    with pytest.raises(RuntimeError, match="speculator_ln: input must be CUDA"):
        ln(x32.bfloat16(), None, None, 1e-6)
    with pytest.raises(RuntimeError, match="sum_lstm: only fp16 and bf16 are supported."):
        lstm(x32, x32, x32, None, None, None, None, 1.0, 1e-6, 1e-6, False)
    with pytest.raises(RuntimeError, match="sum_lstm: inputs must be CUDA tensors"):
        lstm(x32.half(), x32.half(), x32.half(), None, None, None, None, 1.0, 1e-6, 1e-6, False)
    cache = torch.zeros(2, 4, 1, 64)
    with pytest.raises(RuntimeError, match="Unsupported data type of kv cache: nvfp4"):
        bulk(x32, x32, [cache], [cache], slots, "nvfp4", [x32], [x32], 1, 64)
    with pytest.raises(RuntimeError, match="Unsupported input type of kv cache"):
        bulk(x32.to(torch.int8), x32.to(torch.int8), [cache], [cache], slots, "auto", [x32], [x32], 1, 64)
    for accepted in ("auto", "fp8", "fp8_e4m3", "fp8_e5m2"):   # the strings of quant_utils.cuh:532-567 get past the dispatch
        with pytest.raises(RuntimeError, match="element size|same device"):
            bulk(x32, x32, [cache.double()], [cache.double()], slots, accepted, [x32], [x32], 1, 64)
    # empty layer list is a no-op (reference :87-89), mismatched list lengths are an error (:91-94)
    bulk(x32, x32, [], [], slots, "auto", [], [], 1, 64)
    with pytest.raises(RuntimeError, match="value_caches"):
        bulk(x32, x32, [x32], [], slots, "auto", [x32], [x32], 1, 64)
    with pytest.raises(RuntimeError, match="not a Tensor"):
        bulk(x32, x32, [cache], [None], slots, "auto", [x32], [x32], 1, 64)
    # per-layer geometry is compared with layer 0's on every call, whatever was accepted before
    with pytest.raises(RuntimeError, match="must share dtype, block stride, number of blocks"):
        bulk(x32, x32, [cache, cache.view(4, 2, 1, 64)], [cache, cache], slots, "auto", [x32] * 2, [x32] * 2, 1, 32)


def test_no_host_pointer_reaches_a_launch(loaded):
    """Called directly (past the dispatcher, which would turn CPU tensors away), every host-layer function refuses
    tensors that are not on a GPU before it hands a pointer to the library."""
    f = ops._IMPLS
    x = torch.randn(4, 64).bfloat16()
    slots = torch.zeros(4, dtype=torch.int64)
    cache = torch.zeros(2, 4, 1, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="must be CUDA tensors"):
        f["reshape_and_cache_flash_bulk"](x, x, [cache[0]], [cache[1]], slots, "auto", [x], [x], 1, 64)
    layers = ops.prepare_bulk_kv_layers([cache[0]], [cache[1]], [x], [x])
    assert layers.num_layers == 1
    with pytest.raises(RuntimeError, match="must be CUDA tensors"):
        layers.write(x, x, slots, "auto", 1, 64)
    with pytest.raises(RuntimeError, match="logits_indices must be a 1-D int32 or int64 CUDA tensor"):
        f["reshape_and_cache_flash_bulk_select"](x, x, [cache[0]], [cache[1]], slots, "auto", [x], [x], 1, 64, slots, x, x)
    key = torch.zeros(4, 2, 32).bfloat16()
    packed, scales = torch.zeros(4, 1, 2, 16, dtype=torch.uint8), torch.zeros(4, 1, 2, 2, dtype=torch.uint8)
    with pytest.raises(RuntimeError, match="one CUDA device"):
        f["reshape_and_cache_flash_fp4"](key, key, packed, packed, slots, "nvfp4", x, x, scales, scales)
    with pytest.raises(RuntimeError, match="contiguous 1-D CUDA tensor"):
        f["gather_rows"]([x], slots, [x])
    with pytest.raises(RuntimeError, match="contiguous 1-D CUDA tensor"):
        f["scatter_rows"]([x], slots, [x])
    with pytest.raises(RuntimeError, match="logits must be CUDA"):
        f["speculator_argmax_cuda"](x, 63)
    with pytest.raises(RuntimeError, match="input must be CUDA"):
        f["speculator_add_ln_act_cuda"](x, x, None, None, 1.0, 1e-6, "gelu", 1.0)
    with pytest.raises(RuntimeError, match="input must be CUDA"):
        f["speculator_embed_add_ln_act_cuda"](x, x, slots, None, None, 1.0, 1e-6, "gelu", 1.0)
    s4 = torch.randn(4, 256).bfloat16()
    for name, args in (("sum_lstm_zero_cell_cuda", (s4, s4)), ("sum_lstm_shared_z_cuda", (s4, x, x)),
                       ("sum_lstm_embedded_cuda", (s4, x, slots, x))):
        with pytest.raises(RuntimeError, match="inputs must be CUDA tensors"):
            f[name](*args, None, None, None, None, 1.0, 1e-6, 1e-6, False)
    # sizes that do not fit the library's ints are an error, not a wrapped value
    with pytest.raises(RuntimeError, match="num_heads and head_size must be positive"):
        f["reshape_and_cache_flash_bulk"](x, x, [cache[0]], [cache[1]], slots, "auto", [x], [x], 1 << 40, 64)


def test_missing_library_fails_loudly(monkeypatch):
    """Without the shared object: try_load returns False (as the reference does) and the
    operators raise; nothing falls back to another implementation."""
    monkeypatch.setattr(_native, "library_path", lambda: None)
    monkeypatch.setattr(_native, "_lib", None)
    monkeypatch.setattr(ops, "_registered", False)
    monkeypatch.setattr(ops, "_IMPLS", {})
    assert ops.try_load_torch_library() is False
    x = torch.randn(4, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="not loaded"):
        ops.speculator_ln(x, None, None, 1e-6)
    with pytest.raises(RuntimeError, match="not loaded"):
        ops.sum_lstm(x, x, x, None, None, None, None, 1.0, 1e-6, 1e-6, False)
    with pytest.raises(RuntimeError, match="not loaded"):
        ops.reshape_and_cache_flash_bulk(x, x, [x], [x], torch.zeros(4, dtype=torch.int64), "auto", [x], [x], 1, 64)
    with pytest.raises(RuntimeError, match="not found"):
        _native.load()
