"""GPU parity of the bulk KV-cache write with the row selection folded in
(reshape_and_cache_flash_bulk followed by the k_states / v_states index_select calls of swiftkv_select,
arctic_inference/vllm/swiftkv/llama_swiftkv.py:617-622, 663-679): the caches bit-exact against the CPU oracle,
the selected rows bit-exact against torch.index_select."""
import ctypes

import pytest
import torch

import oracle
from arcticinference_amd import _native
from helpers import assert_bulk_equal, bulk_args, bulk_case_to, make_bulk_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run_select(ops, case, idx, buffer_rows, out_pad=0):
    """Caches against the oracle, selected rows against index_select, buffer rows beyond the selection untouched."""
    dcase = bulk_case_to(case, DEV)
    width = case["keys"].size(1)

    def buffer():
        full = torch.empty(buffer_rows, width + out_pad, dtype=case["keys"].dtype, device=DEV)
        full.view(torch.uint8).fill_(0xA5)
        return full[:, :width]

    k_out, v_out = buffer(), buffer()
    k_sel, v_sel = ops.reshape_and_cache_flash_bulk_select(*bulk_args(dcase), idx.to(DEV), k_out, v_out)
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    assert_bulk_equal(dcase["bufs"], case["bufs"])
    n = idx.numel()
    assert k_sel.shape == (n, width) and (n == 0 or k_sel.data_ptr() == k_out.data_ptr())
    bits = lambda t: t.cpu().contiguous().view(torch.uint8)
    assert torch.equal(bits(k_sel), bits(case["keys"].index_select(0, idx.long())))
    assert torch.equal(bits(v_sel), bits(case["values"].index_select(0, idx.long())))
    assert (bits(k_out[n:]) == 0xA5).all() and (bits(v_out[n:]) == 0xA5).all()
    return dcase


@pytest.mark.parametrize("kv", ["auto", "fp8", "fp8_e5m2"])
@pytest.mark.parametrize("src_dtype", [torch.bfloat16, torch.float32])
def test_decode_batch_every_token_selected(ops, kv, src_dtype):
    case = make_bulk_case(T=192, L=6, H=8, D=128, bs=16, NB=64, src_dtype=src_dtype, kv_cache_dtype=kv, seed=41, std=1.5)
    run_select(ops, case, torch.arange(192), 256)


@pytest.mark.parametrize("kv", ["auto", "fp8"])
@pytest.mark.parametrize("index_dtype", [torch.int64, torch.int32])
def test_mixed_batch_few_tokens_selected(ops, kv, index_dtype):
    case = make_bulk_case(T=2048, L=8, H=8, D=128, bs=16, NB=256, kv_cache_dtype=kv, seed=42, std=1.5, pad_fraction=0.1,
                          key_pad=8)
    g = torch.Generator().manual_seed(1)
    idx = torch.sort(torch.randperm(2048, generator=g)[:37]).values.to(index_dtype)
    run_select(ops, case, idx, 64, out_pad=8)


def test_unsorted_selection_and_selected_padding_tokens(ops):
    # a token whose slot is padding is still copied out: index_select does not look at slot_mapping
    case = make_bulk_case(T=300, L=5, H=4, D=64, bs=16, NB=32, kv_cache_dtype="fp8", seed=43, pad_fraction=0.3)
    pads = torch.nonzero(case["slot_mapping"] < 0).flatten()
    valid = torch.nonzero(case["slot_mapping"] >= 0).flatten()
    idx = torch.cat([pads[:7], valid[:9], pads[7:9]])[torch.randperm(18, generator=torch.Generator().manual_seed(2))]
    run_select(ops, case, idx, 18)


@pytest.mark.parametrize("T,L", [(16, 40), (1, 3), (700, 70)])
def test_layer_groups_more_than_one_launch_and_tiny_batches(ops, T, L):
    case = make_bulk_case(T=T, L=L, H=2, D=64, bs=16, NB=max(4, T // 8), kv_cache_dtype="fp8", seed=44)
    g = torch.Generator().manual_seed(3)
    idx = torch.sort(torch.randperm(T, generator=g)[: max(1, T // 2)]).values
    run_select(ops, case, idx, T)


@pytest.mark.parametrize("kv", ["auto", "fp8"])
def test_rows_that_force_the_element_wise_kernel(ops, kv):
    # 3 heads x 20 = 60 elements per row and an odd output pitch: no 16-byte access possible
    case = make_bulk_case(T=50, L=3, H=3, D=20, bs=4, NB=16, kv_cache_dtype=kv, seed=45, key_pad=3)
    idx = torch.tensor([49, 0, 7, 8, 30])
    run_select(ops, case, idx, 9, out_pad=1)


@pytest.mark.parametrize("kv", ["auto", "fp8"])
def test_one_slot_but_more_source_rows_with_a_pitch_that_is_no_multiple_of_16_bytes(ops, kv):
    """A single token needs no row pitch, so a lone slot used to qualify for 16-byte accesses whatever the pitch;
    with an index list the launch also reads source rows beyond the slot mapping, at multiples of that pitch.  Rows
    of 256 elements (16-byte chunks possible) 259 elements apart, one slot, three source rows, all three selected."""
    case = make_bulk_case(T=3, L=2, H=2, D=64, bs=16, NB=2, kv_cache_dtype=kv, seed=46, key_pad=3)
    case["slot_mapping"] = case["slot_mapping"][:1].contiguous()
    run_select(ops, case, torch.tensor([2, 0, 1, 2]), 6)


def test_random_configurations(ops):
    """Seeded sweep over shapes, dtypes, layouts, pitches, padding and selections (none, few, all, shuffled)."""
    import random
    rnd = random.Random(77)
    for it in range(30):
        H = rnd.choice([1, 2, 3, 8])
        D = rnd.choice([16, 64, 80, 128, 20])
        cfg = dict(T=rnd.choice([1, 2, 7, 33, 130, 600]), L=rnd.choice([1, 2, 5, 16, 33, 65]), H=H, D=D,
                   bs=rnd.choice([1, 4, 16, 32]), NB=0,
                   src_dtype=rnd.choice([torch.bfloat16, torch.float16, torch.float32]),
                   kv_cache_dtype=rnd.choice(["auto", "fp8", "fp8_e5m2"]), seed=3000 + it, std=rnd.choice([0.1, 1.5, 30.0]),
                   pad_fraction=rnd.choice([0.0, 0.1, 0.5]), layout=rnd.choice(["flash", "flashinfer"]),
                   key_pad=rnd.choice([0, 0, 8, 3]))
        cfg["NB"] = (cfg["T"] + cfg["bs"] - 1) // cfg["bs"] + rnd.choice([0, 1, 5])
        if cfg["T"] * cfg["L"] * H * D > 20_000_000:
            cfg["L"] = max(1, 20_000_000 // (cfg["T"] * H * D))
        T = cfg["T"]
        g = torch.Generator().manual_seed(it)
        n_sel = rnd.choice([0, 1, max(1, T // 3), T])
        if rnd.random() < 0.3:
            idx = torch.randint(0, T, (n_sel,), generator=g)       # with repeats
        else:
            idx = torch.randperm(T, generator=g)[:n_sel]
        if rnd.random() < 0.6:
            idx = torch.sort(idx).values
        try:
            run_select(ops, make_bulk_case(**cfg), idx, n_sel + rnd.choice([0, 3]), out_pad=rnd.choice([0, 8, 1]))
        except AssertionError as e:
            raise AssertionError(f"configuration {it}: {cfg}, {n_sel} selected: {e}") from None


@pytest.mark.parametrize("kv", ["auto", "fp8"])
@pytest.mark.parametrize("shape", ["vector", "element_wise"])
def test_repeated_indices_and_rows_beyond_the_slot_mapping_match_index_select(ops, kv, shape):
    # index_select semantics for every index inside keys / values: an index named twice fills both output rows, and
    # a source row at or beyond slot_mapping.size(0) (keys may hold more rows than there are slots) is copied too
    H, D, pad = (8, 128, 0) if shape == "vector" else (3, 20, 3)
    case = make_bulk_case(T=120, L=5, H=H, D=D, bs=16, NB=16, kv_cache_dtype=kv, seed=49, pad_fraction=0.2, key_pad=pad)
    case["slot_mapping"] = case["slot_mapping"][:100].contiguous()
    idx = torch.tensor([5, 5, 99, 100, 119, 5, 0, 118, 99, 7, 7])
    run_select(ops, case, idx, 16, out_pad=pad and 1)
    # more layers than one launch holds, every index repeated
    case = make_bulk_case(T=9, L=70, H=2, D=64, bs=16, NB=4, kv_cache_dtype=kv, seed=50)
    run_select(ops, case, torch.tensor([8, 8, 0, 0, 3, 3, 3]), 7)


@pytest.mark.parametrize("kv", ["auto", "fp8"])
def test_index_lists_too_long_to_scan_go_through_the_row_map(ops, kv):
    # more than 2048 indices: the operator builds the inverse of the list first; repeats and rows beyond the slot
    # mapping are then served by the index workgroups
    case = make_bulk_case(T=3300, L=3, H=8, D=128, bs=16, NB=256, kv_cache_dtype=kv, seed=52, pad_fraction=0.1)
    case["slot_mapping"] = case["slot_mapping"][:3200].contiguous()
    g = torch.Generator().manual_seed(6)
    idx = torch.cat([torch.randperm(3300, generator=g)[:2600], torch.randint(0, 3300, (150,), generator=g)])
    assert idx.numel() > 2048
    run_select(ops, case, idx, idx.numel() + 3)
    # the element-wise kernel with a long list
    case = make_bulk_case(T=2200, L=2, H=1, D=20, bs=4, NB=600, kv_cache_dtype=kv, seed=53, key_pad=3)
    idx = torch.cat([torch.arange(2200), torch.tensor([7, 7, 2199])])
    run_select(ops, case, idx, idx.numel(), out_pad=1)


def test_scan_and_row_map_agree_through_the_c_abi(ops):
    # the same short list served both ways: without a row map (the token workgroups scan the list) and with one
    lib = _native.load()
    stream = torch.cuda.current_stream().cuda_stream
    case = make_bulk_case(T=200, L=5, H=8, D=128, bs=16, NB=16, kv_cache_dtype="fp8", seed=54, pad_fraction=0.2)
    idx = torch.tensor([5, 199, 5, 0, 77, 5, 198, 0], device=DEV)
    tab = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    outs = []
    for with_map in (False, True):
        d = bulk_case_to(case, DEV)
        k_out = torch.zeros(8, 5 * 1024, dtype=torch.bfloat16, device=DEV)
        v_out = torch.zeros_like(k_out)
        row_map = torch.empty(200, dtype=torch.int64, device=DEV)
        assert lib.arctic_build_row_map(row_map.data_ptr(), 200, idx.data_ptr(), 8, 8, stream) == 0
        rc = lib.arctic_reshape_and_cache_flash_bulk_select(
            d["keys"].data_ptr(), d["values"].data_ptr(), d["keys"].stride(0), d["values"].stride(0), tab(d["key_caches"]),
            tab(d["value_caches"]), tab(d["k_scales"]), tab(d["v_scales"]), d["slot_mapping"].data_ptr(), 200, 5, 8, 128, 16,
            d["key_caches"][0].stride(0), 16, _native.DTYPE_BF16, _native.KV_FP8_E4M3,
            row_map.data_ptr() if with_map else None, idx.data_ptr(), 8, 8, 200, k_out.data_ptr(), v_out.data_ptr(),
            k_out.stride(0), v_out.stride(0), stream)
        assert rc == 0, lib.arctic_last_error()
        torch.cuda.synchronize()
        outs.append((d, k_out, v_out))
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    for d, k_out, v_out in outs:
        assert_bulk_equal(d["bufs"], case["bufs"])
        assert torch.equal(k_out.cpu(), case["keys"][idx.cpu()]) and torch.equal(v_out.cpu(), case["values"][idx.cpu()])


def test_indices_outside_the_source_leave_their_rows_untouched(ops):
    case = make_bulk_case(T=40, L=3, H=8, D=128, bs=16, NB=4, kv_cache_dtype="fp8", seed=51)
    d = bulk_case_to(case, DEV)
    width = case["keys"].size(1)
    k_out = torch.full((6, width), 3.0, dtype=torch.bfloat16, device=DEV)
    v_out = torch.full((6, width), 3.0, dtype=torch.bfloat16, device=DEV)
    idx = torch.tensor([2, 40, -1, 39, 1 << 40, 2], device=DEV)
    ops.reshape_and_cache_flash_bulk_select(*bulk_args(d), idx, k_out, v_out)
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    assert_bulk_equal(d["bufs"], case["bufs"])
    for out, src in ((k_out, case["keys"]), (v_out, case["values"])):
        out = out.cpu()
        assert torch.equal(out[0], src[2]) and torch.equal(out[5], src[2]) and torch.equal(out[3], src[39])
        assert (out[[1, 2, 4]] == 3.0).all()


def test_empty_selection_and_no_layers(ops):
    case = make_bulk_case(T=64, L=4, H=8, D=128, bs=16, NB=8, kv_cache_dtype="fp8", seed=46)
    run_select(ops, case, torch.empty(0, dtype=torch.int64), 4)
    d = bulk_case_to(case, DEV)
    k_out = torch.zeros(8, 4 * 1024, dtype=torch.bfloat16, device=DEV)
    v_out = torch.zeros_like(k_out)
    idx = torch.tensor([5, 9], device=DEV)
    # no layers: no columns, nothing is written anywhere (whatever the width of the buffers)
    ops.reshape_and_cache_flash_bulk_select(d["keys"], d["values"], [], [], d["slot_mapping"], "fp8", [], [], 8, 128, idx,
                                            k_out[:, :100], v_out)
    assert not k_out.any() and not v_out.any()
    # no slots: no cache row is written, the first layers x heads x head_size columns are still selected
    wide = torch.cat([d["keys"], d["keys"][:, :8]], dim=1)
    before = [b.clone() for b in d["bufs"]]
    k_sel, v_sel = ops.reshape_and_cache_flash_bulk_select(wide, d["values"], d["key_caches"], d["value_caches"],
                                                           d["slot_mapping"][:0], "fp8", d["k_scales"], d["v_scales"],
                                                           8, 128, idx, k_out, v_out)
    assert torch.equal(k_sel, d["keys"][idx]) and torch.equal(v_sel, d["values"][idx])
    assert all(torch.equal(a.view(torch.uint8), b.view(torch.uint8)) for a, b in zip(d["bufs"], before))


def test_row_map_helper_and_out_of_range_rows_through_the_c_abi(ops):
    lib = _native.load()
    stream = torch.cuda.current_stream().cuda_stream
    idx = torch.tensor([4, 9, -1, 100, 0], dtype=torch.int32, device=DEV)
    row_map = torch.full((10,), 77, dtype=torch.int64, device=DEV)
    assert lib.arctic_build_row_map(row_map.data_ptr(), 10, idx.data_ptr(), 4, 5, stream) == 0
    assert row_map.tolist() == [4, -1, -1, -1, 0, -1, -1, -1, -1, 1]
    assert lib.arctic_build_row_map(row_map.data_ptr(), 10, idx.data_ptr(), 2, 5, stream) != 0

    # rows at or beyond num_out_rows are not written
    case = make_bulk_case(T=10, L=2, H=2, D=64, bs=16, NB=2, kv_cache_dtype="auto", seed=47)
    d = bulk_case_to(case, DEV)
    k_out = torch.zeros(10, 256, dtype=torch.bfloat16, device=DEV)
    v_out = torch.zeros_like(k_out)
    tab = lambda ts: (ctypes.c_void_p * len(ts))(*[t.data_ptr() for t in ts])
    rc = lib.arctic_reshape_and_cache_flash_bulk_select(
        d["keys"].data_ptr(), d["values"].data_ptr(), 256, 256, tab(d["key_caches"]), tab(d["value_caches"]), None, None,
        d["slot_mapping"].data_ptr(), 10, 2, 2, 64, 16, d["key_caches"][0].stride(0), 2, _native.DTYPE_BF16,
        _native.KV_AUTO, row_map.data_ptr(), None, 0, 2, 10, k_out.data_ptr(), v_out.data_ptr(), 256, 256, stream)
    assert rc == 0, lib.arctic_last_error()
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    assert_bulk_equal(d["bufs"], case["bufs"])
    want = torch.zeros(10, 256, dtype=torch.bfloat16)
    want[0] = case["keys"][4]        # row_map[4] = 0
    want[1] = case["keys"][9]        # row_map[9] = 1; row_map[0] = 4 is beyond the two output rows
    assert torch.equal(k_out.cpu(), want)


def test_errors(ops):
    case = make_bulk_case(T=8, L=2, H=2, D=64, bs=16, NB=2, kv_cache_dtype="fp8", seed=48)
    d = bulk_case_to(case, DEV)
    idx = torch.arange(4, device=DEV)
    good = torch.zeros(4, 256, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="at least 4 rows"):
        ops.reshape_and_cache_flash_bulk_select(*bulk_args(d), idx, good[:3], good)
    with pytest.raises(RuntimeError, match="must have 256 columns"):
        ops.reshape_and_cache_flash_bulk_select(*bulk_args(d), idx, good[:, :128], good[:, :128])
    with pytest.raises(RuntimeError, match="of their type"):
        ops.reshape_and_cache_flash_bulk_select(*bulk_args(d), idx, good.half(), good)
    with pytest.raises(RuntimeError, match="1-D int32 or int64"):
        ops.reshape_and_cache_flash_bulk_select(*bulk_args(d), idx.float(), good, good)
