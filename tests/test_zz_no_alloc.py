"""The entry point that allocates nothing, arctic_reshape_and_cache_flash_bulk_select_static, against the entry points
it stands in for (arctic_build_row_map + arctic_reshape_and_cache_flash_bulk_select with a row map of the caller's):
every cache byte and every selected row bit for bit, on two calls in a row, the second with a smaller input, so that
whatever the first call left in the library's device array would show.  All calls go through the C ABI."""
import ctypes
import functools

import pytest
import torch

import oracle
from arcticinference_amd import _native
from helpers import assert_bulk_equal, bulk_args, bulk_case_to, make_bulk_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SRC = {torch.bfloat16: _native.DTYPE_BF16, torch.float16: _native.DTYPE_F16, torch.float32: _native.DTYPE_F32}
KV = {"auto": _native.KV_AUTO, "fp8": _native.KV_FP8_E4M3, "fp8_e5m2": _native.KV_FP8_E5M2}


def table(tensors):
    return (ctypes.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def common_args(d):
    kc, vc = d["key_caches"], d["value_caches"]
    return (d["keys"].data_ptr(), d["values"].data_ptr(), d["keys"].stride(0), d["values"].stride(0),
            table(kc), table(vc), table(d["k_scales"]), table(d["v_scales"]),
            d["slot_mapping"].data_ptr(), d["slot_mapping"].numel(), len(kc), d["num_heads"], d["head_size"],
            kc[0].size(1), kc[0].stride(0), kc[0].size(0), SRC[d["keys"].dtype], KV[d["kv_cache_dtype"]])


def out_buffers(rows, width, dtype):
    out = []
    for _ in range(2):
        t = torch.empty(rows, width, dtype=dtype, device=DEV)
        t.view(torch.uint8).fill_(0xA5)
        out.append(t)
    return out


def both_ways(lib, case, idx):
    """Runs the workspace form and the static form on two device copies of `case`; returns what each wrote."""
    stream = torch.cuda.current_stream().cuda_stream
    idx = idx.to(DEV)
    width = case["keys"].size(1)
    rows = idx.numel() + 2
    results = []
    for static in (False, True):
        d = bulk_case_to(case, DEV)
        k_out, v_out = out_buffers(rows, width, case["keys"].dtype)
        tail = (idx.data_ptr(), idx.element_size(), idx.numel(), d["keys"].size(0), k_out.data_ptr(), v_out.data_ptr(),
                k_out.stride(0), v_out.stride(0), stream)
        if static:
            rc = lib.arctic_reshape_and_cache_flash_bulk_select_static(*common_args(d), *tail)
            assert rc == 0, lib.arctic_last_error()
            torch.cuda.synchronize()
        else:
            row_map = torch.empty(d["slot_mapping"].numel(), dtype=torch.int64, device=DEV)
            rc = lib.arctic_build_row_map(row_map.data_ptr(), row_map.numel(), idx.data_ptr(), idx.element_size(),
                                          idx.numel(), stream)
            assert rc == 0, lib.arctic_last_error()
            rc = lib.arctic_reshape_and_cache_flash_bulk_select(*common_args(d), row_map.data_ptr(), *tail)
            assert rc == 0, lib.arctic_last_error()
            torch.cuda.synchronize()
        results.append((d, k_out, v_out))
    return results


def check_pair(lib, case, idx):
    (d_ws, k_ws, v_ws), (d_st, k_st, v_st) = both_ways(lib, case, idx)
    bits = lambda t: t.cpu().contiguous().view(torch.uint8)
    for a, b in zip(d_st["bufs"], d_ws["bufs"]):
        assert torch.equal(bits(a), bits(b)), "static and workspace forms wrote different cache bytes"
    assert torch.equal(bits(k_st), bits(k_ws)) and torch.equal(bits(v_st), bits(v_ws))
    # and both are right: caches against the CPU oracle, selected rows against index_select
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    assert_bulk_equal(d_st["bufs"], case["bufs"])
    n = idx.numel()
    assert torch.equal(bits(k_st[:n]), bits(case["keys"].index_select(0, idx.long())))
    assert torch.equal(bits(v_st[:n]), bits(case["values"].index_select(0, idx.long())))
    assert (bits(k_st[n:]) == 0xA5).all() and (bits(v_st[n:]) == 0xA5).all()


def test_two_calls_in_a_row_the_second_smaller(ops):
    lib = _native.load()
    g = torch.Generator().manual_seed(5)
    # Index lists of more than 2048 entries are what makes the entry point use its device array (shorter lists are
    # scanned by the token workgroups and need no row map).  First call: 3000 tokens, 2600 of them selected, some twice.
    big = make_bulk_case(T=3000, L=4, H=8, D=128, bs=16, NB=256, kv_cache_dtype="fp8", seed=60, std=1.5, pad_fraction=0.1)
    idx_big = torch.cat([torch.randperm(3000, generator=g)[:2600], torch.tensor([2999, 2999, 1500])])
    check_pair(lib, big, idx_big)
    # second call, smaller in every respect and again through the array: tokens 0..2399 had other entries in the
    # first call's row map, entries 2400..2999 of the array still hold the first call's
    small = make_bulk_case(T=2400, L=3, H=8, D=128, bs=16, NB=160, kv_cache_dtype="fp8", seed=61, std=1.5, pad_fraction=0.2)
    idx_small = torch.cat([torch.randperm(2400, generator=g)[:2100], torch.tensor([7, 3, 2399, 3, 0])]).to(torch.int32)
    assert idx_small.numel() > 2048
    check_pair(lib, small, idx_small)
    # third: a bf16 cache, the element-wise kernel (60-element rows), keys with more rows than slots, a long list
    odd = make_bulk_case(T=2300, L=2, H=3, D=20, bs=4, NB=600, kv_cache_dtype="auto", seed=62, key_pad=3)
    odd["slot_mapping"] = odd["slot_mapping"][:2250].contiguous()
    check_pair(lib, odd, torch.cat([torch.arange(2300), torch.tensor([49, 0, 2260, 12, 12])]))
    # short lists (no row map in either form) and an empty one (the plain write)
    tiny = make_bulk_case(T=90, L=3, H=8, D=128, bs=16, NB=8, kv_cache_dtype="fp8", seed=64, std=1.5, pad_fraction=0.2)
    check_pair(lib, tiny, torch.tensor([7, 3, 88, 3, 0], dtype=torch.int32))
    check_pair(lib, tiny, torch.empty(0, dtype=torch.int64))


def static_call(lib, d, idx, k_out, v_out, stream):
    rc = lib.arctic_reshape_and_cache_flash_bulk_select_static(
        *common_args(d), idx.data_ptr(), idx.element_size(), idx.numel(), d["keys"].size(0), k_out.data_ptr(),
        v_out.data_ptr(), k_out.stride(0), v_out.stride(0), stream)
    assert rc == 0, lib.arctic_last_error()


def workspace_result(lib, case, idx):
    """(cache buffers, k_out, v_out) as the workspace form leaves them, on the host."""
    d = bulk_case_to(case, DEV)
    k_out, v_out = out_buffers(idx.numel() + 2, case["keys"].size(1), case["keys"].dtype)
    stream = torch.cuda.current_stream().cuda_stream
    row_map = torch.empty(d["slot_mapping"].numel(), dtype=torch.int64, device=DEV)
    assert lib.arctic_build_row_map(row_map.data_ptr(), row_map.numel(), idx.data_ptr(), idx.element_size(), idx.numel(),
                                    stream) == 0
    rc = lib.arctic_reshape_and_cache_flash_bulk_select(
        *common_args(d), row_map.data_ptr(), idx.data_ptr(), idx.element_size(), idx.numel(), d["keys"].size(0),
        k_out.data_ptr(), v_out.data_ptr(), k_out.stride(0), v_out.stride(0), stream)
    assert rc == 0, lib.arctic_last_error()
    torch.cuda.synchronize()
    return [b.cpu() for b in d["bufs"]], k_out.cpu(), v_out.cpu()


def assert_same(got, want, what):
    bits = lambda t: t.cpu().contiguous().view(torch.uint8)
    bufs, k_out, v_out = got
    for a, b in zip(bufs, want[0]):
        assert torch.equal(bits(a), bits(b)), f"{what}: cache bytes differ from the workspace form's"
    assert torch.equal(bits(k_out), bits(want[1])) and torch.equal(bits(v_out), bits(want[2])), f"{what}: selected rows differ"


@functools.lru_cache(maxsize=None)
def two_long_list_cases():
    """A large and a small case whose index lists need the row map; the host copies are read only."""
    g = torch.Generator().manual_seed(9)
    a = make_bulk_case(T=20000, L=8, H=8, D=128, bs=16, NB=1300, kv_cache_dtype="fp8", seed=65, std=1.5, pad_fraction=0.1)
    idx_a = torch.randperm(20000, generator=g)[:9000].to(DEV)
    b = make_bulk_case(T=2500, L=2, H=8, D=128, bs=16, NB=160, kv_cache_dtype="fp8", seed=66, std=1.5, pad_fraction=0.1)
    idx_b = torch.cat([torch.randperm(2500, generator=g)[:2200], torch.tensor([5, 5, 2499])]).to(torch.int32).to(DEV)
    return (a, idx_a), (b, idx_b)


def test_nothing_is_allocated_and_calls_queue_up_without_a_wait_between_them(ops):
    """What the entry point is for: after a first call on the device (which looks the array's address up), a call
    leaves the free device memory as it found it (hipMemGetInfo), and two calls issued back to back on one stream,
    the second smaller, with no synchronisation in between, both give the workspace form's result."""
    lib = _native.load()
    (a, idx_a), (b, idx_b) = two_long_list_cases()
    want_a, want_b = workspace_result(lib, a, idx_a), workspace_result(lib, b, idx_b)
    da, db = bulk_case_to(a, DEV), bulk_case_to(b, DEV)
    ka, va = out_buffers(idx_a.numel() + 2, a["keys"].size(1), a["keys"].dtype)
    kb, vb = out_buffers(idx_b.numel() + 2, b["keys"].size(1), b["keys"].dtype)
    stream = torch.cuda.current_stream().cuda_stream
    static_call(lib, da, idx_a, ka, va, stream)      # first calls: the array's address is looked up, both kernel
    static_call(lib, db, idx_b, kb, vb, stream)      # shapes have run once
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    static_call(lib, da, idx_a, ka, va, stream)
    static_call(lib, db, idx_b, kb, vb, stream)      # no wait in between: the stream orders the two uses of the array
    free_after = torch.cuda.mem_get_info()[0]
    torch.cuda.synchronize()
    assert free_after == free_before, f"free device memory changed by {free_before - free_after} bytes across two calls"
    assert_same((da["bufs"], ka, va), want_a, "first call")
    assert_same((db["bufs"], kb, vb), want_b, "second call")


def test_calls_on_two_streams_take_turns_at_the_array(ops):
    """Two calls with long lists on two streams that nothing orders: the library makes the second stream wait for the
    first call's use of the array (an event behind its kernels), so both give the workspace form's result.  The first
    call is large (its kernel runs for tens of microseconds), the second small and issued right behind it."""
    lib = _native.load()
    (a, idx_a), (b, idx_b) = two_long_list_cases()
    want_a, want_b = workspace_result(lib, a, idx_a), workspace_result(lib, b, idx_b)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    for round_ in range(3):
        da, db = bulk_case_to(a, DEV), bulk_case_to(b, DEV)
        ka, va = out_buffers(idx_a.numel() + 2, a["keys"].size(1), a["keys"].dtype)
        kb, vb = out_buffers(idx_b.numel() + 2, b["keys"].size(1), b["keys"].dtype)
        torch.cuda.synchronize()
        static_call(lib, da, idx_a, ka, va, s1.cuda_stream)
        static_call(lib, db, idx_b, kb, vb, s2.cuda_stream)
        static_call(lib, da, idx_a, ka, va, s1.cuda_stream)     # back on the first stream: waits for the second's use
        torch.cuda.synchronize()
        assert_same((da["bufs"], ka, va), want_a, f"round {round_}, first stream")
        assert_same((db["bufs"], kb, vb), want_b, f"round {round_}, second stream")


def test_recorded_into_a_hip_graph(ops):
    """A call with a long list recorded into a HIP graph (after a first call outside capture) and replayed three
    times, with eager work and synchronisations between the replays; every replay gives the eager result."""
    lib = _native.load()
    (_, _), (b, idx_b) = two_long_list_cases()
    want = workspace_result(lib, b, idx_b)
    d = bulk_case_to(b, DEV)
    fresh = [buf.clone() for buf in d["bufs"]]
    k_out, v_out = out_buffers(idx_b.numel() + 2, b["keys"].size(1), b["keys"].dtype)
    static_call(lib, d, idx_b, k_out, v_out, torch.cuda.current_stream().cuda_stream)   # outside capture
    torch.cuda.synchronize()
    assert_same((d["bufs"], k_out, v_out), want, "eager call")
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_call(lib, d, idx_b, k_out, v_out, torch.cuda.current_stream().cuda_stream)
    for replay in range(3):
        for buf, init in zip(d["bufs"], fresh):
            buf.copy_(init)
        k_out.view(torch.uint8).fill_(0xA5)
        v_out.view(torch.uint8).fill_(0xA5)
        (torch.ones(1000, device=DEV) * 2).sum().item()      # the program's own eager work and a synchronisation
        graph.replay()
        torch.cuda.synchronize()
        assert_same((d["bufs"], k_out, v_out), want, f"replay {replay}")


def test_size_limit_and_argument_errors(ops):
    lib = _native.load()
    case = make_bulk_case(T=8, L=2, H=2, D=64, bs=16, NB=2, kv_cache_dtype="fp8", seed=63)
    d = bulk_case_to(case, DEV)
    args = list(common_args(d))
    idx = torch.arange(4, device=DEV)
    out = torch.zeros(4, 256, dtype=torch.bfloat16, device=DEV)
    tail = (idx.data_ptr(), 8, 4, 8, out.data_ptr(), out.data_ptr(), 256, 256, None)
    too_many = list(args)
    too_many[9] = 262144 + 1
    rc = lib.arctic_reshape_and_cache_flash_bulk_select_static(*too_many, *tail)
    assert rc == 1 and b"exceeds the 262144 tokens" in lib.arctic_last_error()
    rc = lib.arctic_reshape_and_cache_flash_bulk_select_static(*args, None, 8, 4, 8, *tail[4:])
    assert rc == 1 and b"null indices" in lib.arctic_last_error()
    rc = lib.arctic_reshape_and_cache_flash_bulk_select_static(*args, idx.data_ptr(), 2, 4, 8, *tail[4:])
    assert rc == 2 and b"int32 or int64" in lib.arctic_last_error()
    # a list long enough to need the array, refused for its other arguments: nothing may have been enqueued by then
    long_idx = torch.arange(3000, device=DEV) % 8
    long_tail = (long_idx.data_ptr(), 8, 3000, 8, out.data_ptr(), out.data_ptr(), 256, 256, None)
    rc = lib.arctic_reshape_and_cache_flash_bulk_select_static(*args, *long_tail[:4], None, *long_tail[5:])
    assert rc == 1 and b"null keys_out" in lib.arctic_last_error()
    bad_type = list(args)
    bad_type[16] = 7
    rc = lib.arctic_reshape_and_cache_flash_bulk_select_static(*bad_type, *long_tail)
    assert rc == 2 and b"Unsupported input type" in lib.arctic_last_error()
    rc = lib.arctic_reshape_and_cache_flash_bulk_select_static(*args, long_idx.data_ptr(), 8, 1 << 31, 8, *long_tail[4:])
    assert rc == 1 and b"2^31 output rows" in lib.arctic_last_error()
    torch.cuda.synchronize()
    assert not out.any()
