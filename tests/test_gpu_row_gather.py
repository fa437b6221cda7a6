"""GPU parity of gather_rows / scatter_rows (the index_select calls and the write-back around the
bulk KV write, llama_swiftkv.py:663-679, 733-742) against torch's own indexing: bit-exact."""
import ctypes

import pytest
import torch

import oracle
from arcticinference_amd import _native

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def swiftkv_tensors(T, hidden, kv_width, gen, pos_dtype=torch.int64):
    rn = lambda *s: torch.randn(*s, generator=gen).to(torch.bfloat16)
    return [rn(T, hidden), rn(T, hidden), torch.randint(0, 1 << 20, (T,), generator=gen).to(pos_dtype),
            rn(T, kv_width), rn(T, kv_width)]


def sentinel_like(t, rows):
    out = torch.empty((rows,) + tuple(t.shape[1:]), dtype=t.dtype)
    out.view(torch.uint8).fill_(0xA5)
    return out


def check_gather(ops, tensors, indices, buffer_rows):
    bufs = [sentinel_like(t, buffer_rows) for t in tensors]
    want = oracle.gather_rows(tensors, indices.cpu(), [b.clone() for b in bufs])
    dbufs = [b.to(DEV) for b in bufs]
    got = ops.gather_rows([t.to(DEV) for t in tensors], indices.to(DEV), dbufs)
    torch.cuda.synchronize()
    for k, (g, w) in enumerate(zip(got, want)):
        assert g.data_ptr() == dbufs[k].data_ptr()
        assert torch.equal(g.cpu().view(torch.uint8), w.view(torch.uint8)), f"tensor {k} differs"


@pytest.mark.parametrize("index_dtype", [torch.int64, torch.int32])
def test_decode_batch_all_rows_survive(ops, index_dtype):
    # 512 decode tokens of the 70B model: hidden 8192, K and V of 40 layers x 8 heads x 128
    g = torch.Generator().manual_seed(0)
    tensors = swiftkv_tensors(512, 8192, 40 * 1024, g)
    check_gather(ops, tensors, torch.arange(512, dtype=index_dtype), 512)


def test_prefill_chunk_few_rows_survive(ops):
    g = torch.Generator().manual_seed(1)
    tensors = swiftkv_tensors(4096, 4096, 16 * 1024, g)
    idx = torch.sort(torch.randperm(4096, generator=g)[:9]).values
    check_gather(ops, tensors, idx, 64)       # buffer rows beyond the batch keep their contents


def test_odd_row_sizes_pitches_and_repeats(ops):
    g = torch.Generator().manual_seed(2)
    base = torch.randn(40, 300, generator=g).to(torch.float16)
    tensors = [
        base[:, :260],                                            # pitched rows, 8-byte units
        torch.randint(0, 255, (40, 3), generator=g).to(torch.uint8),   # 3-byte rows
        torch.randint(0, 1000, (40,), generator=g).to(torch.int32),    # 4-byte rows
        torch.randn(40, 2, 5, 7, generator=g),                    # rank 4
        base[:, 1:258],                                           # rows start at an odd element
    ]
    idx = torch.tensor([5, 5, 39, 0, 17, 5, 38])
    bufs = [sentinel_like(t, 16) for t in tensors]
    want = oracle.gather_rows(tensors, idx, [b.clone() for b in bufs])
    dsrc = []
    for t in tensors:                       # keep the pitch on the device
        if t.dim() == 2 and t.stride(0) != t.size(1):
            full = torch.empty(t.size(0), 300, dtype=t.dtype, device=DEV)
            off = t.storage_offset()
            full.copy_(base.to(DEV))
            dsrc.append(full[:, off:off + t.size(1)])
        else:
            dsrc.append(t.to(DEV))
    got = ops.gather_rows(dsrc, idx.to(DEV), [b.to(DEV) for b in bufs])
    for k, (gk, wk) in enumerate(zip(got, want)):
        assert torch.equal(gk.cpu().view(torch.uint8), wk.view(torch.uint8)), f"tensor {k} differs"
    # without output buffers the results are allocated like tensor.index_select(0, indices)
    alloc = ops.gather_rows(dsrc, idx.to(DEV))
    for t, a in zip(tensors, alloc):
        assert torch.equal(a.cpu(), t.index_select(0, idx))


def test_out_of_range_indices_move_nothing(ops):
    g = torch.Generator().manual_seed(3)
    tensors = swiftkv_tensors(32, 256, 512, g)
    idx = torch.tensor([3, -1, 32, 31, 1 << 40, 0])
    check_gather(ops, tensors, idx, 8)


def test_scatter_back(ops):
    # orig_hidden_states[logits_indices] = hidden_states[:batch_size]
    g = torch.Generator().manual_seed(4)
    orig = torch.randn(4096, 8192, generator=g).to(torch.bfloat16)
    hs = torch.randn(64, 8192, generator=g).to(torch.bfloat16)     # padded decode buffer
    idx = torch.sort(torch.randperm(4096, generator=g)[:37]).values
    want = orig.clone()
    want[idx] = hs[:37]
    also = orig.clone()
    oracle.scatter_rows([hs], idx, [also])
    assert torch.equal(also, want)
    d = orig.to(DEV)
    ops.scatter_rows([hs.to(DEV)], idx.to(DEV), [d])
    assert torch.equal(d.cpu().view(torch.int16), want.view(torch.int16))


def test_more_indices_than_one_grid_dimension_holds(ops):
    # 70000 indices: the grid's second dimension stops at 65535, the kernel walks the rest
    g = torch.Generator().manual_seed(7)
    tensors = [torch.randn(1000, 24, generator=g).to(torch.bfloat16), torch.randint(0, 1 << 30, (1000,), generator=g)]
    idx = torch.randint(0, 1000, (70000,), generator=g)
    idx[65535:65540] = torch.tensor([-1, 1000, 0, 999, 5])
    check_gather(ops, tensors, idx, 70000)
    perm = torch.randperm(70000, generator=g)
    rows = torch.randn(70000, 6, generator=g)
    want = torch.zeros(70000, 6)
    want[perm] = rows
    d = torch.zeros(70000, 6, device=DEV)
    ops.scatter_rows([rows.to(DEV)], perm.to(DEV), [d])
    assert torch.equal(d.cpu(), want)


def test_empty_and_errors(ops):
    x = torch.randn(8, 64, device=DEV)
    empty = torch.empty(0, dtype=torch.int64, device=DEV)
    assert ops.gather_rows([x], empty)[0].shape == (0, 64)
    ops.gather_rows([], torch.arange(3, device=DEV))
    idx = torch.arange(4, device=DEV)
    with pytest.raises(RuntimeError, match="row shapes differ"):
        ops.gather_rows([x], idx, [torch.empty(4, 32, device=DEV)])
    with pytest.raises(RuntimeError, match="dtypes differ"):
        ops.gather_rows([x], idx, [torch.empty(4, 64, device=DEV, dtype=torch.float16)])
    with pytest.raises(RuntimeError, match="4 indices but only 2 rows"):
        ops.gather_rows([x], idx, [torch.empty(2, 64, device=DEV)])
    with pytest.raises(RuntimeError, match="int32 or int64"):
        ops.gather_rows([x], idx.to(torch.int16))
    with pytest.raises(RuntimeError, match="rows must be contiguous"):
        ops.gather_rows([x.t()], idx)
    with pytest.raises(RuntimeError, match="between 0 and 8 tensors"):
        ops.gather_rows([x] * 9, idx)


def test_c_abi_directly(ops):
    lib = _native.load()
    src = torch.arange(6 * 10, dtype=torch.int32, device=DEV).view(6, 10)
    dst = torch.zeros(3, 10, dtype=torch.int32, device=DEV)
    idx = torch.tensor([4, 0, 5], dtype=torch.int32, device=DEV)
    vp = lambda *p: (ctypes.c_void_p * len(p))(*p)
    i64 = lambda *v: (ctypes.c_int64 * len(v))(*v)
    rc = lib.arctic_gather_rows(1, vp(src.data_ptr()), vp(dst.data_ptr()), i64(40), i64(40), i64(40), idx.data_ptr(),
                                4, 3, 6, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(dst, src[idx.long()])
    assert lib.arctic_gather_rows(1, vp(src.data_ptr()), vp(dst.data_ptr()), i64(40), i64(40), i64(40), idx.data_ptr(),
                                  2, 3, 6, 0, None) == 2
    assert b"int32 or int64" in lib.arctic_last_error()


def test_random_configurations(ops):
    """Seeded sweep over tensor counts, element types, row lengths, pitches, start offsets (so that every unit
    size from 1 to 16 bytes is used) and index lists, gather and scatter."""
    import random
    rnd = random.Random(11)
    dtypes = [torch.uint8, torch.int16, torch.bfloat16, torch.float32, torch.int64]
    for it in range(40):
        g = torch.Generator().manual_seed(500 + it)
        rows = rnd.choice([1, 3, 40, 257])
        n_idx = rnd.choice([0, 1, 5, rows, rows + 7])
        tensors, dsrc = [], []
        for _ in range(rnd.choice([1, 2, 5, 8])):
            dt = rnd.choice(dtypes)
            cols, pad, off = rnd.choice([1, 3, 8, 33, 256, 1000]), rnd.choice([0, 0, 1, 8]), rnd.choice([0, 0, 1, 4])
            base = torch.randint(0, 127, (rows, off + cols + pad), generator=g).to(dt)
            tensors.append(base[:, off:off + cols])
            dsrc.append(base.to(DEV)[:, off:off + cols])
        idx = torch.randint(-1, rows + 1, (n_idx,), generator=g)         # a few out of range on both sides
        try:
            bufs = [sentinel_like(t, n_idx + 2) for t in tensors]
            want = oracle.gather_rows(tensors, idx, [b.clone() for b in bufs])
            got = ops.gather_rows(dsrc, idx.to(DEV), [b.to(DEV) for b in bufs])
            for k, (gk, wk) in enumerate(zip(got, want)):
                assert torch.equal(gk.cpu().view(torch.uint8), wk.view(torch.uint8)), f"gather: tensor {k} differs"
            # scatter the first rows of each tensor to distinct places of a sentinel-filled destination
            n_sc = min(rows, 6)
            perm = torch.randperm(rows + 3, generator=g)[:n_sc]
            dst = [sentinel_like(t, rows + 3) for t in tensors]
            ddst = [d.to(DEV) for d in dst]
            oracle.scatter_rows(tensors, perm, dst)
            ops.scatter_rows(dsrc, perm.to(DEV), ddst)
            for k, (gk, wk) in enumerate(zip(ddst, dst)):
                assert torch.equal(gk.cpu().view(torch.uint8), wk.view(torch.uint8)), f"scatter: tensor {k} differs"
        except AssertionError as e:
            raise AssertionError(f"configuration {it}: {[(t.dtype, tuple(t.shape), t.stride(0)) for t in tensors]}, "
                                 f"{n_idx} indices: {e}") from None
