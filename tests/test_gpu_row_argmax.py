"""GPU parity of speculator_argmax (torch.argmax(logits, -1).clamp_(0, vocab_size - 1),
arctic_speculator.py:846-848, 862) against torch itself: exact indices."""
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def reference(logits, vocab_size):
    # the reference's expression, on the CPU in fp32 (every 16-bit value is exact in fp32, so the order and
    # the ties are the same)
    return torch.argmax(logits.float().cpu(), dim=-1).clamp_(0, vocab_size - 1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("shape", [(512, 128256), (64, 32000), (7, 513), (3, 5, 1000), (9, 1), (2, 7), (33, 4100)])
def test_random_logits(ops, dtype, shape):
    g = torch.Generator().manual_seed(5)
    logits = torch.randn(*shape, generator=g).to(dtype)          # bf16 makes many exact ties
    got = ops.speculator_argmax(logits.to(DEV), shape[-1])
    assert got.dtype == torch.int64 and got.shape == logits.shape[:-1]
    assert torch.equal(got.cpu(), reference(logits, shape[-1]))
    # the GPU's own torch.argmax agrees as well
    assert torch.equal(got, torch.argmax(logits.to(DEV), dim=-1))


def test_ties_take_the_lowest_index(ops):
    x = torch.zeros(6, 5000, dtype=torch.bfloat16)
    x[1, 4097], x[1, 77], x[1, 4999] = 3.0, 3.0, 3.0
    x[2] = -float("inf")                                            # a row of -inf answers 0
    x[3, 100] = -0.0                                                 # -0 == +0: still index 0
    x[4, 17], x[4, 2050] = float("inf"), float("inf")
    x[5, 4999] = 1.0
    got = ops.speculator_argmax(x.to(DEV), 5000).cpu()
    assert got.tolist() == [0, 77, 0, 0, 17, 4999]
    assert torch.equal(got, reference(x, 5000))


def test_nan_beats_every_number_and_the_first_nan_wins(ops):
    g = torch.Generator().manual_seed(6)
    x = torch.randn(5, 9000, generator=g)
    x[0, 8000] = float("nan")
    x[1, 5], x[1, 8999] = float("nan"), float("nan")
    x[2, 3000], x[2, 10] = float("nan"), float("inf")
    x[3, 100], x[3, 101] = float("inf"), -float("inf")              # a chunk sum that is NaN without any NaN in it
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        xs = x.to(dtype)
        got = ops.speculator_argmax(xs.to(DEV), 9000).cpu()
        assert got[:4].tolist() == [8000, 5, 3000, 100]
        assert torch.equal(got, reference(xs, 9000))


def test_clamp_and_row_pitch(ops):
    g = torch.Generator().manual_seed(7)
    full = torch.randn(40, 1100, generator=g).to(torch.bfloat16).to(DEV)
    for view in (full[:, :1000], full[:, 4:1003], full[::2, :999]):   # aligned pitch, odd start, skipped rows
        got = ops.speculator_argmax(view, 1000)
        assert torch.equal(got, torch.argmax(view.float(), dim=-1).clamp_(0, 999))
    # logits wider than the vocabulary (padded head): indices beyond it are clamped
    padded = torch.zeros(4, 1024, dtype=torch.float16, device=DEV)
    padded[:, 1010] = 5.0
    assert ops.speculator_argmax(padded, 1000).tolist() == [999] * 4


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_rows_that_start_between_16_byte_boundaries(ops, dtype):
    """A contiguous [rows, vocab] with an odd vocabulary (GPT-2's 50257) puts every row at another offset from a
    16-byte boundary: the elements in front of the first boundary, the 16-byte chunks and the elements behind the
    last chunk are three stretches of one row, and the lowest index among equal values may lie in any of them."""
    rows, cols = 24, 50257
    g = torch.Generator().manual_seed(8)
    x = (torch.randint(0, 9, (rows, cols), generator=g).float() - 4).to(dtype)      # ties everywhere
    x[1, :] = -float("inf")                        # answers 0, which lies in front of row 1's first boundary
    x[2, 0] = 50.0                                 # the very first element wins
    x[3, 1], x[3, 9000] = 50.0, 50.0               # equal values in front of the boundary and in a chunk
    x[4, cols - 1], x[4, 30000] = 50.0, 50.0       # ... in a chunk and behind the last chunk
    x[5, cols - 1] = 50.0                          # the very last element wins
    x[6, 2], x[6, 40000] = float("nan"), float("nan")   # the first NaN lies in front of the boundary
    x[7, 3], x[7, 4] = float("inf"), float("nan")
    d = x.to(DEV)
    assert d.data_ptr() % 16 == 0 and (cols * x.element_size()) % 16 != 0
    got = ops.speculator_argmax(d, cols)
    assert torch.equal(got.cpu(), reference(x, cols))
    assert got[[1, 2, 3, 4, 5, 6, 7]].tolist() == [0, 0, 1, 30000, cols - 1, 2, 4]
    # a view that starts one element into such a buffer, and one row alone
    view = d[:, 1:]
    assert torch.equal(ops.speculator_argmax(view, cols - 1).cpu(), reference(x[:, 1:], cols - 1))
    assert torch.equal(ops.speculator_argmax(d[5:6, 3:], cols).cpu(), reference(x[5:6, 3:], cols))


def test_empty_and_errors(ops):
    assert ops.speculator_argmax(torch.empty(0, 64, device=DEV), 64).shape == (0,)
    with pytest.raises(RuntimeError, match="non-empty last dimension"):
        ops.speculator_argmax(torch.empty(4, 0, device=DEV), 1)
    with pytest.raises(RuntimeError, match="fp32, fp16 or bf16"):
        ops.speculator_argmax(torch.zeros(4, 8, dtype=torch.float64, device=DEV), 8)
    with pytest.raises(RuntimeError, match="last dimension must be contiguous"):
        ops.speculator_argmax(torch.zeros(8, 4, device=DEV).t(), 8)


def test_random_configurations(ops):
    """Seeded sweep over types, row counts, row lengths around the chunk and workgroup sizes, row pitches, start
    offsets (rows that start between two 16-byte boundaries read their first elements one by one), value ranges with many ties, and sprinkled NaN / inf."""
    import random
    rnd = random.Random(13)
    for it in range(60):
        g = torch.Generator().manual_seed(700 + it)
        dtype = rnd.choice([torch.bfloat16, torch.float16, torch.float32])
        rows = rnd.choice([1, 2, 17, 130])
        cols = rnd.choice([1, 2, 7, 8, 9, 63, 64, 65, 255, 256, 257, 1023, 1025, 4096, 8200, 33000])
        pad, off = rnd.choice([0, 0, 1, 8, 24]), rnd.choice([0, 0, 1, 3, 8])
        levels = rnd.choice([2, 5, 1000])                 # few distinct values: ties everywhere
        base = torch.randint(0, levels, (rows, off + cols + pad), generator=g).float() - levels / 2
        for special in (float("nan"), float("inf"), -float("inf")):
            if rnd.random() < 0.3:
                r, c = rnd.randrange(rows), rnd.randrange(off + cols + pad)
                base[r, c] = special
        base = base.to(dtype)
        logits = base[:, off:off + cols]
        vocab = rnd.choice([cols, max(1, cols - 3), cols + 5])
        got = ops.speculator_argmax(base.to(DEV)[:, off:off + cols], vocab)
        want = torch.argmax(logits.float(), dim=-1).clamp_(0, vocab - 1)
        assert torch.equal(got.cpu(), want), f"configuration {it}: {dtype}, {rows} x {cols}, pad {pad}, offset {off}"


@pytest.mark.parametrize("rows", [257, 300, 768, 769])   # 257-768 rows take the kernel whose waves move in step
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_row_counts_around_the_in_step_kernel(ops, rows, dtype):
    """Launches of 257 to 768 rows keep the waves of a row in step, a 16-byte chunk at a time, behind a barrier whose
    trip count has to be the same for every wave whatever the row length: rows shorter than one chunk per lane, rows
    with a ragged last batch and an element-wise tail, ties everywhere, NaN and infinities, pitched rows."""
    g = torch.Generator().manual_seed(900 + rows)
    for cols, pad in ((8, 0), (1000, 8), (4100, 0), (8200, 24), (33001, 7)):
        base = (torch.randint(0, 7, (rows, cols + pad), generator=g).float() - 3)
        base[rows // 2, cols // 2] = float("nan")
        base[rows - 1, 0] = float("inf")
        base[0, cols - 1] = float("inf")
        base[1] = -float("inf")
        base = base.to(dtype)
        got = ops.speculator_argmax(base.to(DEV)[:, :cols], cols)
        want = torch.argmax(base[:, :cols].float(), dim=-1)
        assert torch.equal(got.cpu(), want), f"{rows} x {cols} (+{pad}), {dtype}"
