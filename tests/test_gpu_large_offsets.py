"""The speculator operators, the argmax, the row gather, the fp4 cache write and the bulk write's source on tensors of
more than 2^32 bytes:
row offsets that no 32-bit product holds (the reference indexes rows with int64 throughout, e.g.
csrc/custom_ops/sum_lstm.cu:100-116, csrc/custom_ops/speculator_ln.cu:44-60).  The buffers are too large to bring to
the host whole, so the exact operators (argmax, gather) are compared with torch's own on the GPU, and the
floating-point ones with the CPU oracle on their first and last rows, which are independent of the rows between."""
import pytest
import torch

import oracle
from helpers import assert_close, speculator_alpha

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL, ATOL = 1e-2, 2e-2
EDGE = 48   # rows checked at each end


def randn_bf16(rows, cols, seed):
    """rows x cols of bf16 noise made on the GPU a slab at a time (an fp32 temporary of the whole would double it)."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    out = torch.empty(rows, cols, dtype=torch.bfloat16, device=DEV)
    step = max(1, (256 << 20) // cols)
    for r0 in range(0, rows, step):
        out[r0:r0 + step] = torch.randn(min(step, rows - r0), cols, generator=g, device=DEV).to(torch.bfloat16)
    return out


def edges(t):
    return torch.cat([t[:EDGE], t[-EDGE:]]).cpu()


def test_argmax_beyond_four_gib(ops):
    rows, vocab = 17_000, 128_256                      # 4.36 GB of logits
    logits = randn_bf16(rows, vocab, 11)
    assert logits.numel() * 2 > 1 << 32
    logits[-1, vocab - 1] = 100.0                      # the very last element of the buffer wins its row
    logits[-2, 0] = float("nan")
    got = ops.speculator_argmax(logits, vocab)
    want = torch.empty(rows, dtype=torch.int64, device=DEV)
    for r0 in range(0, rows, 2048):
        want[r0:r0 + 2048] = torch.argmax(logits[r0:r0 + 2048], dim=-1)
    assert torch.equal(got, want)
    assert int(got[-1]) == vocab - 1 and int(got[-2]) == 0


def test_gather_and_scatter_beyond_four_gib(ops):
    rows, width = 36_000, 65_536                       # 4.7 GB per tensor, 128 KiB rows
    big = randn_bf16(rows, width, 12)
    ids = torch.arange(rows, device=DEV)               # a second, narrow tensor in the same launch
    g = torch.Generator().manual_seed(12)
    idx = torch.cat([torch.tensor([rows - 1, 0, rows - 2]), torch.randint(0, rows, (253,), generator=g)]).to(DEV)
    out_big = torch.zeros(idx.numel() + 3, width, dtype=torch.bfloat16, device=DEV)
    out_ids = torch.full((idx.numel() + 3,), -7, dtype=torch.int64, device=DEV)
    ops.gather_rows([big, ids], idx, [out_big, out_ids])
    assert torch.equal(out_big[:idx.numel()], big.index_select(0, idx))
    assert torch.equal(out_ids[:idx.numel()], idx) and bool((out_ids[idx.numel():] == -7).all())
    assert not out_big[idx.numel():].any()
    # the way back: distinct rows of a small tensor into the large one
    target = torch.randperm(rows, generator=g)[:256]
    target[0], target[1] = rows - 1, 0
    target = target.to(DEV)
    before = big[target].clone()
    small = randn_bf16(256, width, 13)
    checksum = big.view(torch.int16).sum(dtype=torch.int64)
    ops.scatter_rows([small], target, [big])
    assert torch.equal(big[target], small)
    moved = (small.view(torch.int16).sum(dtype=torch.int64) - before.view(torch.int16).sum(dtype=torch.int64))
    assert int(big.view(torch.int16).sum(dtype=torch.int64)) == int(checksum + moved)   # no other row changed


def test_sum_lstm_beyond_four_gib(ops):
    rows, D = 140_000, 4096                            # states and z4: 4.6 GB each
    states, z4 = randn_bf16(rows, 4 * D, 14), randn_bf16(rows, 4 * D, 15)
    assert states.numel() * 2 > 1 << 32
    cell = randn_bf16(rows, D, 16)
    g = torch.Generator().manual_seed(17)
    vec = lambda m: (m + 0.02 * torch.randn(D, generator=g)).to(torch.bfloat16)
    w_cell, b_cell, w_state, b_state = vec(1.0), vec(0.0), vec(1.0), vec(0.0)
    alpha = speculator_alpha(3, D)
    got_s, got_c = ops.sum_lstm(states, z4, cell, w_cell.to(DEV), b_cell.to(DEV), w_state.to(DEV), b_state.to(DEV),
                                alpha, 1e-6, 1e-6, False)
    want_s, want_c = oracle.sum_lstm(edges(states), edges(z4), edges(cell), w_cell, b_cell, w_state, b_state, alpha,
                                     1e-6, 1e-6, False)
    assert_close(edges(got_c), want_c, RTOL, ATOL, "cell")
    assert_close(edges(got_s), want_s, RTOL, ATOL, "state")
    # every row was written: with these inputs no output row is all zero
    for out in (got_s, got_c):
        assert bool(out.view(torch.int16).ne(0).any(dim=1).all())


def test_speculator_ln_beyond_four_gib(ops):
    rows, hidden = 270_000, 8192                       # 4.4 GB in, 4.4 GB out
    x = randn_bf16(rows, hidden, 18)
    assert x.numel() * 2 > 1 << 32
    g = torch.Generator().manual_seed(19)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(torch.bfloat16)
    b = (0.1 * torch.randn(hidden, generator=g)).to(torch.bfloat16)
    got = ops.speculator_ln(x, w.to(DEV), b.to(DEV), 1e-6)
    assert_close(edges(got), oracle.speculator_ln(edges(x), w, b, 1e-6), RTOL, ATOL, "speculator_ln")
    assert bool(got.view(torch.int16).ne(0).any(dim=1).all())


def test_fp4_write_source_beyond_four_gib(ops):
    T, H, D, bs = 2_200_000, 8, 128, 16                # K and V: 4.5 GB each; packed caches 1.1 GB, scales 141 MB
    NB = (T + bs - 1) // bs
    key, value = randn_bf16(T, H * D, 20).view(T, H, D), randn_bf16(T, H * D, 21).view(T, H, D)
    assert key.numel() * 2 > 1 << 32
    g = torch.Generator().manual_seed(22)
    slots = torch.randperm(NB * bs, generator=g)[:T]
    slots[5::97] = -1
    kc, vc = (torch.full((NB, bs, H, D // 2), 0xA5, dtype=torch.uint8, device=DEV) for _ in range(2))
    ks, vs = (torch.full((NB, bs, H, D // 16), 0xA5, dtype=torch.uint8, device=DEV) for _ in range(2))
    zero = torch.zeros((), device=DEV)
    ops.reshape_and_cache_flash_fp4(key, value, kc, vc, ks, vs, slots.to(DEV), "fp4", zero, zero)
    # the first and the last tokens against the oracle, which writes them into a pool just large enough
    pick = torch.cat([torch.arange(2048), torch.arange(T - 2048, T)])
    sub_slots = slots[pick]
    valid = sub_slots >= 0
    remap = torch.full_like(sub_slots, -1)
    remap[valid] = torch.arange(int(valid.sum()))
    nb = (int(valid.sum()) + bs - 1) // bs
    okc, ovc = (torch.zeros(nb, bs, H, D // 2, dtype=torch.uint8) for _ in range(2))
    oks, ovs = (torch.zeros(nb, bs, H, D // 16, dtype=torch.uint8) for _ in range(2))
    z = torch.tensor(0.0)
    oracle.reshape_and_cache_flash_fp4(key[pick.to(DEV)].cpu(), value[pick.to(DEV)].cpu(), okc, ovc, oks, ovs, remap,
                                       "fp4", z, z)
    at = sub_slots[valid].to(DEV)
    n = int(valid.sum())
    for got, want, name in ((kc, okc, "key cache"), (vc, ovc, "value cache"), (ks, oks, "key scales"),
                            (vs, ovs, "value scales")):
        rows = got.view(NB * bs, -1)[at].cpu()
        assert torch.equal(rows, want.view(nb * bs, -1)[:n]), name
    # rows that no valid slot names keep their sentinel; all others lost it
    written = torch.zeros(NB * bs, dtype=torch.bool)
    written[slots[slots >= 0]] = True
    for c in (kc, ks):
        clean = (c.view(NB * bs, -1) == 0xA5).all(dim=1)
        assert torch.equal(clean.cpu(), ~written)


def test_bulk_write_source_beyond_four_gib(ops):
    """keys / values of 4.6 GB each (70 000 tokens x 32 layers x 1024): token rows whose byte offsets pass 2^32, the
    caches of ordinary size.  Every cache row that no valid slot names keeps its sentinel; the first and the last
    tokens' rows equal what the oracle writes for them into a pool just large enough."""
    T, L, H, D, bs = 70_000, 32, 8, 128, 16
    n, NB = H * D, (70_000 + 15) // 16 + 7
    keys, values = randn_bf16(T, L * n, 23), randn_bf16(T, L * n, 24)
    assert keys.numel() * 2 > 1 << 32
    g = torch.Generator().manual_seed(25)
    slots = torch.randperm(NB * bs, generator=g)[:T]
    slots[3::53] = -1
    bufs = [torch.full((2, NB, bs, H, D), 0xA5, dtype=torch.uint8, device=DEV) for _ in range(L)]
    kc, vc = [b[0] for b in bufs], [b[1] for b in bufs]
    ks = [torch.tensor(0.011 + 0.001 * l, device=DEV) for l in range(L)]
    vs = [torch.tensor(0.013 + 0.001 * l, device=DEV) for l in range(L)]
    ops.reshape_and_cache_flash_bulk(keys, values, kc, vc, slots.to(DEV), "fp8", ks, vs, H, D)
    written = torch.zeros(NB * bs, dtype=torch.bool)
    written[slots[slots >= 0]] = True
    dwritten = written.to(DEV)
    for c in kc + vc:
        assert torch.equal((c.view(NB * bs, n) == 0xA5).all(dim=1), ~dwritten)
    pick = torch.cat([torch.arange(1024), torch.arange(T - 1024, T)])
    sub = slots[pick]
    valid = sub >= 0
    count = int(valid.sum())
    remap = torch.full_like(sub, -1)
    remap[valid] = torch.arange(count)
    obufs = [torch.zeros(2, (count + bs - 1) // bs, bs, H, D, dtype=torch.uint8) for _ in range(L)]
    oracle.reshape_and_cache_flash_bulk(keys[pick.to(DEV)].cpu(), values[pick.to(DEV)].cpu(), [b[0] for b in obufs],
                                        [b[1] for b in obufs], remap, "fp8", [s.cpu() for s in ks], [s.cpu() for s in vs],
                                        H, D)
    at = sub[valid].to(DEV)
    for l in range(L):
        for which, c in enumerate((kc[l], vc[l])):
            assert torch.equal(c.view(NB * bs, n)[at].cpu(), obufs[l][which].view(-1, n)[:count]), f"layer {l}"
