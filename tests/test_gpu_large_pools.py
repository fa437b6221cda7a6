"""The bulk KV-cache write at the pool sizes a serving process has (vLLM gives each layer GiB of cache,
arctic_inference/vllm/swiftkv/llama_swiftkv.py:600-615): rows whose element and byte offsets lie beyond 2^31 and 2^32
(the reference indexes the cache with an int64, csrc/custom_ops/reshape_and_cache_flash_bulk.cu:27-48), and the
decode-step workload at its full size in one HIP graph.  Too large for whole-buffer comparisons on the host, so the
caches are checked through size-independent properties: every row that no valid slot addresses keeps its sentinel,
and every written row is compared with the CPU oracle run on a compacted pool."""
import pytest
import torch

import oracle
from helpers import assert_close, make_lstm_case, speculator_alpha

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SENTINEL = 0xA5


def check_pool(bufs, key_caches, value_caches, slots, keys, values, kv, k_scales, v_scales, H, D, NB, bs):
    """`bufs` were filled with the sentinel byte before the write.  (1) rows that no valid slot names are untouched,
    rows that one names are not; (2) the written rows equal the oracle's, which writes the same tokens into a pool
    just large enough for them."""
    n = H * D
    L = len(key_caches)
    valid = slots >= 0
    written = torch.zeros(NB * bs, dtype=torch.bool)
    written[slots[valid]] = True
    dwritten = written.to(DEV)
    for l in range(L):
        for c in (key_caches[l], value_caches[l]):
            if c.is_contiguous():
                rows = c.view(NB * bs, -1).view(torch.uint8)
                clean = torch.empty(NB * bs, dtype=torch.bool, device=DEV)
                for r0 in range(0, NB * bs, 1 << 20):    # in pieces: a comparison result is as large as its input
                    clean[r0:r0 + (1 << 20)] = (rows[r0:r0 + (1 << 20)] == SENTINEL).all(dim=1)
            else:                                        # FlashInfer view [NB, bs, H, D] of [NB, 2, bs, H, D]
                clean = torch.empty(NB, bs, dtype=torch.bool, device=DEV)
                for b0 in range(0, NB, 1 << 16):
                    piece = c[b0:b0 + (1 << 16)].reshape(-1, bs, n).view(torch.uint8)
                    clean[b0:b0 + (1 << 16)] = (piece == SENTINEL).all(dim=2)
                clean = clean.view(-1)
            assert torch.equal(clean, ~dwritten), f"layer {l}: the set of touched rows is not the set of valid slots"
    nvalid = int(valid.sum())
    remap = torch.full_like(slots, -1)
    remap[valid] = torch.arange(nvalid)
    cache_dtype = torch.uint8 if kv != "auto" else keys.dtype
    obufs = [torch.zeros(2, (nvalid + bs - 1) // bs, bs, H, D, dtype=cache_dtype) for _ in range(L)]
    oracle.reshape_and_cache_flash_bulk(keys.cpu(), values.cpu(), [b[0] for b in obufs], [b[1] for b in obufs], remap, kv,
                                        [s.cpu() for s in k_scales], [s.cpu() for s in v_scales], H, D)
    rows_of = slots[valid].to(DEV)
    blk, off = rows_of // bs, rows_of % bs
    for l in range(L):
        for which, c in enumerate((key_caches[l], value_caches[l])):
            got = c[blk, off].reshape(nvalid, n).cpu()
            want = obufs[l][which].view(-1, n)[:nvalid]
            assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), f"layer {l} {'KV'[which]}: written rows differ"


def edge_slots(T, NB, bs, g, edge_blocks=1000, pad_every=11):
    """T distinct slots from the first and the last `edge_blocks` blocks of the pool, some tokens padding."""
    lo = 1 + torch.randperm(edge_blocks * bs - 1, generator=g)[: T // 2]
    hi = (NB - edge_blocks) * bs + torch.randperm(edge_blocks * bs - 1, generator=g)[: T - T // 2]
    slots = torch.cat([lo, hi])[torch.randperm(T, generator=g)].to(torch.int64)
    slots[::pad_every] = -1
    slots[0] = NB * bs - 1            # the very last row of the pool
    slots[1] = 0                      # and the very first
    return slots


@pytest.mark.parametrize("kv,layout,L", [("fp8", "flash", 2), ("auto", "flashinfer", 1), ("auto", "flash", 1)])
def test_cache_halves_beyond_four_gib(ops, kv, layout, L):
    """300 000 blocks of 16 x 8 x 128: 4.9 GB per K half as fp8 codes, 9.8 GB as bf16; with the FlashInfer layout the
    block stride doubles, so element offsets pass 2^32 as well."""
    T, H, D, bs, NB = 4096, 8, 128, 16, 300_000
    n = H * D
    g = torch.Generator().manual_seed(7)
    keys = (torch.randn(T, L * n, generator=g) * 1.5).to(torch.bfloat16).to(DEV)
    values = (torch.randn(T, L * n, generator=g) * 1.5).to(torch.bfloat16).to(DEV)
    slots = edge_slots(T, NB, bs, g)
    cache_dtype = torch.uint8 if kv == "fp8" else torch.bfloat16
    shape = (2, NB, bs, H, D) if layout == "flash" else (NB, 2, bs, H, D)
    bufs, kc, vc = [], [], []
    for _ in range(L):
        raw = torch.full((2 * NB * bs * n * (1 if kv == "fp8" else 2),), SENTINEL, dtype=torch.uint8, device=DEV)
        buf = raw.view(cache_dtype).view(shape)
        bufs.append(buf)
        kc.append(buf[0] if layout == "flash" else buf[:, 0])
        vc.append(buf[1] if layout == "flash" else buf[:, 1])
    assert kc[0].numel() * kc[0].element_size() > (1 << 32)
    ks = [(keys[:, l * n:(l + 1) * n].float().abs().max() / 448.0) for l in range(L)]
    vs = [(values[:, l * n:(l + 1) * n].float().abs().max() / 448.0) for l in range(L)]
    print(f"bulk write into a {NB}-block pool, {kv}, {layout}, {L} layers", flush=True)
    ops.reshape_and_cache_flash_bulk(keys, values, kc, vc, slots.to(DEV), kv, ks, vs, H, D)
    torch.cuda.synchronize()
    check_pool(bufs, kc, vc, slots, keys, values, kv, ks, vs, H, D, NB, bs)


def test_slots_beyond_two_to_the_31(ops):
    """block_size 1 and tiny rows: slot numbers themselves pass 2^31 (the kernel's 64-bit slot division)."""
    T, L, H, D, bs = 512, 1, 1, 16, 1
    NB = (1 << 31) + 4096
    n = H * D
    g = torch.Generator().manual_seed(8)
    keys = torch.randn(T, L * n, generator=g).to(torch.bfloat16).to(DEV)
    values = torch.randn(T, L * n, generator=g).to(torch.bfloat16).to(DEV)
    pool = torch.full((2, NB, bs, H, D), SENTINEL, dtype=torch.uint8, device=DEV)     # 2 x 34 GB
    kc, vc = [pool[0]], [pool[1]]
    slots = torch.cat([torch.randperm(4096, generator=g)[: T // 2], (1 << 31) + torch.randperm(4095, generator=g)[: T // 2]])
    slots = slots[torch.randperm(T, generator=g)].to(torch.int64)
    slots[::7] = -1
    slots[3] = NB - 1
    ks, vs = [torch.tensor(0.01, device=DEV)], [torch.tensor(0.03, device=DEV)]
    print("bulk write with slots beyond 2^31", flush=True)
    ops.reshape_and_cache_flash_bulk(keys, values, kc, vc, slots.to(DEV), "fp8", ks, vs, H, D)
    torch.cuda.synchronize()
    # property (1) on the edges only (the middle 2^31 rows cannot be named by any slot drawn above)
    valid = slots >= 0
    for c in kc + vc:
        for lo, hi in ((0, 4096), (1 << 31, NB)):
            written = torch.zeros(hi - lo, dtype=torch.bool)
            sel = valid & (slots >= lo) & (slots < hi)
            written[slots[sel] - lo] = True
            clean = (c[lo:hi].reshape(hi - lo, n) == SENTINEL).all(dim=1)
            assert torch.equal(clean.cpu(), ~written)
        assert bool((c[4096:1 << 20] == SENTINEL).all()) and bool((c[(1 << 31) - (1 << 20):1 << 31] == SENTINEL).all())
    nvalid = int(valid.sum())
    remap = torch.full_like(slots, -1)
    remap[valid] = torch.arange(nvalid)
    obufs = [torch.zeros(2, nvalid, bs, H, D, dtype=torch.uint8) for _ in range(L)]
    oracle.reshape_and_cache_flash_bulk(keys.cpu(), values.cpu(), [b[0] for b in obufs], [b[1] for b in obufs], remap, "fp8",
                                        [s.cpu() for s in ks], [s.cpu() for s in vs], H, D)
    rows_of = slots[valid].to(DEV)
    for l in range(L):
        for which, c in enumerate((kc[l], vc[l])):
            assert torch.equal(c[rows_of].reshape(nvalid, n).cpu(), obufs[l][which].view(-1, n))


def test_decode_step_at_full_size_in_one_graph(ops):
    """The decode-step mix as specified: 512 tokens; fp8 bulk write over 16 layers into 32 768-block caches
    (32 x 537 MB); ln0 without scale / shift on [512, 4096]; three chained sum_lstm steps at 4096; all in one HIP
    graph, replayed twice with the caches reset in between.  Each replay: cache properties + oracle on the written
    rows, ln0 and every LSTM step within the path's tolerance of the oracle, and equal to the eager run bit for bit."""
    T, L, H, D, bs, NB, W = 512, 16, 8, 128, 16, 32768, 4096
    n = H * D
    g = torch.Generator().manual_seed(4)
    keys = (torch.randn(T, L * n, generator=g) * 1.5).to(torch.bfloat16).to(DEV)
    values = (torch.randn(T, L * n, generator=g) * 1.5).to(torch.bfloat16).to(DEV)
    slots = torch.randperm(NB * bs, generator=g)[:T].to(torch.int64)
    slots[5::37] = -1
    dslots = slots.to(DEV)
    bufs = [torch.full((2, NB, bs, H, D), SENTINEL, dtype=torch.uint8, device=DEV) for _ in range(L)]
    kc, vc = [b[0] for b in bufs], [b[1] for b in bufs]
    ks = [(keys[:, l * n:(l + 1) * n].float().abs().max() / 448.0) for l in range(L)]
    vs = [(values[:, l * n:(l + 1) * n].float().abs().max() / 448.0) for l in range(L)]
    steps = [make_lstm_case(rows=T, D=W, seed=40 + k) for k in range(3)]
    dsteps = [{k: (None if v is None else v.to(DEV)) for k, v in s.items()} for s in steps]
    x = torch.randn(T, W, generator=g).to(torch.bfloat16)
    dx = x.to(DEV)
    alpha = speculator_alpha(3, W)

    def step():
        ops.reshape_and_cache_flash_bulk(keys, values, kc, vc, dslots, "fp8", ks, vs, H, D)
        h = ops.speculator_ln(dx, None, None, 1e-6)
        cell = torch.zeros(T, W, dtype=torch.bfloat16, device=DEV)
        states, cells = [], []
        for s in dsteps:
            st, cell = ops.sum_lstm(s["states"], s["z4"], cell, s["w_cell"], s["b_cell"], s["w_state"], s["b_state"],
                                    alpha, 1e-6, 1e-6, False)
            states.append(st)
            cells.append(cell)
        return [h] + states + cells

    print("decode step at full size: eager", flush=True)
    eager = [t.clone() for t in step()]
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    want_h = oracle.speculator_ln(x, None, None, 1e-6)
    for replay in range(2):
        for b in bufs:
            b.fill_(SENTINEL)
        for t in outs:
            t.zero_()
        torch.cuda.synchronize()
        print(f"decode step at full size: replay {replay}", flush=True)
        graph.replay()
        torch.cuda.synchronize()
        check_pool(bufs, kc, vc, slots, keys, values, "fp8", ks, vs, H, D, NB, bs)
        for a, e in zip(outs, eager):
            assert torch.equal(a, e), f"replay {replay} differs from the eager run"
        assert_close(outs[0], want_h, what="ln0")
        prev = torch.zeros(T, W, dtype=torch.bfloat16)
        for k, s in enumerate(steps):
            want_st, want_cell = oracle.sum_lstm(s["states"], s["z4"], prev, s["w_cell"], s["b_cell"], s["w_state"],
                                                 s["b_state"], alpha, 1e-6, 1e-6, False)
            assert_close(outs[1 + k], want_st, what=f"state {k}")
            assert_close(outs[4 + k], want_cell, what=f"cell {k}")
            prev = outs[4 + k].cpu()          # chain through the GPU's own cell: only this step's arithmetic is compared
