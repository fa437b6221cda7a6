"""GPU parity of sum_lstm against the CPU oracle (1e-2 rel / 2e-2 abs)."""
import pytest
import torch

import oracle
from helpers import assert_close, make_lstm_case, speculator_alpha, to_device_pitched

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL, ATOL = 1e-2, 2e-2


def dev(t):
    return None if t is None else to_device_pitched(t, DEV)


def run(ops, c, alpha, eps_cell=1e-6, eps_state=1e-6, fast=False):
    got_s, got_c = ops.sum_lstm(dev(c["states"]), dev(c["z4"]), dev(c["prev_cell"]), dev(c["w_cell"]),
                                dev(c["b_cell"]), dev(c["w_state"]), dev(c["b_state"]), alpha, eps_cell,
                                eps_state, fast)
    torch.cuda.synchronize()
    want_s, want_c = oracle.sum_lstm(c["states"], c["z4"], c["prev_cell"], c["w_cell"], c["b_cell"],
                                     c["w_state"], c["b_state"], alpha, eps_cell, eps_state, fast)
    pc = c["prev_cell"]
    for got in (got_s, got_c):
        assert got.shape == pc.shape and got.dtype == pc.dtype
        if pc.size(0) > 1:                           # (the pitch of a single row is not defined)
            assert got.stride() == pc.stride()      # outputs inherit prev_cell's row pitch
    assert_close(got_c, want_c, RTOL, ATOL, "cell")
    assert_close(got_s, want_s, RTOL, ATOL, "state")
    return got_s, got_c, want_s, want_c


# the reference's cases (tests/unit_tests/test_sum_lstm.py:174-179): pad4=7/padD=3 forces the element-wise kernel
@pytest.mark.parametrize("cfg", [
    dict(rows=1, D=64, pad4=0, padD=0),
    dict(rows=4, D=128, pad4=7, padD=3),
    dict(rows=32, D=256, pad4=0, padD=0),
    dict(rows=64, D=512, pad4=16, padD=8),
    dict(rows=3, D=12, pad4=0, padD=0),
    dict(rows=2, D=8200, pad4=0, padD=0),
    dict(rows=2, D=16392, pad4=0, padD=0),
])
@pytest.mark.parametrize("wb_cell", [True, False])
@pytest.mark.parametrize("wb_state", [True, False])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_reference_cases(ops, cfg, wb_cell, wb_state, dtype):
    c = make_lstm_case(dtype=dtype, seed=1234, wb_cell=wb_cell, wb_state=wb_state, repeat_z=True, **cfg)
    run(ops, c, alpha=0.35)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_fast_gelu(ops, dtype):
    c = make_lstm_case(rows=16, D=512, dtype=dtype, seed=5)
    run(ops, c, alpha=0.35, fast=True)


@pytest.mark.parametrize("alpha", [speculator_alpha(3, 4096), 1.0])
def test_config4_three_steps(ops, alpha):
    """The speculator benchmark shape: T=512, H=4096, bf16, 3 chained steps (cell_{k+1} = out_cell_k,
    fresh pre-activations per step)."""
    cell_gpu = cell_cpu = None
    for step in range(3):
        c = make_lstm_case(rows=512, D=4096, seed=3 + 10 * step)
        if step:
            # both sides continue from the oracle's cell so that one step's rounding
            # differences are not fed through the next
            c["prev_cell"] = cell_cpu
        got_s, got_c, want_s, want_c = run(ops, c, alpha=alpha)
        cell_cpu = want_c
        same = (got_c.cpu().view(torch.int16) == want_c.view(torch.int16)).float().mean().item()
        assert same > 0.97, f"step {step}: only {same:.4f} of the cells are bit-identical to the oracle"


@pytest.mark.parametrize("cfg", [dict(rows=64, D=512, pad4=16, padD=8), dict(rows=4, D=128, pad4=7, padD=3),
                                 dict(rows=512, D=4096, pad4=0, padD=0), dict(rows=3, D=8200, pad4=0, padD=0)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_shared_z_equals_repeated_z(ops, cfg, dtype):
    """sum_lstm_shared_z(states, z) must give the very bits of sum_lstm(states, z.repeat(1, 4)),
    and both must match the oracle run on the repeated tensor."""
    c = make_lstm_case(dtype=dtype, seed=99, repeat_z=True, **cfg)
    D = cfg["D"]
    z = c["z4"][:, :D].contiguous()
    assert torch.equal(c["z4"], z.repeat(1, 4))
    alpha = 0.35
    args = [dev(c[k]) for k in ("prev_cell", "w_cell", "b_cell", "w_state", "b_state")]
    st_r, ce_r = ops.sum_lstm(dev(c["states"]), dev(c["z4"]), *args, alpha, 1e-6, 1e-6, False)
    st_s, ce_s = ops.sum_lstm_shared_z(dev(c["states"]), z.to(DEV), *args, alpha, 1e-6, 1e-6, False)
    torch.cuda.synchronize()
    assert st_s.stride() == c["prev_cell"].stride()
    assert torch.equal(st_s, st_r) and torch.equal(ce_s, ce_r)
    want_s, want_c = oracle.sum_lstm(c["states"], c["z4"], c["prev_cell"], c["w_cell"], c["b_cell"], c["w_state"],
                                     c["b_state"], alpha, 1e-6, 1e-6, False)
    assert_close(ce_s, want_c, RTOL, ATOL, "cell (shared z)")
    assert_close(st_s, want_s, RTOL, ATOL, "state (shared z)")


@pytest.mark.parametrize("cfg", [dict(rows=512, D=4096, pad4=0, padD=0, vocab=32000, table_pad=0),
                                 dict(rows=33, D=512, pad4=16, padD=8, vocab=100, table_pad=8),
                                 dict(rows=5, D=100, pad4=0, padD=0, vocab=7, table_pad=3),     # element-wise kernel
                                 dict(rows=1, D=8200, pad4=0, padD=0, vocab=3, table_pad=0)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_embedded_equals_lookup_then_shared_z(ops, cfg, dtype):
    """sum_lstm_embedded(states, table, ids) must give the very bits of
    sum_lstm_shared_z(states, table[ids.clamp(0, V - 1)]): forget_emb(last_tokens) with the caller's clamp
    (arctic_speculator.py:744, 845, 862); ids outside the table included."""
    cfg = dict(cfg)
    vocab, table_pad = cfg.pop("vocab"), cfg.pop("table_pad")
    c = make_lstm_case(dtype=dtype, seed=123, **cfg)
    D, rows = cfg["D"], cfg["rows"]
    g = torch.Generator().manual_seed(5)
    table = torch.randn(vocab, D + table_pad, generator=g).to(dtype)[:, :D]
    ids = torch.randint(0, vocab, (rows, 1), generator=g)
    ids[0, 0] = -3
    ids[-1, 0] = vocab + 5
    z = torch.nn.functional.embedding(ids.clamp(0, vocab - 1), table).flatten(0, 1)
    alpha = speculator_alpha(3, D)
    args = [dev(c[k]) for k in ("prev_cell", "w_cell", "b_cell", "w_state", "b_state")]
    dtable = to_device_pitched(table, DEV)
    assert dtable.stride(0) == D + table_pad
    st_e, ce_e = ops.sum_lstm_embedded(dev(c["states"]), dtable, ids.to(DEV), *args, alpha, 1e-6, 1e-6, False)
    st_s, ce_s = ops.sum_lstm_shared_z(dev(c["states"]), z.to(DEV), *args, alpha, 1e-6, 1e-6, False)
    torch.cuda.synchronize()
    assert st_e.stride() == c["prev_cell"].stride()
    assert torch.equal(st_e, st_s) and torch.equal(ce_e, ce_s)
    want_s, want_c = oracle.sum_lstm(c["states"], z.repeat(1, 4), c["prev_cell"], c["w_cell"], c["b_cell"],
                                     c["w_state"], c["b_state"], alpha, 1e-6, 1e-6, False)
    assert_close(ce_e, want_c, RTOL, ATOL, "cell (embedded z)")
    assert_close(st_e, want_s, RTOL, ATOL, "state (embedded z)")


def test_embedded_errors(ops):
    bf = dict(dtype=torch.bfloat16, device=DEV)
    s, pc, table = torch.randn(4, 256, **bf), torch.randn(4, 64, **bf), torch.randn(10, 64, **bf)
    ids = torch.arange(4, device=DEV)
    tail = (pc, None, None, None, None, 1.0, 1e-6, 1e-6, False)
    st, _ = ops.sum_lstm_embedded(s.view(4, 1, 256), table, ids.view(4, 1), pc.view(4, 1, 64), *tail[1:])
    assert st.shape == (4, 1, 64)
    with pytest.raises(RuntimeError, match="token ids must be int64"):
        ops.sum_lstm_embedded(s, table, ids.int(), *tail)
    with pytest.raises(RuntimeError, match="one contiguous token id per row"):
        ops.sum_lstm_embedded(s, table, ids[:3], *tail)
    with pytest.raises(RuntimeError, match="z must have last dim D_gate"):
        ops.sum_lstm_embedded(s, torch.randn(10, 32, **bf), ids, *tail)
    with pytest.raises(RuntimeError, match="all input dtypes must match"):
        ops.sum_lstm_embedded(s, table.half(), ids, *tail)
    with pytest.raises(RuntimeError, match="no rows"):
        ops.sum_lstm_embedded(s, table[:0], ids, *tail)


def test_rank3_inputs(ops):
    c = make_lstm_case(rows=6, D=256, seed=8)
    for k in ("states", "z4", "prev_cell"):
        c[k] = c[k].contiguous().view(2, 3, -1)
    got_s, got_c, _, _ = run(ops, c, alpha=0.5)
    assert got_s.shape == (2, 3, 256)


def test_empty(ops):
    z = torch.empty(0, 256, dtype=torch.bfloat16, device=DEV)
    s, c = ops.sum_lstm(z, z, torch.empty(0, 64, dtype=torch.bfloat16, device=DEV), None, None, None, None,
                        1.0, 1e-6, 1e-6, False)
    assert s.shape == (0, 64) and c.shape == (0, 64)


def test_errors(ops):
    bf = dict(dtype=torch.bfloat16, device=DEV)
    s, z, pc = torch.randn(4, 256, **bf), torch.randn(4, 256, **bf), torch.randn(4, 64, **bf)
    args = (None, None, None, None, 1.0, 1e-6, 1e-6, False)
    with pytest.raises(RuntimeError, match="sum_lstm: only fp16 and bf16"):
        ops.sum_lstm(s.float(), z.float(), pc.float(), *args)
    with pytest.raises(RuntimeError, match="all input dtypes must match"):
        ops.sum_lstm(s, z.half(), pc, *args)
    with pytest.raises(RuntimeError, match="last dim of states must be 4\\*D_gate"):
        ops.sum_lstm(s[:, :254], z[:, :254], pc, *args)
    with pytest.raises(RuntimeError, match="z4 must have last dim"):
        ops.sum_lstm(s, z[:, :128], pc, *args)
    with pytest.raises(RuntimeError, match="prev_cell last dim must equal D_gate"):
        ops.sum_lstm(s, z, pc[:, :32], *args)
    with pytest.raises(RuntimeError, match="w_cell must have length >= D_eff"):
        ops.sum_lstm(s, z, pc, torch.ones(8, **bf), None, None, None, 1.0, 1e-6, 1e-6, False)
    with pytest.raises(RuntimeError, match="b_state dtype mismatch"):
        ops.sum_lstm(s, z, pc, None, None, None, torch.ones(64, device=DEV), 1.0, 1e-6, 1e-6, False)


def test_random_configurations(ops):
    """Seeded sweep over row counts, gate widths (vector and element-wise kernels, one and two chunks per lane),
    pitches, optional vectors, both GELUs and all three ways of passing z (repeated, once, by token id)."""
    import random
    rnd = random.Random(19)
    for it in range(40):
        rows = rnd.choice([1, 2, 9, 70, 300])
        D = rnd.choice([8, 64, 100, 520, 1024, 4096, 4104, 8192])
        dtype = rnd.choice([torch.float16, torch.bfloat16])
        pad4, padD = rnd.choice([(0, 0), (16, 8), (7, 3)])
        c = make_lstm_case(rows=rows, D=D, dtype=dtype, seed=1200 + it, pad4=pad4, padD=padD,
                           wb_cell=rnd.random() < 0.7, wb_state=rnd.random() < 0.7, repeat_z=True)
        alpha, fast = rnd.choice([0.35, 1.0, speculator_alpha(3, D)]), rnd.random() < 0.3
        eps = rnd.choice([1e-6, 1e-3])
        try:
            got_s, got_c, _, _ = run(ops, c, alpha, eps, eps, fast)
            args = [dev(c[k]) for k in ("prev_cell", "w_cell", "b_cell", "w_state", "b_state")]
            z = c["z4"][:, :D].contiguous()
            st, ce = ops.sum_lstm_shared_z(dev(c["states"]), z.to(DEV), *args, alpha, eps, eps, fast)
            assert torch.equal(st, got_s) and torch.equal(ce, got_c), "shared z differs from repeated z"
            # the same rows again, found through token ids in a shuffled table with a few rows never used
            g = torch.Generator().manual_seed(it)
            perm = torch.randperm(rows + 3, generator=g)
            table = torch.zeros(rows + 3, D, dtype=dtype)
            table[perm[:rows]] = z
            st, ce = ops.sum_lstm_embedded(dev(c["states"]), table.to(DEV), perm[:rows].to(DEV), *args, alpha, eps, eps,
                                           fast)
            assert torch.equal(st, got_s) and torch.equal(ce, got_c), "embedded z differs from repeated z"
        except AssertionError as e:
            raise AssertionError(f"configuration {it}: rows={rows} D={D} {dtype} pads=({pad4},{padD}) alpha={alpha} "
                                 f"fast={fast}: {e}") from None


@pytest.mark.parametrize("cfg", [
    dict(rows=64, D=4096),                       # the speculator's shape: the kernel that does not read the cell at all
    dict(rows=5, D=512, wb_cell=False),          # a scale / shift pair missing
    dict(rows=3, D=8200),                        # two chunks per lane
    dict(rows=7, D=12),                          # element-wise kernel
    dict(rows=4, D=128, pad4=7),                 # element-wise kernel through unaligned pitches
])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("fast", [False, True])
def test_no_previous_cell_equals_a_cell_of_zeros(ops, cfg, dtype, fast):
    """prev_cell_d=None (not in the reference's schema) stands for the zero cell every proposal round starts from
    (arctic_speculator.py:899-903): bit-identical to passing zeros, for all three forms of the operator, and within
    tolerance of the oracle run on zeros."""
    c = make_lstm_case(dtype=dtype, seed=77, **cfg)
    rows, D = cfg["rows"], cfg["D"]
    d = {k: dev(v) for k, v in c.items()}
    zeros = torch.zeros(rows, D, dtype=dtype, device=DEV)
    tail = (d["w_cell"], d["b_cell"], d["w_state"], d["b_state"], 0.35, 1e-6, 1e-5, fast)
    want = ops.sum_lstm(d["states"], d["z4"], zeros, *tail)
    got = ops.sum_lstm(d["states"], d["z4"], None, *tail)
    via_op = torch.ops.arctic_inference.sum_lstm_zero_cell_cuda(d["states"], d["z4"], *tail)
    for g, v, w in zip(got, via_op, want):
        assert g.shape == (rows, D) and g.is_contiguous() and torch.equal(g, w) and torch.equal(v, w)
    o_state, o_cell = oracle.sum_lstm(c["states"], c["z4"], torch.zeros(rows, D, dtype=dtype), c["w_cell"], c["b_cell"],
                                      c["w_state"], c["b_state"], 0.35, 1e-6, 1e-5, fast)
    assert_close(got[0], o_state, RTOL, ATOL, "state")
    assert_close(got[1], o_cell, RTOL, ATOL, "cell")
    z = d["z4"][:, :D].contiguous()
    want = ops.sum_lstm_shared_z(d["states"], z, zeros, *tail)
    got = ops.sum_lstm_shared_z(d["states"], z, None, *tail)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    table = torch.randn(50, D, generator=torch.Generator().manual_seed(3)).to(dtype).to(DEV)
    ids = torch.randint(0, 50, (rows,), generator=torch.Generator().manual_seed(4)).to(DEV)
    want = ops.sum_lstm_embedded(d["states"], table, ids, zeros, *tail)
    got = ops.sum_lstm_embedded(d["states"], table, ids, None, *tail)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    # rank-3 states: outputs take their leading dimensions
    s3 = d["states"][: rows - rows % 1].contiguous().view(rows, 1, 4 * D) if d["states"].is_contiguous() else None
    if s3 is not None:
        g3 = ops.sum_lstm(s3, d["z4"].contiguous().view(rows, 1, 4 * D), None, *tail)
        assert g3[0].shape == (rows, 1, D) and torch.equal(g3[1].view(rows, D), ops.sum_lstm(d["states"], d["z4"], zeros, *tail)[1])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [512, 100])        # the 16-byte-lane kernel and the element-wise one
def test_saturated_gates_zero_rows_and_extreme_magnitudes(ops, dtype, D):
    """Finite inputs at the ends of the formats' ranges: gates driven to both ends of the sigmoid, rows of zeros
    (the norm divides by sqrt(eps)), tiny values, and values whose squares overflow fp32 (the inverse RMS is then
    0 and the normalised row 0).  The results stay finite and match the oracle."""
    big = 6.0e4 if dtype == torch.float16 else 3.0e38
    c = make_lstm_case(rows=8, D=D, dtype=dtype, seed=77)
    s, z, pc = c["states"], c["z4"], c["prev_cell"]
    f, i, o, g = (slice(k * D, (k + 1) * D) for k in range(4))   # any order covers every gate: all four are driven
    s[0, f], s[0, i], s[0, o] = 80.0, -80.0, 80.0              # saturated gates, ordinary candidate
    s[1, :], z[1, :] = 0.0, 0.0                                # a row of zeros
    pc[1, :] = 0.0
    s[2, :], z[2, :] = 1.0e-7 if dtype == torch.float16 else 1.0e-30, 0.0   # tiny
    s[3, g], z[3, :] = big / 8, 0.0                            # squares overflow fp32 in one gate
    s[4, :] = -80.0                                            # everything closed
    pc[5, :] = big / 4                                         # a huge previous cell, kept by an open gate
    s[5, f], s[5, i], s[5, o], s[5, g] = 80.0, 80.0, 80.0, 80.0
    z[5, :] = 0.0
    got_s, got_c, want_s, want_c = run(ops, c, alpha=1.0)
    assert torch.isfinite(want_s.float()).all() and torch.isfinite(want_c.float()).all()


@pytest.mark.parametrize("D", [512, 1000, 1024, 1536, 2048, 2880, 3072, 4000, 4096, 4608, 5000, 5120, 6144, 8192])
@pytest.mark.parametrize("rows", [1, 5, 300])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_staged_kernel_shapes(ops, D, rows, dtype):
    """Rows of up to 8192 elements with all four vectors take the kernel that requests a row in stages (one 16-byte
    chunk per lane; rows that are no multiple of 512 elements leave lanes of the last wave idle): against the oracle
    with and without a previous cell, with pitched rows and the tanh GELU, and bit for bit against the general kernel,
    which the same row takes as soon as one vector is missing (an absent scale acts as 1, an absent shift as 0, so
    ones and zeros in their place change no bit).  Beyond 4096 elements the general kernel gives a lane two chunks, so
    its row sums add up in another order: there the two are compared within the tolerance."""
    pad = 8 if rows > 1 else 0   # pitches stay multiples of 16 bytes
    c = make_lstm_case(rows=rows, D=D, dtype=dtype, seed=900 + D // 8 + rows, pad4=pad, padD=pad)
    for fast in (False, True):
        run(ops, c, alpha=0.35, fast=fast)
    d = {k: dev(v) for k, v in c.items()}
    ones, zeros = torch.ones(D, dtype=dtype, device=DEV), torch.zeros(D, dtype=dtype, device=DEV)
    tail = (0.35, 1e-6, 1e-5, False)
    for cell in (d["prev_cell"], None):
        def same(a, b):
            for x, y in zip(a, b):
                if D <= 4096:
                    assert torch.equal(x, y)
                else:
                    assert_close(x, y, RTOL, ATOL, "staged against general")

        staged = ops.sum_lstm(d["states"], d["z4"], cell, ones, zeros, d["w_state"], d["b_state"], *tail)
        general = ops.sum_lstm(d["states"], d["z4"], cell, None, None, d["w_state"], d["b_state"], *tail)
        same(staged, general)
        z = d["z4"][:, :D].contiguous()
        staged = ops.sum_lstm_shared_z(d["states"], z, cell, d["w_cell"], d["b_cell"], ones, zeros, *tail)
        general = ops.sum_lstm_shared_z(d["states"], z, cell, d["w_cell"], d["b_cell"], None, None, *tail)
        same(staged, general)
