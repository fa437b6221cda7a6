"""HIP-graph capture of the whole path and direct calls into the C ABI."""
import ctypes

import pytest
import torch

import oracle
from arcticinference_amd import _native
from helpers import (assert_bulk_equal, assert_close, bulk_args, bulk_case_to, make_bulk_case, make_lstm_case,
                     speculator_alpha)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_decode_step_in_one_graph(ops):
    """The decode-step workload in miniature: bulk fp8 KV write, ln0 (no affine) and three chained
    sum_lstm steps captured as one graph.  The graph is replayed several times with eager
    work and synchronisation in between; every replay must equal the eager result and
    the oracle."""
    T, D = 64, 1024
    case = make_bulk_case(T=T, L=4, H=8, D=128, bs=16, NB=16, kv_cache_dtype="fp8", seed=4, std=1.5)
    dcase = bulk_case_to(case, DEV)
    steps = [make_lstm_case(rows=T, D=D, seed=40 + k) for k in range(3)]
    dsteps = [{k: (None if v is None else v.to(DEV)) for k, v in s.items()} for s in steps]
    g = torch.Generator().manual_seed(44)
    x = torch.randn(T, D, generator=g).to(torch.bfloat16)
    dx = x.to(DEV)
    alpha = speculator_alpha(3, D)

    def step():
        ops.reshape_and_cache_flash_bulk(*bulk_args(dcase))
        h = ops.speculator_ln(dx, None, None, 1e-6)
        cell = torch.zeros(T, D, dtype=torch.bfloat16, device=DEV)
        states = []
        for s in dsteps:
            st, cell = ops.sum_lstm(s["states"], s["z4"], cell, s["w_cell"], s["b_cell"], s["w_state"], s["b_state"],
                                    alpha, 1e-6, 1e-6, False)
            states.append(st)
        return h, states, cell

    # oracle
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    want_h = oracle.speculator_ln(x, None, None, 1e-6)

    sentinel = [b.clone() for b in dcase["bufs"]]
    eager_h, eager_states, eager_cell = step()
    torch.cuda.synchronize()
    assert_bulk_equal(dcase["bufs"], case["bufs"])
    assert_close(eager_h, want_h, what="ln0")
    cell = torch.zeros(T, D, dtype=torch.bfloat16)
    for k, s in enumerate(steps):
        # chain through the GPU's own cell so that only this step's arithmetic is compared
        prev = cell
        want_st, want_cell = oracle.sum_lstm(s["states"], s["z4"], prev, s["w_cell"], s["b_cell"], s["w_state"],
                                             s["b_state"], alpha, 1e-6, 1e-6, False)
        assert_close(eager_states[k], want_st, what=f"state {k}")
        cell = want_cell
    eager = [eager_h.clone()] + [s.clone() for s in eager_states] + [eager_cell.clone()]

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        gh, gstates, gcell = step()
    for replay in range(4):
        for b, s in zip(dcase["bufs"], sentinel):
            b.copy_(s)                       # eager work between replays: restore the untouched caches
        gh.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_bulk_equal(dcase["bufs"], case["bufs"])
        got = [gh] + list(gstates) + [gcell]
        for a, b in zip(got, eager):
            assert torch.equal(a, b), f"replay {replay} differs from the eager run"


def test_next_row_operators_in_one_graph(ops):
    """gather_rows, the bulk write, ln0 / sqrt2, add + norm + GELU, sum_lstm with the shared embedding row
    scatter_rows, argmax + clamp and the operators with the embedding lookup captured as one graph; every
    replay must equal the eager run bit for bit."""
    T, D, n_sel = 96, 1024, 40
    g = torch.Generator().manual_seed(77)
    case = make_bulk_case(T=T, L=4, H=8, D=128, bs=16, NB=16, kv_cache_dtype="fp8", seed=5, std=1.5)
    dcase = bulk_case_to(case, DEV)
    rn = lambda *sh: torch.randn(*sh, generator=g).to(torch.bfloat16).to(DEV)
    hidden, residual = rn(T, D), rn(T, D)
    positions = torch.randint(0, 4096, (T,), generator=g).to(DEV)
    idx = torch.sort(torch.randperm(T, generator=g)[:n_sel]).values.to(DEV)
    bufs = [torch.zeros(64, D, dtype=torch.bfloat16, device=DEV), torch.zeros(64, D, dtype=torch.bfloat16, device=DEV),
            torch.zeros(64, dtype=torch.int64, device=DEV)]
    z, w, b = rn(64, D), rn(D), rn(D)
    s4, pc = rn(64, 4 * D), rn(64, D)
    orig = rn(T, D)
    table = rn(500, D)
    alpha = speculator_alpha(3, D)

    kv_bufs = [torch.zeros(64, 4 * 1024, dtype=torch.bfloat16, device=DEV) for _ in range(2)]

    def step():
        h, r, p = ops.gather_rows([hidden, residual, positions], idx, bufs)
        k_sel, v_sel = ops.reshape_and_cache_flash_bulk_select(*bulk_args(dcase), idx, *kv_bufs)
        x0 = ops.speculator_ln_scaled(h, None, None, 1e-6, 0.70710678)
        act = ops.speculator_add_ln_gelu(x0, z, w, b, alpha, 1e-6)
        st, cell = ops.sum_lstm_shared_z(s4, act, pc, w, b, w, b, alpha, 1e-6, 1e-6, False)
        out = orig.clone()
        ops.scatter_rows([st], idx, [out])
        # the next head: tokens from the argmax of (stand-in) logits, looked up inside the operators
        tokens = ops.speculator_argmax(st[:, :600], 499)
        st2, cell2 = ops.sum_lstm_embedded(s4, table, tokens, cell, w, b, w, b, alpha, 1e-6, 1e-6, False)
        act2 = ops.speculator_embed_add_ln_gelu(x0, table, tokens, w, b, alpha, 1e-6)
        return x0, act, st, cell, out, p, tokens, st2, cell2, act2, k_sel, v_sel

    eager = [t.clone() for t in step()]
    torch.cuda.synchronize()
    want = orig.clone()
    want[idx] = eager[2][:n_sel]
    assert torch.equal(eager[4], want)
    assert torch.equal(eager[5][:n_sel], positions[idx])
    assert torch.equal(eager[10], dcase["keys"][idx]) and torch.equal(eager[11], dcase["values"][idx])
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    assert_bulk_equal(dcase["bufs"], case["bufs"])
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step()
    for replay in range(3):
        for t in bufs + kv_bufs + dcase["bufs"]:
            t.zero_()                          # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for a, e in zip(outs, eager):
            assert torch.equal(a, e), f"replay {replay} differs from the eager run"
        # the caches were cleared before the replay: every written row is back, the rest stays zero
        want = [torch.zeros_like(b) for b in case["bufs"]]
        zcase = dict(case, bufs=want, key_caches=[b[0] for b in want], value_caches=[b[1] for b in want])
        oracle.reshape_and_cache_flash_bulk(*bulk_args(zcase))
        assert_bulk_equal(dcase["bufs"], want)


def test_direct_c_abi_calls(ops):
    """Raw pointers straight into libarctic_mi355x.so (what another host language would do)."""
    lib = _native.load()
    stream = torch.cuda.current_stream().cuda_stream
    g = torch.Generator().manual_seed(12)
    rows, hidden = 10, 512
    x = torch.randn(rows, hidden, generator=g).to(torch.float16)
    w = torch.randn(hidden, generator=g).to(torch.float16)
    dx, dw = x.to(DEV), w.to(DEV)
    out = torch.empty_like(dx)
    rc = lib.arctic_speculator_ln(out.data_ptr(), dx.data_ptr(), dw.data_ptr(), None, rows, hidden, hidden, 1e-6,
                                  _native.DTYPE_F16, stream)
    assert rc == 0, lib.arctic_last_error()
    torch.cuda.synchronize()
    assert_close(out, oracle.speculator_ln(x, w, None, 1e-6), what="ln via C ABI")

    case = make_bulk_case(T=20, L=3, H=2, D=64, bs=8, NB=4, kv_cache_dtype="fp8", seed=13, std=1.5, pad_fraction=0.2)
    d = bulk_case_to(case, DEV)
    L = 3
    tab = lambda ts: (ctypes.c_void_p * L)(*[t.data_ptr() for t in ts])
    rc = lib.arctic_reshape_and_cache_flash_bulk(
        d["keys"].data_ptr(), d["values"].data_ptr(), d["keys"].stride(0), d["values"].stride(0),
        tab(d["key_caches"]), tab(d["value_caches"]), tab(d["k_scales"]), tab(d["v_scales"]),
        d["slot_mapping"].data_ptr(), 20, L, 2, 64, 8, d["key_caches"][0].stride(0), 4, _native.DTYPE_BF16,
        _native.KV_FP8_E4M3, stream)
    assert rc == 0, lib.arctic_last_error()
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    assert_bulk_equal(d["bufs"], case["bufs"])

    c = make_lstm_case(rows=5, D=256, seed=14)
    dc = {k: (None if v is None else v.to(DEV)) for k, v in c.items()}
    st, ce = torch.empty(5, 256, dtype=torch.bfloat16, device=DEV), torch.empty(5, 256, dtype=torch.bfloat16, device=DEV)
    rc = lib.arctic_sum_lstm(st.data_ptr(), ce.data_ptr(), dc["states"].data_ptr(), dc["z4"].data_ptr(),
                             dc["prev_cell"].data_ptr(), dc["w_cell"].data_ptr(), dc["b_cell"].data_ptr(),
                             dc["w_state"].data_ptr(), dc["b_state"].data_ptr(), 5, 256, 1024, 1024, 256, 256, 0.35,
                             1e-6, 1e-6, 0, _native.DTYPE_BF16, stream)
    assert rc == 0, lib.arctic_last_error()
    torch.cuda.synchronize()
    wst, wce = oracle.sum_lstm(c["states"], c["z4"], c["prev_cell"], c["w_cell"], c["b_cell"], c["w_state"],
                               c["b_state"], 0.35, 1e-6, 1e-6, False)
    assert_close(st, wst, what="state via C ABI")
    assert_close(ce, wce, what="cell via C ABI")


def test_side_stream(ops):
    """The host layer launches on torch's current stream, whichever that is."""
    g = torch.Generator().manual_seed(15)
    x = torch.randn(64, 2048, generator=g).to(torch.bfloat16)
    dx = x.to(DEV)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        y = ops.speculator_ln(dx, None, None, 1e-6)
    s.synchronize()
    assert_close(y, oracle.speculator_ln(x, None, None, 1e-6), what="ln on a side stream")


@pytest.mark.parametrize("backend", ["eager", "aot_eager"])
def test_operators_trace_under_torch_compile(ops, backend):
    """Traced as opaque nodes (the Meta key gives the shapes), the operators compute what they compute eagerly,
    the one that writes into its arguments included."""
    g = torch.Generator().manual_seed(16)
    rn = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(DEV)
    x, w, s4, z4 = rn(64, 1024), rn(1024), rn(64, 4096), rn(64, 4096)

    def step(x, s4, z4, w):
        y = ops.speculator_ln(x, w, None, 1e-6)
        state, cell = ops.sum_lstm(s4, z4, y, w, w, w, w, 0.5, 1e-6, 1e-6, False)
        return state + 1, cell, ops.speculator_argmax(state.float(), 1000)

    want = step(x, s4, z4, w)
    got = torch.compile(step, backend=backend, fullgraph=True)(x, s4, z4, w)
    for a, b in zip(got, want):
        assert torch.equal(a, b)

    def first_step(s4, z4, x, w):
        # no previous cell, in all three forms (the optional argument traces as None)
        a = ops.sum_lstm(s4, z4, None, w, w, w, w, 0.5, 1e-6, 1e-6, False)
        b = ops.sum_lstm_shared_z(s4, x, None, w, w, w, w, 0.5, 1e-6, 1e-6, False)
        return a[0] + b[0], a[1], b[1]

    want = first_step(s4, z4, x, w)
    got = torch.compile(first_step, backend=backend, fullgraph=True)(s4, z4, x, w)
    for a, b in zip(got, want):
        assert torch.equal(a, b)

    layers = 3
    k, v = rn(16, layers * 128), rn(16, layers * 128)
    slots = torch.randperm(64, generator=g)[:16].to(DEV)
    scales = [torch.tensor([0.5], device=DEV) for _ in range(layers)]
    caches = lambda: [torch.zeros(4, 16, 2, 64, dtype=torch.uint8, device=DEV) for _ in range(2 * layers)]

    def write(k, v, kc, vc, slots, ks, vs):
        ops.reshape_and_cache_flash_bulk(k, v, kc, vc, slots, "fp8", ks, vs, 2, 64)
        return k * 2

    eager, traced = caches(), caches()
    write(k, v, eager[:layers], eager[layers:], slots, scales, scales)
    out = torch.compile(write, backend=backend, fullgraph=True)(k, v, traced[:layers], traced[layers:], slots,
                                                                scales, scales)
    assert torch.equal(out, k * 2)
    for a, b in zip(traced, eager):
        assert torch.equal(a, b) and a.any()


def test_reference_schemas_through_the_dispatcher(ops):
    """One eager call of each of the reference's four operators as torch.ops.arctic_inference.<op> (schema parsing,
    dispatch on the CUDA key, the host layer), compared with the oracle."""
    t = torch.ops.arctic_inference
    for kv in ("fp8", "auto"):
        case = make_bulk_case(T=130, L=5, H=8, D=128, bs=16, NB=16, kv_cache_dtype=kv, seed=80, std=1.5, pad_fraction=0.1)
        d = bulk_case_to(case, DEV)
        assert t.reshape_and_cache_flash_bulk(*bulk_args(d)) is None
        torch.cuda.synchronize()
        oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
        assert_bulk_equal(d["bufs"], case["bufs"])
    c = make_lstm_case(rows=40, D=512, seed=81)
    dc = {k: None if v is None else v.to(DEV) for k, v in c.items()}
    state, cell = t.sum_lstm_cuda(dc["states"], dc["z4"], dc["prev_cell"], dc["w_cell"], dc["b_cell"], dc["w_state"],
                                  dc["b_state"], 0.35, 1e-6, 1e-6, False)
    want_state, want_cell = oracle.sum_lstm(c["states"], c["z4"], c["prev_cell"], c["w_cell"], c["b_cell"], c["w_state"],
                                            c["b_state"], 0.35, 1e-6, 1e-6, False)
    assert_close(state, want_state, what="state")
    assert_close(cell, want_cell, what="cell")
    y = t.speculator_ln_cuda(dc["prev_cell"], dc["w_cell"], dc["b_cell"], 1e-6)
    assert_close(y, oracle.speculator_ln(c["prev_cell"], c["w_cell"], c["b_cell"], 1e-6), what="norm")
    T, H, D, bs, NB = 48, 4, 64, 16, 4
    g = torch.Generator().manual_seed(82)
    key, value = torch.randn(T, H, D, generator=g).bfloat16(), torch.randn(T, H, D, generator=g).bfloat16()
    slots = torch.randperm(NB * bs, generator=g)[:T]
    caches = [torch.zeros(NB, bs, H, D // 2, dtype=torch.uint8) for _ in range(2)] + \
             [torch.zeros(NB, bs, H, D // 16, dtype=torch.uint8) for _ in range(2)]
    dcaches = [x.to(DEV) for x in caches]
    one = torch.ones(())
    t.reshape_and_cache_flash_fp4(key.to(DEV), value.to(DEV), dcaches[0], dcaches[1], slots.to(DEV), "fp4", one.to(DEV),
                                  one.to(DEV), dcaches[2], dcaches[3])
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_fp4(key, value, caches[0], caches[1], caches[2], caches[3], slots, "fp4", one, one)
    for a, b in zip(dcaches, caches):
        assert torch.equal(a.cpu(), b)
