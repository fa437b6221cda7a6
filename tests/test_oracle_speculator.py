"""Pins the CPU oracle of speculator_ln and sum_lstm (no GPU needed).

Checked against: the committed golden fixtures (float64 closed forms evaluated with
torch routines only), torch fp32 restatements of the reference's in-test formulas,
algebraic invariants, and degenerate cases that reduce to library routines.
"""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from helpers import assert_close, make_lstm_case, pitched

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
# largest relative error of ONE round-to-nearest into the format (half a unit in the last place)
HALF_ULP = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11}


def from_bits(a, dtype):
    return torch.from_numpy(a).view(dtype)


def assert_within_ulps(got, want64, dtype, ulps, what):
    """got (a 16-bit result) vs an exact value: at most `ulps` units in the last place
    (0.5 = one correct rounding)."""
    g, w = got.double(), want64.double()
    tol = 2 * ulps * HALF_ULP[dtype] * w.abs() + 1e-6
    bad = (g - w).abs() > tol
    assert not bad.any(), f"{what}: {int(bad.sum())} of {g.numel()} beyond {ulps} ulp; worst {((g - w).abs() / tol).max():.2f}x"


def assert_state_close(got, want64, dtype, what):
    """The state is a function of the ROUNDED cell: where the exact cell sits next to a
    rounding boundary the two sides may round it differently, and GELU's negative branch
    magnifies that (relative slope up to ~4).  So: at least 99.5 % of the elements within
    1.6 ulp, and every element within the path's stated tolerance (1e-2 rel + 2e-2 abs)."""
    g, w = got.double(), want64.double()
    err = (g - w).abs()
    near = err <= 2 * 1.6 * HALF_ULP[dtype] * w.abs() + 1e-6
    assert near.double().mean() >= 0.995, f"{what}: only {near.double().mean():.4f} within 1.6 ulp"
    assert bool((err <= 2e-2 + 1e-2 * w.abs()).all()), f"{what}: element beyond 1e-2 rel + 2e-2 abs"


# --------------------------------------------------------------------------- speculator_ln
def rms_norm_ref(x, eps, w, b):
    """The reference's in-test restatement (tests/unit_tests/test_speculator_ln.py:41-48), in fp32."""
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    if w is not None:
        y = w * y
    if b is not None:
        y = y + b
    return y


def test_ln_golden_fixtures():
    z = np.load(os.path.join(GOLDEN, "speculator_ln.npz"))
    for name in z["names"]:
        dtype = torch.float16 if name.startswith("f16") else torch.bfloat16
        x = from_bits(z[f"{name}.x"], dtype)
        w = from_bits(z[f"{name}.w"], dtype) if f"{name}.w" in z else None
        b = from_bits(z[f"{name}.b"], dtype) if f"{name}.b" in z else None
        got = oracle.speculator_ln(x, w, b, 1e-6)
        assert got.shape == x.shape and got.dtype == dtype
        assert_within_ulps(got, torch.from_numpy(z[f"{name}.want"]), dtype, 0.51, f"ln {name}")


@pytest.mark.parametrize("shape", [(32, 128), (16, 260), (7, 513), (2, 3, 1024)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("affine", [False, True])
def test_ln_matches_torch_fp32(shape, dtype, affine):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(*shape, generator=g).to(dtype)
    w = torch.randn(shape[-1], generator=g).to(dtype) if affine else None
    b = torch.randn(shape[-1], generator=g).to(dtype) if affine else None
    want = rms_norm_ref(x.float(), 1e-6, None if w is None else w.float(), None if b is None else b.float())
    assert_within_ulps(oracle.speculator_ln(x, w, b, 1e-6), want, dtype, 0.52, "ln vs torch fp32")


def test_ln_invariants():
    g = torch.Generator().manual_seed(6)
    x = torch.randn(9, 384, generator=g).to(torch.bfloat16)
    y = oracle.speculator_ln(x, None, None, 1e-12).float()
    rms = y.pow(2).mean(-1).sqrt()
    assert torch.allclose(rms, torch.ones_like(rms), atol=4e-3)           # unit RMS without affine
    y4 = oracle.speculator_ln((x.float() * 4).to(torch.bfloat16), None, None, 1e-12).float()
    assert torch.equal(y, y4)                                              # scale by 2^k: identical bits
    yn = oracle.speculator_ln(-x, None, None, 1e-12).float()
    assert torch.equal(yn, -y)                                             # odd function
    # this is an RMS norm, not a LayerNorm: a constant row maps to +-1, not to 0
    c = torch.full((1, 64), 3.0, dtype=torch.bfloat16)
    assert torch.equal(oracle.speculator_ln(c, None, None, 0.0).float(), torch.ones(1, 64))
    # weight then bias (order matters): y = x_hat * w + b
    w = torch.full((64,), 2.0, dtype=torch.bfloat16)
    b = torch.full((64,), 0.5, dtype=torch.bfloat16)
    assert torch.equal(oracle.speculator_ln(c, w, b, 0.0).float(), torch.full((1, 64), 2.5))
    # eps dominates a zero row
    assert torch.equal(oracle.speculator_ln(torch.zeros(2, 32, dtype=torch.float16), None, None, 1e-6).float(),
                       torch.zeros(2, 32))


def test_ln_pitched_rows_and_dense_output():
    g = torch.Generator().manual_seed(7)
    x = pitched(5, 96, 11, torch.bfloat16, g)
    got = oracle.speculator_ln(x, None, None, 1e-6)
    assert got.is_contiguous()
    assert torch.equal(got, oracle.speculator_ln(x.contiguous(), None, None, 1e-6))


# --------------------------------------------------------------------------- sum_lstm
def sum_lstm_ref(s4, z4, pc, w_cell, b_cell, w_state, b_state, alpha, eps_c, eps_s, fast, dtype):
    """reference_sum_lstm of the reference's test (tests/unit_tests/test_sum_lstm.py:31-70) in fp32,
    plus the one detail the kernel adds: the state phase normalises the ROUNDED cell
    (csrc/custom_ops/sum_lstm.cu:163,174) with the inverse RMS of the unrounded one (:136)."""
    D = pc.size(-1)
    s4, z4, pc = s4.float(), z4.float(), pc.float()
    f32 = lambda t: None if t is None else t.float()
    pre = s4 + alpha * z4
    pf, pi, po, c_pre = pre.split(D, dim=-1)
    act = lambda v: F.gelu(v, approximate="tanh" if fast else "none")
    c_new = pc * torch.sigmoid(pf) + act(rms_norm_ref(c_pre, eps_c, f32(w_cell), f32(b_cell))) * torch.sigmoid(pi)
    inv = torch.rsqrt(c_new.pow(2).mean(-1, keepdim=True) + eps_s)
    sn = c_new.to(dtype).float() * inv
    if w_state is not None:
        sn = sn * w_state.float()
    if b_state is not None:
        sn = sn + b_state.float()
    return act(sn) * torch.sigmoid(po), c_new


def test_lstm_golden_fixtures():
    z = np.load(os.path.join(GOLDEN, "sum_lstm.npz"))
    for name in z["names"]:
        dtype = torch.float16 if name.startswith("f16") else torch.bfloat16
        rows, D, pad4, padD, fast = [int(v) for v in z[f"{name}.meta"]]
        alpha, eps_c, eps_s = [float(v) for v in z[f"{name}.scalars"]]

        def pitch(bits, cols, pad):
            base = torch.zeros(rows, cols + pad, dtype=dtype)
            base[:, :cols] = from_bits(bits, dtype)
            return base[:, :cols]

        s4, z4 = pitch(z[f"{name}.states"], 4 * D, pad4), pitch(z[f"{name}.z4"], 4 * D, pad4)
        pc = pitch(z[f"{name}.prev_cell"], D, padD)
        vec = lambda k: from_bits(z[f"{name}.{k}"], dtype) if f"{name}.{k}" in z else None
        st, ce = oracle.sum_lstm(s4, z4, pc, vec("w_cell"), vec("b_cell"), vec("w_state"), vec("b_state"), alpha,
                                 eps_c, eps_s, bool(fast))
        assert st.stride() == pc.stride() and ce.stride() == pc.stride()
        assert_within_ulps(ce, torch.from_numpy(z[f"{name}.want_cell"]), dtype, 0.51, f"cell {name}")
        # the state sees the cell after its rounding, so a cell that rounds the other
        # way moves the state by up to one more unit
        assert_state_close(st, torch.from_numpy(z[f"{name}.want_state"]), dtype, f"state {name}")


@pytest.mark.parametrize("cfg", [dict(rows=1, D=64, pad4=0, padD=0), dict(rows=4, D=128, pad4=7, padD=3),
                                 dict(rows=32, D=256, pad4=0, padD=0), dict(rows=64, D=512, pad4=16, padD=8)])
@pytest.mark.parametrize("wb", [(True, True), (True, False), (False, True), (False, False)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("fast", [False, True])
def test_lstm_matches_torch_fp32(cfg, wb, dtype, fast):
    c = make_lstm_case(dtype=dtype, seed=77, wb_cell=wb[0], wb_state=wb[1], repeat_z=True, **cfg)
    args = (c["states"], c["z4"], c["prev_cell"], c["w_cell"], c["b_cell"], c["w_state"], c["b_state"])
    st, ce = oracle.sum_lstm(*args, 0.35, 1e-6, 1e-6, fast)
    want_st, want_ce = sum_lstm_ref(*args, 0.35, 1e-6, 1e-6, fast, dtype)
    assert_within_ulps(ce, want_ce, dtype, 0.52, "cell")
    assert_state_close(st, want_st, dtype, "state")


def test_lstm_degenerate_cases():
    g = torch.Generator().manual_seed(8)
    rows, D, dt = 6, 128, torch.bfloat16
    s4 = torch.randn(rows, 4 * D, generator=g).to(dt)
    z4 = torch.randn(rows, 4 * D, generator=g).to(dt)
    pc = torch.randn(rows, D, generator=g).to(dt)
    ones, zeros = torch.ones(D, dtype=dt), torch.zeros(D, dtype=dt)
    # alpha = 0: z4 has no influence at all
    a = oracle.sum_lstm(s4, z4, pc, None, None, None, None, 0.0, 1e-6, 1e-6, False)
    b = oracle.sum_lstm(s4, torch.zeros_like(z4), pc, None, None, None, None, 0.0, 1e-6, 1e-6, False)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    # w = 1, b = 0 equals no affine
    c = oracle.sum_lstm(s4, z4, pc, ones, zeros, ones, zeros, 0.35, 1e-6, 1e-6, False)
    d = oracle.sum_lstm(s4, z4, pc, None, None, None, None, 0.35, 1e-6, 1e-6, False)
    assert torch.equal(c[0], d[0]) and torch.equal(c[1], d[1])
    # prev_cell = 0: c_new = gelu(rmsnorm(pre_c)) * sigmoid(pre_i), built from library routines
    st, ce = oracle.sum_lstm(s4, z4, torch.zeros_like(pc), None, None, None, None, 0.5, 1e-6, 1e-6, False)
    pre = s4.float() + 0.5 * z4.float()
    want = F.gelu(rms_norm_ref(pre[:, 3 * D:], 1e-6, None, None)) * torch.sigmoid(pre[:, D:2 * D])
    assert_within_ulps(ce, want, dt, 0.52, "cell with zero prev_cell")
    # forget gate saturated open, input gate shut: the cell passes through unchanged
    big = torch.zeros(rows, 4 * D)
    big[:, :D] = 80.0
    big[:, D:2 * D] = -80.0
    st, ce = oracle.sum_lstm(big.to(dt), torch.zeros_like(z4), pc, None, None, None, None, 1.0, 1e-6, 1e-6, False)
    assert torch.equal(ce, pc)
    # gate order is f | i | o | c: swapping the f and i blocks must change the result
    sw = torch.cat([s4[:, D:2 * D], s4[:, :D], s4[:, 2 * D:]], dim=1)
    e = oracle.sum_lstm(sw, z4, pc, None, None, None, None, 0.0, 1e-6, 1e-6, False)
    assert not torch.equal(e[1], a[1])
    # tanh and erf GELU differ
    f_ = oracle.sum_lstm(s4, z4, pc, None, None, None, None, 0.35, 1e-6, 1e-6, True)
    assert not torch.equal(f_[0], d[0])


# --------------------------------------------------------------------------- #
# ao_speculator_add_ln_act: the element-wise steps around the norm
# (arctic_inference/vllm/spec_dec/arctic_speculator.py:296-307, 733-734, 809-816)
# --------------------------------------------------------------------------- #
def glue_case(rows, hidden, dtype, seed, pad=0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn(rows, hidden + pad, generator=g) * 1.3).to(dtype)[:, :hidden]
    z = torch.randn(rows, hidden + pad, generator=g).to(dtype)[:, :hidden]
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    b = (0.1 * torch.randn(hidden, generator=g)).to(dtype)
    return x, z, w, b


def same_fraction(a, b):
    return (a.view(torch.int16) == b.view(torch.int16)).float().mean().item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("hidden,pad", [(4096, 0), (260, 0), (513, 3)])
def test_glue_equals_the_separate_torch_ops(dtype, hidden, pad):
    """states.add_(z, alpha); gelu(ln(states)) with torch's GELU around the pinned ao_speculator_ln.
    The add is written out in fp32 (one rounding into the tensor's type): torch's CPU add_ rounds alpha
    to the tensor's type and rounds alpha*z once more in its scalar tail, which the GPU kernel the
    speculator runs on does not.  alpha = 0.75 makes alpha*z exact in fp32, so the sum does not depend
    on fused or separate multiply-add either."""
    x, z, w, b = glue_case(24, hidden, dtype, 7, pad)
    alpha = 0.75
    s = (x.float() + alpha * z.float()).to(dtype)
    t = x.clone()
    t.add_(z, alpha=alpha)
    assert same_fraction(s, t) > 0.99                 # torch's own in-place add agrees but for its tail elements
    want = torch.nn.functional.gelu(oracle.speculator_ln(s, w, b, 1e-6))
    got = oracle.speculator_add_ln_act(x, z, w, b, alpha, 1e-6, "gelu", 1.0)
    # torch's vectorised erf and libm's differ in the last fp32 bits now and then; fp16 keeps three more of them
    assert same_fraction(got, want) > (0.999 if dtype == torch.bfloat16 else 0.997)
    assert_close(got, want, 8e-3 if dtype == torch.bfloat16 else 1.1e-3, 1e-6, "glue vs separate ops (one ulp)")
    # the tanh form against torch's
    want_t = torch.nn.functional.gelu(oracle.speculator_ln(s, w, b, 1e-6).float(), approximate="tanh").to(dtype)
    got_t = oracle.speculator_add_ln_act(x, z, w, b, alpha, 1e-6, "gelu_tanh", 1.0)
    assert same_fraction(got_t, want_t) > (0.999 if dtype == torch.bfloat16 else 0.997)


def test_glue_float64_closed_form_with_general_alpha():
    x, z, w, b = glue_case(16, 1024, torch.bfloat16, 8)
    alpha = 2.3716
    a32 = float(torch.tensor(alpha, dtype=torch.float32))
    s = (x.double() + a32 * z.double()).to(torch.bfloat16)          # rounding after the in-place add
    y = rms_norm_ref(s.double(), 1e-6, w.double(), b.double()).to(torch.bfloat16)
    want = torch.nn.functional.gelu(y.double()).to(torch.bfloat16)
    got = oracle.speculator_add_ln_act(x, z, w, b, alpha, 1e-6, "gelu", 1.0)
    assert same_fraction(got, want) > 0.995
    # an add that lands on the other side of a rounding boundary moves the end result by a few ulps
    assert_close(got, want, 1e-2, 2e-2, "glue vs float64")


def test_glue_degenerate_cases():
    x, z, w, b = glue_case(9, 512, torch.bfloat16, 9)
    plain = oracle.speculator_ln(x, w, b, 1e-6)
    # nothing switched on: the norm itself, bit for bit
    assert torch.equal(oracle.speculator_add_ln_act(x, None, w, b, 0.0, 1e-6, "none", 1.0), plain)
    # alpha = 0: z must not matter
    assert torch.equal(oracle.speculator_add_ln_act(x, z, w, b, 0.0, 1e-6, "none", 1.0), plain)
    # scaling by a power of two is exact: ln(x) * 0.5 == ln(x) / 2
    assert torch.equal(oracle.speculator_add_ln_act(x, None, w, b, 0.0, 1e-6, "none", 0.5), plain / 2)
    # ln0(x) / SQRT2 (no affine) against torch's division, which the GPU turns into a multiplication
    inv = float(torch.tensor(1.0, dtype=torch.float32) / torch.tensor(2 ** 0.5, dtype=torch.float32))
    got = oracle.speculator_add_ln_act(x, None, None, None, 0.0, 1e-6, "none", inv)
    want = oracle.speculator_ln(x, None, None, 1e-6) / 2 ** 0.5
    assert same_fraction(got, want) > 0.995
    assert_close(got, want, 8e-3, 1e-6, "ln0 / sqrt2")
    # the order is norm -> activation -> scale: the other orders give something else
    a = oracle.speculator_add_ln_act(x, z, w, b, 1.5, 1e-6, "gelu", 0.5)
    ln = oracle.speculator_ln((x.float() + 1.5 * z.float()).to(torch.bfloat16), w, b, 1e-6)
    assert_close(a, torch.nn.functional.gelu(ln) * 0.5, 8e-3, 1e-6, "order")
    wrong = torch.nn.functional.gelu(ln * 0.5)
    assert (a.float() - wrong.float()).abs().max() > 0.05
    # the sign of alpha matters
    assert not torch.equal(oracle.speculator_add_ln_act(x, z, w, b, -1.5, 1e-6, "gelu", 0.5), a)


def test_glue_rejects_unknown_modes():
    x = torch.zeros(2, 8)
    with pytest.raises(RuntimeError):
        oracle.speculator_add_ln_act(x, None, None, None, 0.0, 1e-6, "none", 1.0)   # fp32
    with pytest.raises(KeyError):
        oracle.speculator_add_ln_act(x.bfloat16(), None, None, None, 0.0, 1e-6, "relu", 1.0)


def test_reference_pytorch_fallbacks_agree_with_the_oracle():
    """The reference's own PyTorch fallback (what it runs without its compiled operators, and what the benchmark
    times as the CPU baseline of the speculator operators) computes the same function as the C oracle: in fp32 it
    agrees to rounding, in bf16 (every intermediate rounded) within a few bf16 ulps."""
    from oracle.torch_fallback import speculator_ln_fallback, sum_lstm_fallback
    c = make_lstm_case(rows=24, D=512, seed=91)
    alpha = 1.3
    want_state, want_cell = oracle.sum_lstm(c["states"], c["z4"], c["prev_cell"], c["w_cell"], c["b_cell"], c["w_state"],
                                            c["b_state"], alpha, 1e-6, 1e-6, False)
    f32 = {k: (None if v is None else v.float()) for k, v in c.items()}
    st, ce = sum_lstm_fallback(f32["states"], f32["z4"], f32["prev_cell"], f32["w_cell"], f32["b_cell"], f32["w_state"],
                               f32["b_state"], alpha, 1e-6, 1e-6, False)
    # the oracle rounds the cell to bf16 before the state phase (sum_lstm.cu:163,174); the fallback in fp32 does not
    assert_close(ce, want_cell, rtol=4e-3, atol=4e-3, what="fp32 fallback cell")
    assert_close(st, want_state, rtol=8e-3, atol=8e-3, what="fp32 fallback state")
    st, ce = sum_lstm_fallback(c["states"], c["z4"], c["prev_cell"], c["w_cell"], c["b_cell"], c["w_state"], c["b_state"],
                               alpha, 1e-6, 1e-6, False)
    assert st.dtype == torch.bfloat16 and ce.dtype == torch.bfloat16
    assert_close(ce, want_cell, rtol=3e-2, atol=3e-2, what="bf16 fallback cell")
    assert_close(st, want_state, rtol=3e-2, atol=3e-2, what="bf16 fallback state")
    x = c["prev_cell"]
    assert_close(speculator_ln_fallback(x.float(), c["w_cell"].float(), c["b_cell"].float(), 1e-6),
                 oracle.speculator_ln(x, c["w_cell"], c["b_cell"], 1e-6), rtol=4e-3, atol=4e-3, what="fp32 fallback norm")
    assert_close(speculator_ln_fallback(x, None, None, 1e-6), oracle.speculator_ln(x, None, None, 1e-6), rtol=2e-2,
                 atol=2e-2, what="bf16 fallback norm")
