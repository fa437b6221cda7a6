"""GPU parity of speculator_ln against the CPU oracle (1e-2 rel / 2e-2 abs)."""
import pytest
import torch

import oracle
from helpers import assert_close, pitched, to_device_pitched

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL, ATOL = 1e-2, 2e-2


def run(ops, x, w, b, eps=1e-6):
    got = ops.speculator_ln(to_device_pitched(x, DEV), None if w is None else w.to(DEV),
                            None if b is None else b.to(DEV), eps)
    torch.cuda.synchronize()
    want = oracle.speculator_ln(x, w, b, eps)
    assert got.shape == x.shape and got.dtype == x.dtype and got.is_contiguous()
    assert_close(got, want, RTOL, ATOL, "speculator_ln")
    return got, want


# the reference's own shapes: vec8, vec4, tail and rank-3 (tests/unit_tests/test_speculator_ln.py:97-102)
@pytest.mark.parametrize("shape", [(32, 128), (16, 260), (7, 513), (2, 3, 1024), (1, 64), (3, 8), (5, 12288)])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("affine", [False, True])
def test_reference_shapes(ops, shape, dtype, affine):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(*shape, generator=g).to(dtype)
    w = torch.randn(shape[-1], generator=g).to(dtype) if affine else None
    b = torch.randn(shape[-1], generator=g).to(dtype) if affine else None
    run(ops, x, w, b)


@pytest.mark.parametrize("weight_only", [True, False])
def test_config4_layernorm(ops, weight_only):
    # the speculator benchmark shape: [512, 4096] bf16, weight ~ N(1, .02), bias ~ N(0, .02), eps 1e-6
    g = torch.Generator().manual_seed(3)
    x = torch.randn(512, 4096, generator=g).to(torch.bfloat16)
    w = (1 + 0.02 * torch.randn(4096, generator=g)).to(torch.bfloat16)
    b = None if weight_only else (0.02 * torch.randn(4096, generator=g)).to(torch.bfloat16)
    got, want = run(ops, x, w, b)
    same = (got.cpu().view(torch.int16) == want.view(torch.int16)).float().mean().item()
    assert same > 0.98, f"only {same:.4f} of the outputs are bit-identical to the oracle"


@pytest.mark.parametrize("pad", [8, 3])
def test_pitched_rows(ops, pad):
    # row stride larger than hidden; pad 3 breaks 16-byte alignment and takes the element-wise kernel
    g = torch.Generator().manual_seed(1)
    x = pitched(19, 256, pad, torch.bfloat16, g)
    run(ops, x, None, None)


def test_large_magnitudes_and_eps(ops):
    g = torch.Generator().manual_seed(2)
    x = (torch.randn(8, 512, generator=g) * 1e3).to(torch.float16)
    run(ops, x, None, None, eps=1e-6)
    z = torch.zeros(4, 512, dtype=torch.bfloat16)
    got, _ = run(ops, z, None, None, eps=1e-6)
    assert bool((got == 0).all())


def test_empty(ops):
    x = torch.empty(0, 128, dtype=torch.bfloat16, device=DEV)
    assert ops.speculator_ln(x, None, None, 1e-6).shape == (0, 128)


def test_errors(ops):
    x = torch.randn(4, 128, device=DEV)
    with pytest.raises(RuntimeError, match="speculator_ln: only fp16 and bf16"):
        ops.speculator_ln(x, None, None, 1e-6)
    xb = x.to(torch.bfloat16)
    with pytest.raises(RuntimeError, match="last dimension must be contiguous"):
        ops.speculator_ln(xb.t(), None, None, 1e-6)
    with pytest.raises(RuntimeError, match="weight dtype must match"):
        ops.speculator_ln(xb, torch.ones(128, device=DEV), None, 1e-6)
    with pytest.raises(RuntimeError, match="weight must be 1D of size hidden"):
        ops.speculator_ln(xb, torch.ones(64, device=DEV, dtype=torch.bfloat16), None, 1e-6)
    with pytest.raises(RuntimeError, match="bias must be 1D of size hidden"):
        ops.speculator_ln(xb, None, torch.ones(1, 128, device=DEV, dtype=torch.bfloat16), 1e-6)


# --------------------------------------------------------------------------- #
# speculator_add_ln_act: add + norm + GELU / scaling in one launch
# --------------------------------------------------------------------------- #
def glue_inputs(rows, hidden, dtype, seed, pad=0):
    g = torch.Generator().manual_seed(seed)
    x = pitched(rows, hidden, pad, dtype, g, std=1.3)
    z = pitched(rows, hidden, pad, dtype, g)
    w = (1 + 0.1 * torch.randn(hidden, generator=g)).to(dtype)
    b = (0.1 * torch.randn(hidden, generator=g)).to(dtype)
    return x, z, w, b


def same_fraction(a, b):
    return (a.cpu().view(torch.int16) == b.cpu().view(torch.int16)).float().mean().item()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,hidden,pad", [(512, 4096, 0), (33, 1024, 8), (7, 513, 0), (5, 260, 3), (3, 12288, 0)])
@pytest.mark.parametrize("activation", ["gelu", "gelu_tanh"])
def test_add_ln_gelu_against_oracle(ops, dtype, rows, hidden, pad, activation):
    x, z, w, b = glue_inputs(rows, hidden, dtype, 21, pad)
    alpha = 2.3716
    xd, zd = to_device_pitched(x, DEV), to_device_pitched(z, DEV)
    before = xd.clone()
    got = torch.ops.arctic_inference.speculator_add_ln_act_cuda(xd, zd, w.to(DEV), b.to(DEV), alpha, 1e-6,
                                                                activation, 1.0)
    torch.cuda.synchronize()
    want = oracle.speculator_add_ln_act(x, z, w, b, alpha, 1e-6, activation, 1.0)
    assert got.shape == x.shape and got.dtype == dtype and got.is_contiguous()
    assert torch.equal(xd, before), "the input must stay untouched"
    assert_close(got, want, RTOL, ATOL, "speculator_add_ln_act")
    assert same_fraction(got, want) > 0.97
    if activation == "gelu":
        got2 = ops.speculator_add_ln_gelu(xd, zd, w.to(DEV), b.to(DEV), alpha, 1e-6)
        assert torch.equal(got2, got)


def test_add_ln_gelu_against_the_three_separate_gpu_ops(ops):
    """states.add_(z, alpha=...); gelu(speculator_ln(states)) run as the speculator runs them
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:300-307) on the GPU."""
    x, z, w, b = glue_inputs(512, 4096, torch.bfloat16, 22)
    alpha = 2.3716
    xd, zd, wd, bd = x.to(DEV), z.to(DEV), w.to(DEV), b.to(DEV)
    fused = ops.speculator_add_ln_gelu(xd, zd, wd, bd, alpha, 1e-6)
    s = xd.clone()
    s.add_(zd, alpha=alpha)
    separate = torch.nn.functional.gelu(ops.speculator_ln(s, wd, bd, 1e-6))
    assert_close(fused, separate.cpu(), RTOL, ATOL, "fused vs separate")
    assert same_fraction(fused, separate) > 0.99


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,hidden,vocab,table_pad", [(512, 4096, 32000, 0), (33, 1024, 50, 8), (5, 260, 7, 3),
                                                         (1, 12288, 2, 0)])
def test_embed_add_ln_gelu_equals_lookup_then_add_ln_gelu(ops, dtype, rows, hidden, vocab, table_pad):
    """z = emb(last_tokens) looked up inside the launch (arctic_speculator.py:301-309) with the caller's
    clamp of last_tokens (:845, :862): the very bits of the lookup followed by speculator_add_ln_gelu."""
    x, _, w, b = glue_inputs(rows, hidden, dtype, 31)
    g = torch.Generator().manual_seed(32)
    table = torch.randn(vocab, hidden + table_pad, generator=g).to(dtype)[:, :hidden]
    ids = torch.randint(0, vocab, (rows,), generator=g)
    ids[0] = -1
    ids[-1] = vocab
    z = torch.nn.functional.embedding(ids.clamp(0, vocab - 1), table)
    alpha = 2.3716
    xd, wd, bd = x.to(DEV), w.to(DEV), b.to(DEV)
    dtable = to_device_pitched(table, DEV)
    fused = ops.speculator_embed_add_ln_gelu(xd, dtable, ids.to(DEV), wd, bd, alpha, 1e-6)
    two_step = ops.speculator_add_ln_gelu(xd, z.to(DEV), wd, bd, alpha, 1e-6)
    assert torch.equal(fused, two_step)
    assert_close(fused, oracle.speculator_add_ln_act(x, z, w, b, alpha, 1e-6, "gelu", 1.0), RTOL, ATOL, "embedded z")
    with pytest.raises(RuntimeError, match="one contiguous token id per row"):
        ops.speculator_embed_add_ln_gelu(xd, dtable, ids.to(DEV)[: rows - 1] if rows > 1 else ids.to(DEV).repeat(2),
                                         wd, bd, alpha, 1e-6)
    with pytest.raises(RuntimeError, match="embedding table must be"):
        ops.speculator_embed_add_ln_gelu(xd, dtable[:, : hidden - 4], ids.to(DEV), wd, bd, alpha, 1e-6)


@pytest.mark.parametrize("affine", [False, True])
def test_ln_scaled_is_ln_then_scale(ops, affine):
    # ln0(x) / SQRT2 of the speculator (arctic_speculator.py:296-297): no affine terms there
    x, _, w, b = glue_inputs(512, 4096, torch.bfloat16, 23)
    w, b = (w, b) if affine else (None, None)
    wd, bd = (w.to(DEV), b.to(DEV)) if affine else (None, None)
    inv = float(torch.tensor(1.0) / torch.tensor(2 ** 0.5))
    xd = x.to(DEV)
    got = ops.speculator_ln_scaled(xd, wd, bd, 1e-6, inv)
    # bit-identical to the product's own norm followed by a multiplication in fp32, rounded once more
    two_step = (ops.speculator_ln(xd, wd, bd, 1e-6).float() * inv).to(torch.bfloat16)
    assert torch.equal(got, two_step)
    assert_close(got, oracle.speculator_add_ln_act(x, None, w, b, 0.0, 1e-6, "none", inv), RTOL, ATOL, "ln_scaled")
    # and within an ulp of what torch's division gives
    assert same_fraction(got, ops.speculator_ln(xd, wd, bd, 1e-6) / 2 ** 0.5) > 0.99


def test_add_ln_act_degenerate_and_errors(ops):
    x, z, w, b = glue_inputs(9, 512, torch.bfloat16, 24)
    xd, zd, wd, bd = x.to(DEV), z.to(DEV), w.to(DEV), b.to(DEV)
    op = torch.ops.arctic_inference.speculator_add_ln_act_cuda
    plain = ops.speculator_ln(xd, wd, bd, 1e-6)
    assert torch.equal(op(xd, None, wd, bd, 0.0, 1e-6, "none", 1.0), plain)
    assert torch.equal(op(xd, zd, wd, bd, 0.0, 1e-6, "none", 1.0), plain)       # alpha = 0
    assert torch.equal(op(xd, None, wd, bd, 0.0, 1e-6, "none", 0.5), plain / 2)  # exact scaling
    assert op(torch.empty(0, 64, dtype=torch.bfloat16, device=DEV), None, None, None, 0.0, 1e-6, "gelu", 1.0).shape == (0, 64)
    with pytest.raises(RuntimeError, match="activation must be one of"):
        op(xd, zd, wd, bd, 1.0, 1e-6, "relu", 1.0)
    with pytest.raises(RuntimeError, match="z must have the input's shape"):
        op(xd, zd[:4], wd, bd, 1.0, 1e-6, "gelu", 1.0)
    with pytest.raises(RuntimeError, match="z dtype must match"):
        op(xd, zd.half(), wd, bd, 1.0, 1e-6, "gelu", 1.0)
    with pytest.raises(RuntimeError, match="only fp16 and bf16"):
        op(xd.float(), None, None, None, 1.0, 1e-6, "gelu", 1.0)


def ulp16(v: torch.Tensor, dtype) -> torch.Tensor:
    """Spacing of the 16-bit format at |v| (fp32 tensor in, fp32 out)."""
    mant, lowest = (7, -126) if dtype == torch.bfloat16 else (10, -14)
    e = torch.floor(torch.log2(v.abs().clamp_min(2.0 ** lowest)))
    return torch.exp2(e - mant)


def assert_glue_close(got, want, norm_want, act, scale, what):
    """The path's tolerance (1e-2 rel + 2e-2 abs) widened by what an output scale above one may add.  Kernel and
    oracle both round the norm y, the activation g = act(y) and the scaled output to 16 bits.  Their fp32 values in
    front of a rounding differ in the last bits (order of the row sum, reciprocal square root), so where such a value
    lies at a rounding boundary the two may land one 16-bit ulp apart: y by ulp(y), hence g by up to
    max|act'| * ulp(y) + ulp(g) with max|gelu'| = 1.13.  A scale s <= 1 shrinks that difference and the tolerance
    holds as it stands; s > 1 stretches it by s, and the part beyond what s = 1 would show, (s - 1) * (1.13 ulp(y)
    + ulp(g)), is allowed on top."""
    g, w, y = got.detach().cpu().float(), want.float(), norm_want.float()
    act_y = y if act == "none" else torch.nn.functional.gelu(y, approximate="tanh" if act == "gelu_tanh" else "none")
    slope = 1.0 if act == "none" else 1.13
    extra = max(0.0, scale - 1.0) * (slope * ulp16(y, want.dtype) + (0 if act == "none" else 1) * ulp16(act_y, want.dtype))
    tol = ATOL + RTOL * w.abs() + extra
    err = (g - w).abs()
    bad = err > tol
    if bad.any() or not torch.isfinite(g).all():
        i = int(torch.argmax(err - tol))
        raise AssertionError(f"{what}: {int(bad.sum())} of {g.numel()} elements out of tolerance; worst got "
                             f"{g.view(-1)[i].item()} want {w.view(-1)[i].item()} allowed {tol.view(-1)[i].item():.4f}")


def sweep_add_ln_act(ops, seed, only=None):
    """Seeded sweep over shapes (vector kernel with 1-8 chunks per lane, element-wise kernel), pitches, optional
    vectors, activations and output scales (one above one), with z passed directly and by token id.  `only`: run
    just that configuration of the sweep."""
    import random
    rnd = random.Random(seed)
    for it in range(40):
        rows = rnd.choice([1, 2, 9, 70, 300])
        hidden = rnd.choice([8, 64, 260, 513, 2880, 4096, 8200, 16384, 40000])
        dtype = rnd.choice([torch.float16, torch.bfloat16])
        pad = rnd.choice([0, 0, 8, 3])
        keep_w, keep_b = rnd.random() < 0.7, rnd.random() < 0.7
        use_z = rnd.random() < 0.7
        # the speculator's own scales are 1 and 1 / sqrt 2; 3 checks that nothing in the kernel assumes scale <= 1
        act, scale = rnd.choice(["none", "gelu", "gelu_tanh"]), rnd.choice([1.0, 0.70710678, 3.0])
        alpha, eps = rnd.choice([0.0, 0.35, 2.3716]), rnd.choice([1e-6, 1e-3])
        if only is not None and it != only:
            continue
        x, z, w, b = glue_inputs(rows, hidden, dtype, 1500 + it, pad)
        w, b = (w if keep_w else None), (b if keep_b else None)
        d = lambda t: None if t is None else to_device_pitched(t, DEV)
        try:
            want = oracle.speculator_add_ln_act(x, z if use_z else None, w, b, alpha, eps, act, scale)
            norm_want = oracle.speculator_add_ln_act(x, z if use_z else None, w, b, alpha, eps, "none", 1.0)
            got = torch.ops.arctic_inference.speculator_add_ln_act_cuda(d(x), d(z) if use_z else None, d(w), d(b), alpha,
                                                                       eps, act, scale)
            assert got.shape == x.shape and got.is_contiguous()
            assert_glue_close(got, want, norm_want, act, scale, "add_ln_act")
            if use_z:
                g = torch.Generator().manual_seed(it)
                perm = torch.randperm(rows + 2, generator=g)
                table = torch.zeros(rows + 2, hidden, dtype=dtype)
                table[perm[:rows]] = z
                emb = torch.ops.arctic_inference.speculator_embed_add_ln_act_cuda(d(x), table.to(DEV), perm[:rows].to(DEV),
                                                                                  d(w), d(b), alpha, eps, act, scale)
                assert torch.equal(emb, got), "z by token id differs from z passed directly"
            else:
                plain = ops.speculator_ln(d(x), d(w), d(b), eps)
                if act == "none" and scale == 1.0:
                    assert torch.equal(plain, got), "the glue kernel without glue differs from speculator_ln"
        except AssertionError as e:
            raise AssertionError(f"configuration {it}: {rows} x {hidden} {dtype} pad={pad} z={use_z} act={act} "
                                 f"scale={scale} alpha={alpha}: {e}") from None


def test_random_configurations(ops):
    sweep_add_ln_act(ops, 23)


@pytest.mark.parametrize("shift,configuration", [(310, 22), (620, 0), (930, 10), (1550, 11), (1860, 26)])
def test_output_scale_above_one(ops, shift, configuration):
    """Configurations of other seeds of the sweep in which a scale of 3 stretched a one-ulp difference of the rounded
    norm beyond the plain tolerance (70 x 16384, 300 x 8200, 300 x 4096 pitched, 70 x 4096, 70 x 40000 pitched)."""
    sweep_add_ln_act(ops, 23 + shift, only=configuration)
