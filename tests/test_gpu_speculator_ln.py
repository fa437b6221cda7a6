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
