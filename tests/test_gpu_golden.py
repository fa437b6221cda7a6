"""The HIP operators against the committed golden fixtures, directly (the oracle is not involved): the fixtures in
tests/golden/ were written by tests/golden/make_golden.py from torch library routines only - index assignment and
float8 casts for the bulk write, float64 closed forms for the two float operators - and pin the CPU oracle in
tests/test_oracle_*.py.  Here the same files are fed to the kernels through torch.ops.arctic_inference.*:
cache bytes bit for bit; the norm and the LSTM step within 1e-2 relative + 2e-2 absolute of the float64 values, the
path's tolerance (cases of the reference's tests/unit_tests/test_sum_lstm.py:174-179 and test_speculator_ln.py:97-102)."""
import os

import numpy as np
import pytest
import torch

from helpers import bytes_of

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
RTOL, ATOL = 1e-2, 2e-2


def from_bits(a, dtype):
    return torch.from_numpy(a).view(dtype)


def assert_close_to_exact(got, want64, what):
    g, w = got.detach().cpu().double(), want64.double()
    assert g.shape == w.shape, f"{what}: shape {tuple(g.shape)} vs {tuple(w.shape)}"
    err = (g - w).abs()
    tol = ATOL + RTOL * w.abs()
    assert torch.isfinite(g).all() and bool((err <= tol).all()), (
        f"{what}: {int((err > tol).sum())} of {g.numel()} elements beyond 1e-2 rel + 2e-2 abs; worst {float(err.max()):.4g}")
    return float((err / tol).max())


def test_bulk_write_fixtures_byte_for_byte(ops):
    z = np.load(os.path.join(GOLDEN, "bulk_kv_write.npz"))
    for name in ("bf16_auto", "bf16_fp8", "f16_fp8_e5m2"):
        H, D, bs, NB, L = [int(v) for v in z[f"{name}.dims"]]
        src_dtype = torch.float16 if name.startswith("f16") else torch.bfloat16
        kv = {"auto": "auto", "fp8": "fp8", "e5m2": "fp8_e5m2"}[name.split("_")[-1]]
        keys = from_bits(z[f"{name}.keys"], src_dtype).to(DEV)
        values = from_bits(z[f"{name}.values"], src_dtype).to(DEV)
        slots = torch.from_numpy(z[f"{name}.slots"]).to(DEV)
        init = torch.from_numpy(z[f"{name}.cache_init"])
        want = torch.from_numpy(z[f"{name}.cache_out"])
        cdt = torch.uint8 if kv != "auto" else src_dtype
        bufs = [init[l].clone().view(cdt).view(2, NB, bs, H, D).to(DEV) for l in range(L)]
        ks = [torch.tensor(float(v), device=DEV) for v in z[f"{name}.k_scales"]]
        vs = [torch.tensor(float(v), device=DEV) for v in z[f"{name}.v_scales"]]
        torch.ops.arctic_inference.reshape_and_cache_flash_bulk(keys, values, [b[0] for b in bufs], [b[1] for b in bufs],
                                                               slots, kv, ks, vs, H, D)
        torch.cuda.synchronize()
        for l in range(L):
            assert torch.equal(bytes_of(bufs[l].cpu()).view(-1), want[l].view(-1)), f"{name} layer {l}"


def test_speculator_ln_fixtures(ops):
    z = np.load(os.path.join(GOLDEN, "speculator_ln.npz"))
    assert len(z["names"]) > 0
    for name in z["names"]:
        dtype = torch.float16 if name.startswith("f16") else torch.bfloat16
        x = from_bits(z[f"{name}.x"], dtype)
        w = from_bits(z[f"{name}.w"], dtype).to(DEV) if f"{name}.w" in z else None
        b = from_bits(z[f"{name}.b"], dtype).to(DEV) if f"{name}.b" in z else None
        got = torch.ops.arctic_inference.speculator_ln_cuda(x.to(DEV), w, b, 1e-6)
        assert got.shape == x.shape and got.dtype == dtype and got.is_contiguous()
        assert_close_to_exact(got, torch.from_numpy(z[f"{name}.want"]), f"ln {name}")


def test_sum_lstm_fixtures(ops):
    z = np.load(os.path.join(GOLDEN, "sum_lstm.npz"))
    assert len(z["names"]) > 0
    for name in z["names"]:
        dtype = torch.float16 if name.startswith("f16") else torch.bfloat16
        rows, D, pad4, padD, fast = [int(v) for v in z[f"{name}.meta"]]
        alpha, eps_c, eps_s = [float(v) for v in z[f"{name}.scalars"]]

        def pitch(bits, cols, pad):     # the reference's make_pitched_view (tests/unit_tests/test_sum_lstm.py:73-81)
            base = torch.zeros(rows, cols + pad, dtype=dtype, device=DEV)
            base[:, :cols] = from_bits(bits, dtype).to(DEV)
            return base[:, :cols]

        s4, z4 = pitch(z[f"{name}.states"], 4 * D, pad4), pitch(z[f"{name}.z4"], 4 * D, pad4)
        pc = pitch(z[f"{name}.prev_cell"], D, padD)
        vec = lambda k: from_bits(z[f"{name}.{k}"], dtype).to(DEV) if f"{name}.{k}" in z else None
        state, cell = torch.ops.arctic_inference.sum_lstm_cuda(s4, z4, pc, vec("w_cell"), vec("b_cell"), vec("w_state"),
                                                              vec("b_state"), alpha, eps_c, eps_s, bool(fast))
        assert state.stride() == pc.stride() and cell.stride() == pc.stride()     # sum_lstm.cu:356-365
        assert_close_to_exact(cell, torch.from_numpy(z[f"{name}.want_cell"]), f"cell {name}")
        assert_close_to_exact(state, torch.from_numpy(z[f"{name}.want_state"]), f"state {name}")
