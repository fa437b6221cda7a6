"""Seeded workload generators and comparison helpers shared by the tests."""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

FP8_MAX = {"fp8": 448.0, "fp8_e4m3": 448.0, "fp8_e5m2": 57344.0}


def make_slots(num_tokens: int, num_slots: int, gen: torch.Generator, pad_fraction: float = 0.0):
    """Distinct random slots; a fraction of the tokens is padding (slot -1)."""
    n_pad = int(pad_fraction * num_tokens)
    slots = torch.full((num_tokens,), -1, dtype=torch.int64)
    order = torch.randperm(num_tokens, generator=gen)
    valid = order[n_pad:]
    slots[valid] = torch.randperm(num_slots, generator=gen)[: valid.numel()]
    return slots


def make_bulk_case(
    *, T: int, L: int, H: int, D: int, bs: int, NB: int, src_dtype=torch.bfloat16,
    kv_cache_dtype: str = "auto", seed: int = 0, std: float = 1.0, pad_fraction: float = 0.0,
    layout: str = "flash", key_pad: int = 0, scale_mode: str = "amax",
):
    """CPU tensors for one bulk KV-write call.

    layout "flash": per layer one [2, NB, bs, H, D] buffer, K = buf[0], V = buf[1];
    layout "flashinfer": [NB, 2, bs, H, D], K = buf[:, 0], V = buf[:, 1] (block stride 2*bs*H*D).
    Caches are pre-filled with seeded random bytes so untouched rows are checkable.
    """
    g = torch.Generator().manual_seed(seed)
    n = H * D
    keys = (torch.randn(T, L * n + key_pad, generator=g) * std).to(src_dtype)[:, : L * n]
    values = (torch.randn(T, L * n + key_pad, generator=g) * std).to(src_dtype)[:, : L * n]
    slots = make_slots(T, NB * bs, g, pad_fraction)
    quant = kv_cache_dtype != "auto"
    cache_dtype = torch.uint8 if quant else src_dtype
    gc = torch.Generator().manual_seed(seed + 100)
    bufs, kc, vc = [], [], []
    for _ in range(L):
        shape = (2, NB, bs, H, D) if layout == "flash" else (NB, 2, bs, H, D)
        nbytes = 2 * NB * bs * n * (1 if quant else keys.element_size())
        raw = torch.randint(0, 256, (nbytes,), generator=gc, dtype=torch.uint8)
        buf = raw.view(cache_dtype).view(shape)
        bufs.append(buf)
        if layout == "flash":
            kc.append(buf[0])
            vc.append(buf[1])
        else:
            kc.append(buf[:, 0])
            vc.append(buf[:, 1])
    ks, vs = [], []
    for l in range(L):
        if not quant or scale_mode == "one":
            ks.append(torch.tensor(1.0))
            vs.append(torch.tensor(1.0))
        else:
            mx = FP8_MAX[kv_cache_dtype]
            ks.append((keys[:, l * n:(l + 1) * n].float().abs().max() / mx).to(torch.float32))
            vs.append((values[:, l * n:(l + 1) * n].float().abs().max() / mx).to(torch.float32))
    return dict(keys=keys, values=values, key_caches=kc, value_caches=vc, bufs=bufs, slot_mapping=slots,
                layout=layout, kv_cache_dtype=kv_cache_dtype, k_scales=ks, v_scales=vs, num_heads=H, head_size=D)


def bulk_args(case) -> tuple:
    return (case["keys"], case["values"], case["key_caches"], case["value_caches"], case["slot_mapping"],
            case["kv_cache_dtype"], case["k_scales"], case["v_scales"], case["num_heads"], case["head_size"])


def bulk_case_to(case, device):
    """Copy a case to `device`, rebuilding the per-layer K/V views on the copied buffers."""
    out = dict(case)
    for k in ("keys", "values", "slot_mapping"):
        base = case[k]
        if k != "slot_mapping" and base.stride(0) != base.size(1):
            # preserve the padded row pitch
            full = torch.empty(base.size(0), base.stride(0), dtype=base.dtype, device=device)
            full[:, : base.size(1)].copy_(base)
            out[k] = full[:, : base.size(1)]
        else:
            out[k] = base.to(device)
    out["bufs"] = [b.to(device) for b in case["bufs"]]
    flash = case["layout"] == "flash"
    if flash:
        out["key_caches"] = [b[0] for b in out["bufs"]]
        out["value_caches"] = [b[1] for b in out["bufs"]]
    else:
        out["key_caches"] = [b[:, 0] for b in out["bufs"]]
        out["value_caches"] = [b[:, 1] for b in out["bufs"]]
    out["k_scales"] = [s.to(device) for s in case["k_scales"]]
    out["v_scales"] = [s.to(device) for s in case["v_scales"]]
    return out


def bytes_of(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous().view(torch.uint8)


def assert_bulk_equal(got_bufs: List[torch.Tensor], want_bufs: List[torch.Tensor]):
    for l, (g, w) in enumerate(zip(got_bufs, want_bufs)):
        gb, wb = bytes_of(g.cpu()), bytes_of(w)
        if not torch.equal(gb, wb):
            bad = (gb != wb).nonzero()
            raise AssertionError(
                f"layer {l}: {bad.numel()} differing bytes, first at {bad[0].item()}: "
                f"got {gb.view(-1)[bad[0]].item()} want {wb.view(-1)[bad[0]].item()}")


def pitched(rows: int, cols: int, pad: int, dtype, gen: torch.Generator, std: float = 1.0) -> torch.Tensor:
    """[rows, cols] view with row stride cols + pad (the reference's make_pitched_view,
    tests/unit_tests/test_sum_lstm.py:73-81)."""
    base = (torch.randn(rows, cols + pad, generator=gen) * std).to(dtype)
    return base[:, :cols]


def to_device_pitched(t: torch.Tensor, device) -> torch.Tensor:
    if t.dim() == 2 and t.stride(0) != t.size(1):
        full = torch.empty(t.size(0), t.stride(0), dtype=t.dtype, device=device)
        full[:, : t.size(1)].copy_(t)
        return full[:, : t.size(1)]
    return t.to(device)


def make_lstm_case(*, rows: int, D: int, dtype=torch.bfloat16, seed: int = 3, pad4: int = 0, padD: int = 0,
                   wb_cell: bool = True, wb_state: bool = True, repeat_z: bool = False):
    g = torch.Generator().manual_seed(seed)
    states = pitched(rows, 4 * D, pad4, dtype, g)
    if repeat_z:
        z = torch.randn(rows, D, generator=g).to(dtype)
        z4 = pitched(rows, 4 * D, pad4, dtype, g)
        z4.copy_(z.repeat(1, 4))
    else:
        z4 = pitched(rows, 4 * D, pad4, dtype, g)
    pc = pitched(rows, D, padD, dtype, g)

    def vec(mean, std, on):
        return (mean + std * torch.randn(D, generator=g)).to(dtype) if on else None

    return dict(states=states, z4=z4, prev_cell=pc, w_cell=vec(1.0, 0.02, wb_cell), b_cell=vec(0.0, 0.02, wb_cell),
                w_state=vec(1.0, 0.02, wb_state), b_state=vec(0.0, 0.02, wb_state))


def speculator_alpha(n_predict: int = 3, inner_dim: int = 4096) -> float:
    """alpha = emb_weight / state_weight as the speculator computes it
    (arctic_inference/vllm/spec_dec/arctic_speculator.py:646-648)."""
    state_weight = 0.5 ** (0.5 / n_predict)
    emb_weight = ((1 - state_weight ** 2) * (inner_dim / 2)) ** 0.5
    return emb_weight / state_weight


def assert_close(got: torch.Tensor, want: torch.Tensor, rtol: float = 1e-2, atol: float = 2e-2, what: str = ""):
    """|got - want| <= atol + rtol*|want| element-wise, in fp32."""
    g, w = got.detach().cpu().float(), want.detach().cpu().float()
    assert g.shape == w.shape, f"{what}: shape {g.shape} vs {w.shape}"
    err = (g - w).abs()
    tol = atol + rtol * w.abs()
    bad = err > tol
    if bad.any() or not torch.isfinite(g).all():
        i = int(torch.argmax(err - tol))
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {g.numel()} elements out of tolerance; worst got "
            f"{g.view(-1)[i].item()} want {w.view(-1)[i].item()}")
