"""Pins the CPU oracle of the NVFP4-style cache write (no GPU needed).

The reference's own test only bounds the dequantisation error against fp16 with live GPU
code; here the oracle is checked against a torch restatement of the closed form, a brute
force nearest-value search for the e2m1 rounding, the decoders of the reference's test
(tests/unit_tests/test_reshape_and_cache_flash_nvfp4.py:5-45, restated) and error bounds.
The last ulp of the two approximate reciprocals of the reference stays unpinned.
"""
import pytest
import torch

import oracle

E2M1 = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])


def e2m1_rne_bruteforce(x: torch.Tensor) -> torch.Tensor:
    """Nearest representable magnitude; ties go to the code with an even mantissa bit
    (codes 0, 2, 4, 6 = 0, 1, 2, 4)."""
    a = x.abs().clamp(max=6.0).double()
    d = (a[:, None] - E2M1.double()[None, :]).abs()
    best = d.min(dim=1).values
    cand = d == best[:, None]
    code = torch.zeros(x.numel(), dtype=torch.int64)
    for i in range(x.numel()):
        idx = cand[i].nonzero().view(-1).tolist()
        code[i] = idx[0] if len(idx) == 1 else [c for c in idx if c % 2 == 0][0]
    return code | ((x < 0) | ((x == 0) & (torch.signbit(x)))).to(torch.int64) * 8


def test_e2m1_rounding():
    L = oracle.lib()
    mids = (E2M1[:-1] + E2M1[1:]) / 2
    pts = torch.cat([E2M1, mids, torch.tensor([6.5, 7.0, 100.0, 0.1, 0.24, 0.26])])
    ulp = torch.tensor([-1, 0, 1], dtype=torch.int32)
    grid = (pts.view(torch.int32)[:, None] + ulp[None, :]).view(torch.float32).reshape(-1)
    grid = torch.cat([grid[grid == grid], -grid[grid == grid], torch.linspace(-8, 8, 801)])
    got = torch.tensor([L.ao_f32_to_e2m1(float(v)) for v in grid.tolist()])
    assert torch.equal(got, e2m1_rne_bruteforce(grid))
    # ties: 0.25 -> 0, 0.75 -> 1, 1.25 -> 1, 1.75 -> 2, 2.5 -> 2, 3.5 -> 4, 5 -> 4; saturation; infinities
    assert [L.ao_f32_to_e2m1(v) for v in (0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0)] == [0, 2, 2, 4, 4, 6, 6]
    assert L.ao_f32_to_e2m1(1e30) == 7 and L.ao_f32_to_e2m1(float("-inf")) == 15
    # decode table == the reference test's LUT
    assert [L.ao_e2m1_to_f32(c) for c in range(8)] == E2M1.tolist()
    assert [L.ao_e2m1_to_f32(c + 8) for c in range(1, 8)] == (-E2M1[1:]).tolist()


def torch_fp4_reference(key, value, key_cache, value_cache, ksc, vsc, slots):
    """Closed form of the operator with torch routines (float8 cast, bucketize)."""
    is_nhd, bs, *_ = oracle.fp4_layout(key, key_cache)
    T, H, D = key.shape
    # thresholds with their tie direction: value > t goes up, except where the upper code is even
    bounds = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    up_on_tie = torch.tensor([False, True, False, True, False, True, False])
    for src, cache, sc in ((key, key_cache, ksc), (value, value_cache, vsc)):
        x = src.float().view(T, H, D // 16, 16)
        amax = x.abs().nan_to_num(nan=0.0).amax(-1)
        sf32 = amax * torch.tensor(1.0 / 6.0, dtype=torch.float32)
        code = sf32.clamp(max=448.0).to(torch.float8_e4m3fn)
        SF = code.float()
        inv = torch.where(SF != 0, 1.0 / SF, torch.zeros_like(SF))
        v = x * inv[..., None]
        a = v.abs()
        m = ((a[..., None] > bounds) | ((a[..., None] == bounds) & up_on_tie)).sum(-1)
        nib = (m | (torch.signbit(v).to(torch.int64) << 3)).to(torch.uint8).view(T, H, D // 2, 2)
        packed = nib[..., 0] | (nib[..., 1] << 4)
        for t in range(T):
            s = int(slots[t])
            if s < 0:
                continue
            if is_nhd:
                cache[s // bs, s % bs] = packed[t]
                sc[s // bs, s % bs] = code.view(torch.uint8)[t]
            else:
                cache[s // bs, :, s % bs] = packed[t]
                sc[s // bs, :, s % bs] = code.view(torch.uint8)[t]


def make_case(T, H, D, bs, NB, dtype, nhd, seed, std=0.5, pad=0.2):
    g = torch.Generator().manual_seed(seed)
    key = (torch.randn(T, H, D, generator=g) * std).to(dtype)
    value = (torch.randn(T, H, D, generator=g) * std).to(dtype)
    slots = torch.randperm(NB * bs, generator=g)[:T].to(torch.int64)
    slots[torch.randperm(T, generator=g)[: int(pad * T)]] = -1
    shape = (NB, bs, H) if nhd else (NB, H, bs)
    mk = lambda last: torch.randint(0, 256, (*shape, last), generator=g, dtype=torch.uint8)
    return key, value, mk(D // 2), mk(D // 2), mk(D // 16), mk(D // 16), slots


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("nhd", [True, False])
@pytest.mark.parametrize("shape", [(24, 4, 64, 8, 5), (9, 2, 128, 16, 2), (5, 1, 16, 4, 3)])
def test_matches_torch_closed_form(dtype, nhd, shape):
    T, H, D, bs, NB = shape
    key, value, kc, vc, ksc, vsc, slots = make_case(T, H, D, bs, NB, dtype, nhd, seed=3)
    want = [t.clone() for t in (kc, vc, ksc, vsc)]
    torch_fp4_reference(key, value, *want, slots)
    oracle.reshape_and_cache_flash_fp4(key, value, kc, vc, ksc, vsc, slots, "fp4", torch.tensor(0.0),
                                       torch.tensor(0.0))
    for g, w, name in zip((kc, vc, ksc, vsc), want, ("key", "value", "key scales", "value scales")):
        assert torch.equal(g, w), name


def test_dequantisation_error_bound_and_special_groups():
    T, H, D, bs, NB = 16, 2, 64, 16, 1
    key, value, kc, vc, ksc, vsc, slots = make_case(T, H, D, bs, NB, torch.float16, True, seed=9, pad=0.0)
    key[0, 0, :16] = 0.0                      # all-zero group: scale 0, all nibbles 0
    key[1, 0, :16] = 6.0 * 2.0 ** -3          # amax = 6 * 2^k: scale exactly 2^k, every value maps to +6
    key[2, 0, 0] = float("inf")               # infinite maximum saturates the scale at 448
    slots = torch.arange(T, dtype=torch.int64)
    oracle.reshape_and_cache_flash_fp4(key, value, kc, vc, ksc, vsc, slots, "fp4", torch.tensor(0.0),
                                       torch.tensor(0.0))
    assert int(ksc[0, 0, 0, 0]) == 0 and bool((kc[0, 0, 0, :8] == 0).all())
    assert float(oracle.e4m3fn_decode(ksc[0, 1, 0, 0:1])) == 2.0 ** -3 and bool((kc[0, 1, 0, :8] == 0x77).all())
    assert int(ksc[0, 2, 0, 0]) == 0x7E and int(kc[0, 2, 0, 0]) & 0xF == 7
    # decode the way the reference's test does and bound the error: the e2m1 grid has gaps of at
    # most 2 (between 4 and 6), the scale is within 1/16 of amax/6, so |x - deq| <= 1.07 * SF
    nib = torch.stack((vc & 0xF, vc >> 4), dim=-1).reshape(NB, bs, H, D)
    deq = oracle.e2m1_decode(nib) * oracle.e4m3fn_decode(vsc).repeat_interleave(16, dim=-1)
    x = value.float()[slots].view(NB, bs, H, D)
    SF = oracle.e4m3fn_decode(vsc).repeat_interleave(16, dim=-1)
    assert bool(((x - deq).abs() <= 1.07 * SF + 1e-6).all())
    rel_rmse = ((x - deq).pow(2).mean() / x.pow(2).mean()).sqrt()
    assert rel_rmse < 0.12                    # ~4-bit quantisation noise


def test_padding_and_layout_strides():
    for nhd in (True, False):
        key, value, kc, vc, ksc, vsc, slots = make_case(12, 2, 32, 4, 4, torch.bfloat16, nhd, seed=4, pad=0.0)
        slots[:] = -1
        before = [t.clone() for t in (kc, vc, ksc, vsc)]
        oracle.reshape_and_cache_flash_fp4(key, value, kc, vc, ksc, vsc, slots, "fp4", torch.tensor(0.0),
                                           torch.tensor(0.0))
        assert all(torch.equal(a, b) for a, b in zip((kc, vc, ksc, vsc), before))
        # the scale cache is addressed with the packed cache's strides / 8
        assert [s // 8 for s in kc.stride()[:3]] == list(ksc.stride()[:3])
