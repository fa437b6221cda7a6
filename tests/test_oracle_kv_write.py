"""Pins the CPU oracle of the bulk KV write and of the fp8 encoder (no GPU needed).

The oracle restates the reference kernel; these tests check it against things the
reference does not supply itself (it ships no golden vectors for this path):
torch library routines that compute the same closed form (index_copy_, the CPU
float8 casts), brute force over every 16-bit input, exact rounding boundaries,
the reference test-suite's own e4m3 decoder, and the committed golden fixtures.
"""
import os

import numpy as np
import pytest
import torch

import oracle
from helpers import bulk_args, bytes_of, make_bulk_case

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def torch_bulk_reference(case):
    """Closed form with torch routines: per layer
    cache.view(-1, n).index_copy_(0, slots[valid], cvt(keys[valid, l*n:(l+1)*n]))."""
    n = case["num_heads"] * case["head_size"]
    slots = case["slot_mapping"]
    valid = slots >= 0
    kv = case["kv_cache_dtype"]
    out = [b.clone() for b in case["bufs"]]
    flash = case["layout"] == "flash"
    for l, buf in enumerate(out):
        for which, src, scales in ((0, case["keys"], case["k_scales"]), (1, case["values"], case["v_scales"])):
            x = src[valid][:, l * n:(l + 1) * n]
            if kv == "auto":
                rows = x
            else:
                tdt, mx = (torch.float8_e5m2, 57344.0) if kv == "fp8_e5m2" else (torch.float8_e4m3fn, 448.0)
                q = x.float() / scales[l].float()
                rows = q.clamp(-mx, mx).to(tdt).view(torch.uint8)
            cache = buf[which] if flash else buf[:, which]
            NB, bs = cache.shape[0], cache.shape[1]
            for t, slot in zip(range(rows.shape[0]), slots[valid].tolist()):
                cache[slot // bs, slot % bs] = rows[t].view(cache.shape[2], cache.shape[3])
    return out


@pytest.mark.parametrize("src_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("kv", ["auto", "fp8", "fp8_e5m2"])
@pytest.mark.parametrize("layout", ["flash", "flashinfer"])
def test_scatter_matches_torch_closed_form(src_dtype, kv, layout):
    case = make_bulk_case(T=37, L=3, H=2, D=32, bs=8, NB=7, src_dtype=src_dtype, kv_cache_dtype=kv, seed=4,
                          std=1.5, pad_fraction=0.25, layout=layout, key_pad=8)
    want = torch_bulk_reference(case)
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    for g, w in zip(case["bufs"], want):
        assert torch.equal(bytes_of(g), bytes_of(w))


def test_scatter_brute_force_tiny():
    """Element by element, straight from the kernel's index formula."""
    T, L, H, D, bs, NB = 5, 2, 2, 4, 2, 4
    n = H * D
    case = make_bulk_case(T=T, L=L, H=H, D=D, bs=bs, NB=NB, src_dtype=torch.float32, seed=6, pad_fraction=0.4)
    want = [b.clone() for b in case["bufs"]]
    for l in range(L):
        for t in range(T):
            slot = int(case["slot_mapping"][t])
            if slot < 0:
                continue
            for i in range(n):
                for which, src in ((0, case["keys"]), (1, case["values"])):
                    want[l][which].view(-1)[(slot // bs) * bs * n + (slot % bs) * n + i] = src[t, l * n + i]
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    for g, w in zip(case["bufs"], want):
        assert torch.equal(bytes_of(g), bytes_of(w))   # random sentinel bytes include NaN patterns


def test_padding_only_is_a_noop():
    case = make_bulk_case(T=8, L=2, H=2, D=16, bs=4, NB=4, kv_cache_dtype="fp8", seed=2)
    case["slot_mapping"].fill_(-1)
    before = [b.clone() for b in case["bufs"]]
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    for g, w in zip(case["bufs"], before):
        assert torch.equal(bytes_of(g), bytes_of(w))


SCALES = [1.0, 0.013392857, 0.1, 2.0 ** -7, 3.7, 1e-3, 447.9, 0.33333334]


@pytest.mark.parametrize("src_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kv,tdt,mx", [("fp8", torch.float8_e4m3fn, 448.0), ("fp8_e5m2", torch.float8_e5m2, 57344.0)])
def test_fp8_encoder_exhaustive_vs_torch(src_dtype, kv, tdt, mx):
    """All 65 536 inputs x 8 scales: oracle == clamp + torch's CPU float8 cast (RNE)."""
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(src_dtype)
    for s in SCALES:
        q = x.float() / torch.tensor(s, dtype=torch.float32)
        want = q.clamp(-mx, mx).to(tdt).view(torch.uint8)
        got = oracle.scaled_convert(x, s, kv)
        assert torch.equal(got, want), f"scale {s}"


def test_fp8_special_values():
    f = lambda v: int(oracle.scaled_convert(torch.tensor([v], dtype=torch.float32), 1.0, "fp8")[0])
    assert f(0.0) == 0x00 and f(-0.0) == 0x80
    for v in (448.0, 449.0, 464.0, 480.0, 1e9, float("inf")):
        assert f(v) == 0x7E and f(-v) == 0xFE          # saturate to +-448, never NaN
    assert f(float("nan")) & 0x7F == 0x7F
    assert f(2.0 ** -9) == 0x01                          # smallest subnormal
    assert f(2.0 ** -10) == 0x00                         # tie -> even (zero)
    assert f(2.0 ** -10 * 1.01) == 0x01
    assert f(0.9375 * 2 ** -6) == 0x08 and f(2.0 ** -6) == 0x08   # 7.5/8 ties up to the smallest normal
    assert f(1.0625) == 0x38 and f(1.1875) == 0x3A        # ties to even mantissa
    g = lambda v: int(oracle.scaled_convert(torch.tensor([v], dtype=torch.float32), 1.0, "fp8_e5m2")[0])
    assert g(57344.0) == 0x7B and g(1e9) == 0x7B and g(float("-inf")) == 0xFB
    assert g(2.0 ** -16) == 0x01 and g(2.0 ** -17) == 0x00


def test_fp8_rounding_boundaries_fp32():
    """+-2 fp32 ulps around every value and every midpoint of the e4m3 grid."""
    codes = torch.arange(0, 0x7F, dtype=torch.int64)
    vals = oracle.e4m3fn_decode(codes)
    mids = (vals[:-1] + vals[1:]) / 2
    pts = torch.cat([vals, mids])
    ulp = torch.tensor([-2, -1, 0, 1, 2], dtype=torch.int32)
    grid = (pts.view(torch.int32)[:, None] + ulp[None, :]).view(torch.float32).reshape(-1)
    grid = torch.cat([grid, -grid])
    want = grid.clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    got = oracle.scaled_convert(grid, 1.0, "fp8")
    assert torch.equal(got, want)
    # each midpoint itself goes to the even neighbour
    got_mid = oracle.scaled_convert(mids, 1.0, "fp8").to(torch.int64)
    lo = codes[:-1]
    assert torch.equal(got_mid, torch.where(lo % 2 == 0, lo, lo + 1))


def reference_test_decode_e4m3(code: int) -> float:
    """The e4m3 decoder the reference's own tests use
    (tests/unit_tests/test_reshape_and_cache_flash_nvfp4.py:25-45), restated."""
    sign = -1.0 if code & 0x80 else 1.0
    e, m = (code >> 3) & 0xF, code & 7
    if e == 0xF and m == 7:
        return float("nan")
    if e == 0:
        return sign * (m / 8.0) * 2.0 ** -6
    return sign * (1 + m / 8.0) * 2.0 ** (e - 7)


def test_fp8_decode_round_trip_and_monotone():
    codes = torch.arange(256, dtype=torch.int64)
    dec = oracle.e4m3fn_decode(codes)
    for c in range(256):
        r = reference_test_decode_e4m3(c)
        assert (np.isnan(r) and np.isnan(dec[c].item())) or r == dec[c].item()
    finite = ~torch.isnan(dec)
    enc = oracle.scaled_convert(dec[finite], 1.0, "fp8").to(torch.int64)
    assert torch.equal(enc, codes[finite])                    # encode(decode(c)) == c
    xs = torch.linspace(-500, 500, 200001)
    d = oracle.e4m3fn_decode(oracle.scaled_convert(xs, 1.0, "fp8"))
    assert bool((d[1:] >= d[:-1]).all())                      # monotone
    assert float((d - xs.clamp(-448, 448)).abs().max()) <= 16.0   # within half of the largest grid step
    codes5 = torch.arange(256, dtype=torch.int64)
    dec5 = oracle.e5m2_decode(codes5)
    fin5 = torch.isfinite(dec5)
    assert torch.equal(oracle.scaled_convert(dec5[fin5], 1.0, "fp8_e5m2").to(torch.int64), codes5[fin5])


def test_quotient_is_a_true_division():
    """x * (1/s) is NOT the reference arithmetic: make sure the oracle divides."""
    x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)
    x = x[torch.isfinite(x.float())]
    diff = 0
    for s in (0.013392857, 0.1, 3.7, 0.33333334):
        st = torch.tensor(s, dtype=torch.float32)
        got = oracle.scaled_convert(x, s, "fp8")
        wrong = (x.float() * (1.0 / st)).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
        diff += int((got != wrong).sum())
    assert diff > 0


def test_golden_bulk_fixtures():
    z = np.load(os.path.join(GOLDEN, "bulk_kv_write.npz"))
    for name in ("bf16_auto", "bf16_fp8", "f16_fp8_e5m2"):
        H, D, bs, NB, L = [int(v) for v in z[f"{name}.dims"]]
        src_dtype = torch.float16 if name.startswith("f16") else torch.bfloat16
        kv = {"auto": "auto", "fp8": "fp8", "e5m2": "fp8_e5m2"}[name.split("_")[-1]]
        keys = torch.from_numpy(z[f"{name}.keys"]).view(src_dtype)
        values = torch.from_numpy(z[f"{name}.values"]).view(src_dtype)
        slots = torch.from_numpy(z[f"{name}.slots"])
        init = torch.from_numpy(z[f"{name}.cache_init"])
        want = torch.from_numpy(z[f"{name}.cache_out"])
        cdt = torch.uint8 if kv != "auto" else src_dtype
        bufs = [init[l].clone().view(cdt).view(2, NB, bs, H, D) for l in range(L)]
        ks = [torch.tensor(float(v)) for v in z[f"{name}.k_scales"]]
        vs = [torch.tensor(float(v)) for v in z[f"{name}.v_scales"]]
        oracle.reshape_and_cache_flash_bulk(keys, values, [b[0] for b in bufs], [b[1] for b in bufs], slots, kv,
                                            ks, vs, H, D)
        for l in range(L):
            assert torch.equal(bytes_of(bufs[l]).view(-1), want[l].view(-1)), f"{name} layer {l}"
