"""GPU parity of the NVFP4-style cache write against the CPU oracle: bit-exact (the oracle and
the kernel use the same correctly rounded reciprocals)."""
import pytest
import torch

import oracle
from test_oracle_fp4 import make_case

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ZERO = torch.tensor(0.0)


def run_both(ops, key, value, kc, vc, ksc, vsc, slots):
    d = [t.to(DEV) for t in (key, value, kc, vc, ksc, vsc, slots)]
    ops.reshape_and_cache_flash_fp4(d[0], d[1], d[2], d[3], d[4], d[5], d[6], "fp4", ZERO.to(DEV), ZERO.to(DEV))
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_fp4(key, value, kc, vc, ksc, vsc, slots, "fp4", ZERO, ZERO)
    for got, want, name in zip(d[2:6], (kc, vc, ksc, vsc), ("key cache", "value cache", "key scales", "value scales")):
        g = got.cpu()
        if not torch.equal(g, want):
            bad = (g != want).nonzero()
            raise AssertionError(f"{name}: {bad.shape[0]} bytes differ, first at {bad[0].tolist()}: "
                                 f"got {int(g[tuple(bad[0])])} want {int(want[tuple(bad[0])])}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("nhd", [True, False])
@pytest.mark.parametrize("shape", [
    (64, 16, 128, 16, 4),      # the reference test's sizes (tests/unit_tests/test_reshape_and_cache_flash_nvfp4.py:85-90)
    (256, 8, 64, 32, 8),
    (33, 8, 128, 16, 3),
    (5, 1, 16, 4, 3),
])
def test_random(ops, dtype, nhd, shape):
    T, H, D, bs, NB = shape
    run_both(ops, *make_case(T, H, D, bs, NB, dtype, nhd, seed=21))


@pytest.mark.parametrize("nhd", [True, False])
@pytest.mark.parametrize("shape", [
    (2050, 8, 128, 16, 130),   # thousands of tokens: a last workgroup that is partly idle
    (2051, 3, 80, 4, 520),     # rows that are no multiple of a wave's 64 groups
    (4096, 32, 128, 16, 256),  # rows wider than one workgroup
])
def test_many_tokens(ops, nhd, shape):
    T, H, D, bs, NB = shape
    run_both(ops, *make_case(T, H, D, bs, NB, torch.bfloat16, nhd, seed=31, pad=0.15))


@pytest.mark.parametrize("nhd", [True, False])
def test_slots_outside_the_cache_move_nothing(ops, nhd):
    key, value, kc, vc, ksc, vsc, slots = make_case(20, 4, 64, 8, 3, torch.bfloat16, nhd, seed=23)
    bad = [2, 11]
    d = [t.to(DEV) for t in (key, value, kc, vc, ksc, vsc, slots)]
    d[6][bad[0]], d[6][bad[1]] = 3 * 8, 1 << 35          # first slot past the end, and far past it
    ops.reshape_and_cache_flash_fp4(d[0], d[1], d[2], d[3], d[4], d[5], d[6], "fp4", ZERO.to(DEV), ZERO.to(DEV))
    torch.cuda.synchronize()
    slots[bad] = -1                                       # what the oracle has to see to do the same
    oracle.reshape_and_cache_flash_fp4(key, value, kc, vc, ksc, vsc, slots, "fp4", ZERO, ZERO)
    for got, want in zip(d[2:6], (kc, vc, ksc, vsc)):
        assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_every_finite_sixteen_bit_value(ops, dtype):
    """All 16-bit patterns as inputs (NaN patterns replaced by 0: the NaN nibble is unpinned),
    in groups whose maximum is also forced through every magnitude."""
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
    x = torch.where(torch.isnan(bits.float()), torch.zeros_like(bits), bits)
    g = torch.Generator().manual_seed(5)
    x = x[torch.randperm(65536, generator=g)]
    T, H, D = 64, 8, 128
    key = x.view(T, H, D).clone()
    value = (x.float() * 3.0e-3).to(dtype).view(T, H, D)      # a second pass at a different magnitude
    _, _, kc, vc, ksc, vsc, _ = make_case(T, H, D, 16, 4, dtype, True, seed=6, pad=0.0)
    slots = torch.randperm(64, generator=g).to(torch.int64)
    run_both(ops, key, value, kc, vc, ksc, vsc, slots)


@pytest.mark.parametrize("nhd,bs", [(True, 16), (False, 8)])
def test_dequantised_cache_against_the_fp16_rows_as_in_the_reference_test(ops, nhd, bs):
    """The check of the reference's own test (tests/unit_tests/test_reshape_and_cache_flash_nvfp4.py:77-196) on the
    kernel's output, with its sizes and inputs (64 tokens, 16 heads x 128, blocks of 16, randn * 0.5 in fp16,
    slot t = t, zeroed caches): the cache is decoded with the test's formulas (e2m1 nibbles times the e4m3 group
    scale) and compared with the rows an fp16 cache would hold.  The reference prints the error; here it is bounded:
    the e2m1 grid has gaps of at most 2 and the scale is within 1/16 of amax / 6, so |x - decoded| <= 1.07 * scale,
    and the relative RMS error is that of a 4-bit code.  (Heads-first caches with blocks of 8: with as many heads as
    slots per block the operator, like the reference's, takes a cache for tokens-first.)"""
    T, H, D = 64, 16, 128
    NB = T // bs
    g = torch.Generator().manual_seed(0)
    key = (torch.randn(T, H, D, generator=g) * 0.5).to(torch.float16)
    value = (torch.randn(T, H, D, generator=g) * 0.5).to(torch.float16)
    slots = torch.arange(T, dtype=torch.int64)
    shape = (NB, bs, H) if nhd else (NB, H, bs)
    kc, vc = (torch.zeros(*shape, D // 2, dtype=torch.uint8, device=DEV) for _ in range(2))
    ksc, vsc = (torch.zeros(*shape, D // 16, dtype=torch.uint8, device=DEV) for _ in range(2))
    ops.reshape_and_cache_flash_fp4(key.to(DEV), value.to(DEV), kc, vc, ksc, vsc, slots.to(DEV), "fp4", ZERO.to(DEV),
                                    ZERO.to(DEV))
    torch.cuda.synchronize()
    for src, cache, scales in ((key, kc.cpu(), ksc.cpu()), (value, vc.cpu(), vsc.cpu())):
        if not nhd:   # [blocks, heads, block, bytes] -> [blocks, block, heads, bytes]
            cache, scales = cache.transpose(1, 2), scales.transpose(1, 2)
        packed = cache.reshape(T, H, D // 2)              # slot t = t: token t sits in block t / bs at offset t % bs
        group_scale = oracle.e4m3fn_decode(scales.reshape(T, H, D // 16)).repeat_interleave(16, dim=-1)
        nibbles = torch.stack((packed & 0xF, packed >> 4), dim=-1).reshape(T, H, D)
        decoded = oracle.e2m1_decode(nibbles) * group_scale
        x = src.float()
        assert bool(((x - decoded).abs() <= 1.07 * group_scale + 1e-6).all())
        assert float(((x - decoded).pow(2).mean() / x.pow(2).mean()).sqrt()) < 0.12
        # what the reference's test prints: mean and largest absolute error against the fp16 rows
        assert float((x - decoded.to(torch.float16).float()).abs().mean()) < 0.05
        assert float((x - decoded.to(torch.float16).float()).abs().max()) < 0.5


def test_rounding_ties(ops):
    """Groups whose scale is an exact power of two, holding every e2m1 tie and its neighbours."""
    ties = torch.tensor([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0])
    ulp = torch.tensor([-1, 0, 1], dtype=torch.int32)
    pts = (ties.view(torch.int32)[:, None] + ulp[None, :]).view(torch.float32).reshape(-1)   # 21 values
    pts = torch.cat([pts, -pts])[:30]
    T, H, D = 8, 2, 32
    key = torch.zeros(T * H * D // 16, 16)
    for r in range(key.shape[0]):
        k = r % 5 - 2
        key[r, 0] = 6.0 * 2.0 ** k                      # forces SF = 2^k exactly
        key[r, 1:] = pts[(torch.arange(15) + r) % 30] * 2.0 ** k
    key = key.view(T, H, D)
    for dtype in (torch.float16, torch.bfloat16):
        _, _, kc, vc, ksc, vsc, _ = make_case(T, H, D, 8, 1, dtype, True, seed=8, pad=0.0)
        run_both(ops, key.to(dtype), (-key).to(dtype), kc, vc, ksc, vsc, torch.arange(T, dtype=torch.int64))


def test_errors(ops):
    key, value, kc, vc, ksc, vsc, slots = [t.to(DEV) for t in make_case(4, 2, 32, 4, 2, torch.bfloat16, True, seed=1)]
    z = ZERO.to(DEV)
    with pytest.raises(RuntimeError, match="Must be half or bfloat16"):
        ops.reshape_and_cache_flash_fp4(key.float(), value.float(), kc, vc, ksc, vsc, slots, "fp4", z, z)
    with pytest.raises(RuntimeError, match="KV cache must be rank-4"):
        ops.reshape_and_cache_flash_fp4(key, value, kc[0], vc[0], ksc, vsc, slots, "fp4", z, z)
    with pytest.raises(RuntimeError, match="block_stride mismatch"):
        ops.reshape_and_cache_flash_fp4(key, value, kc, torch.cat([vc, vc], dim=1), ksc, vsc, slots, "fp4", z, z)


def test_random_configurations(ops):
    """Seeded sweep over token counts, head counts, head sizes (powers of two and not), block sizes, both layouts,
    both types and value ranges from denormal-sized to overflowing."""
    import random
    rnd = random.Random(17)
    for it in range(40):
        T, H = rnd.choice([1, 2, 7, 33, 130, 600]), rnd.choice([1, 2, 3, 8])
        D, bs = rnd.choice([16, 32, 48, 64, 80, 128]), rnd.choice([1, 4, 16, 32])
        NB = (T + bs - 1) // bs + rnd.choice([0, 1, 5])
        dtype, nhd = rnd.choice([torch.float16, torch.bfloat16]), rnd.choice([True, False])
        std = rnd.choice([1e-6, 0.01, 0.5, 30.0, 3000.0])
        try:
            run_both(ops, *make_case(T, H, D, bs, NB, dtype, nhd, seed=900 + it, std=std, pad=rnd.choice([0.0, 0.2, 0.6])))
        except AssertionError as e:
            raise AssertionError(f"configuration {it}: T={T} H={H} D={D} bs={bs} NB={NB} {dtype} nhd={nhd} std={std}: {e}") from None
