"""GPU parity of the bulk KV-cache write against the CPU oracle: bit-exact.

The calls go through the module's wrapper functions, as the reference's callers do: for GPU tensors outside
torch.compile those call the C++ host layer directly (_host_ext -> C ABI of libarctic_mi355x.so); the same function is
what the dispatcher runs for torch.ops.arctic_inference.reshape_and_cache_flash_bulk, which
tests/test_gpu_graph_and_abi.py::test_reference_schemas_through_the_dispatcher calls explicitly.
"""
import pytest
import torch

import oracle
from helpers import (assert_bulk_equal, bulk_args, bulk_case_to, bytes_of, make_bulk_case)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run_both(ops, case):
    dcase = bulk_case_to(case, DEV)
    ops.reshape_and_cache_flash_bulk(*bulk_args(dcase))
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    assert_bulk_equal(dcase["bufs"], case["bufs"])
    return dcase


def test_config1_bf16_passthrough(ops):
    # the CPU-runnable benchmark shape: 256 tokens, 16 layers, 8 KV heads x 128, block 16, 512 blocks, bf16 cache
    case = make_bulk_case(T=256, L=16, H=8, D=128, bs=16, NB=512, seed=0)
    run_both(ops, case)


@pytest.mark.parametrize("src_dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("kv", ["auto", "fp8", "fp8_e4m3", "fp8_e5m2"])
@pytest.mark.parametrize("shape", [
    dict(T=33, L=4, H=8, D=128, bs=16, NB=8),     # production row width
    dict(T=2, L=4, H=2, D=16, bs=16, NB=2),        # the reference unit test's sizes
    dict(T=17, L=3, H=1, D=128, bs=16, NB=4),      # TP-sharded single head
    dict(T=9, L=5, H=3, D=80, bs=8, NB=6),         # row chunk count not a power of two
    dict(T=5, L=2, H=1, D=20, bs=4, NB=3),         # not 16-byte divisible: element-wise kernel
    dict(T=7, L=70, H=2, D=64, bs=16, NB=2),       # more layers than one launch carries
])
def test_small_shapes(ops, src_dtype, kv, shape):
    case = make_bulk_case(src_dtype=src_dtype, kv_cache_dtype=kv, seed=11, std=1.5, pad_fraction=0.2, **shape)
    run_both(ops, case)


@pytest.mark.parametrize("kv", ["auto", "fp8"])
def test_flashinfer_layout_and_row_pitch(ops, kv):
    # K = cache[:, 0], V = cache[:, 1] (block stride 2*bs*n) and keys with a padded row pitch
    case = make_bulk_case(T=40, L=4, H=4, D=64, bs=16, NB=8, kv_cache_dtype=kv, seed=5, layout="flashinfer",
                          key_pad=24, pad_fraction=0.1)
    assert case["keys"].stride(0) != case["keys"].size(1)
    run_both(ops, case)


def test_all_padding_leaves_cache_untouched(ops):
    case = make_bulk_case(T=16, L=3, H=2, D=64, bs=16, NB=4, kv_cache_dtype="fp8", seed=7)
    case["slot_mapping"].fill_(-1)
    before = [b.clone() for b in case["bufs"]]
    dcase = bulk_case_to(case, DEV)
    ops.reshape_and_cache_flash_bulk(*bulk_args(dcase))
    torch.cuda.synchronize()
    assert_bulk_equal(dcase["bufs"], before)


def test_slots_outside_the_cache_move_nothing(ops):
    """A slot at or beyond num_blocks * block_size is skipped like a padding slot (the reference would
    write out of bounds); the other tokens are written as usual."""
    case = make_bulk_case(T=24, L=3, H=2, D=64, bs=16, NB=4, kv_cache_dtype="fp8", seed=8, pad_fraction=0.1)
    bad = [1, 7, 20]
    for t, slot in zip(bad, (4 * 16, 4 * 16 + 5, 1 << 40)):
        case["slot_mapping"][t] = slot
    dcase = bulk_case_to(case, DEV)
    ops.reshape_and_cache_flash_bulk(*bulk_args(dcase))
    torch.cuda.synchronize()
    case["slot_mapping"][bad] = -1           # what the oracle has to see to do the same
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    assert_bulk_equal(dcase["bufs"], case["bufs"])


def test_empty_inputs(ops):
    case = make_bulk_case(T=4, L=2, H=2, D=64, bs=16, NB=2, seed=1)
    dcase = bulk_case_to(case, DEV)
    # no layers: no-op (reference returns early)
    ops.reshape_and_cache_flash_bulk(dcase["keys"], dcase["values"], [], [], dcase["slot_mapping"], "auto", [], [],
                                     2, 64)
    # no tokens
    ops.reshape_and_cache_flash_bulk(dcase["keys"][:0], dcase["values"][:0], dcase["key_caches"],
                                     dcase["value_caches"], dcase["slot_mapping"][:0], "auto", dcase["k_scales"],
                                     dcase["v_scales"], 2, 64)
    torch.cuda.synchronize()
    assert_bulk_equal(dcase["bufs"], case["bufs"])


def _exhaustive_case(src_dtype, kv, scales):
    """Every 16-bit pattern appears once per layer: 64 tokens x 1024 elements."""
    L = len(scales)
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(src_dtype).view(64, 1024)
    case = make_bulk_case(T=64, L=L, H=8, D=128, bs=16, NB=4, src_dtype=src_dtype, kv_cache_dtype=kv, seed=3)
    case["keys"] = bits.repeat(1, L).contiguous()
    case["values"] = bits.flip(0).repeat(1, L).contiguous()
    case["k_scales"] = [torch.tensor(s, dtype=torch.float32) for s in scales]
    case["v_scales"] = [torch.tensor(s, dtype=torch.float32) for s in reversed(scales)]
    return case


SCALES = [1.0, 0.013392857, 0.1, 2.0 ** -7, 3.7, 1e-3, 447.9, 0.33333334, 5.9e-8 * 1e-31, 3.0e38]


@pytest.mark.parametrize("src_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("kv", ["fp8", "fp8_e5m2"])
def test_fp8_codes_exhaustive_16bit(ops, src_dtype, kv):
    """All 65 536 source bit patterns (incl. +-0, subnormals, +-inf, NaN) x 10 scales,
    among them a subnormal and a near-overflow scale."""
    case = _exhaustive_case(src_dtype, kv, SCALES)
    run_both(ops, case)


@pytest.mark.parametrize("scale", [0.0, float("inf"), -0.5, float("nan")])
def test_fp8_degenerate_scales(ops, scale):
    """x/0, x/inf, negative and NaN scales follow IEEE division. NaN codes are compared
    without their sign bit: the sign of a NaN produced by 0/0 is not defined by IEEE
    (x86 gives -NaN, the GPU +NaN), and the reference does not pin it either."""
    case = _exhaustive_case(torch.bfloat16, "fp8", [scale])
    dcase = bulk_case_to(case, DEV)
    ops.reshape_and_cache_flash_bulk(*bulk_args(dcase))
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    for g, w in zip(dcase["bufs"], case["bufs"]):
        gb, wb = bytes_of(g.cpu()), bytes_of(w)
        nan = (wb & 0x7F) == 0x7F
        assert torch.equal(gb[~nan], wb[~nan])
        assert torch.equal(gb[nan] & 0x7F, wb[nan] & 0x7F)


def test_fp8_from_fp32_rounding_boundaries(ops):
    """fp32 sources placed on and next to every e4m3 rounding boundary, scale 1 and a
    non-trivial scale chosen so that quotients land near boundaries too."""
    codes = torch.arange(0, 0x7F, dtype=torch.int64)
    vals = oracle.e4m3fn_decode(codes)                       # all finite non-negative values
    mids = (vals[:-1] + vals[1:]) / 2                        # exact in fp32
    pts = torch.cat([vals, mids, torch.tensor([448.0, 464.0, 480.0, 2.0 ** -10, 2.0 ** -11])])
    ulp = torch.tensor([-2, -1, 0, 1, 2], dtype=torch.int32)
    grid = (pts.view(torch.int32)[:, None] + ulp[None, :]).view(torch.float32).reshape(-1)
    grid = torch.cat([grid, -grid])
    n = 1024
    T = (grid.numel() + n - 1) // n
    flat = torch.zeros(T * n)
    flat[: grid.numel()] = grid
    scales = [1.0, 3.0, 0.7]
    case = make_bulk_case(T=T, L=len(scales), H=8, D=128, bs=16, NB=2, src_dtype=torch.float32,
                          kv_cache_dtype="fp8", seed=9)
    keys = torch.cat([flat.view(T, n) * s for s in scales], dim=1).contiguous()   # quotient ~ boundary
    case["keys"] = keys
    case["values"] = keys.flip(0).contiguous()
    case["k_scales"] = [torch.tensor(s, dtype=torch.float32) for s in scales]
    case["v_scales"] = [torch.tensor(s, dtype=torch.float32) for s in scales]
    run_both(ops, case)


def test_config2_fp8_prefill_chunk(ops):
    # the 8B prefill-chunk shape: 8192 tokens, 16 layers, fp8 cache with amax/448 scales
    case = make_bulk_case(T=8192, L=16, H=8, D=128, bs=16, NB=8192, kv_cache_dtype="fp8", seed=1, std=1.5)
    run_both(ops, case)


@pytest.mark.parametrize("kv", ["fp8", "auto"])
def test_long_prefill_launch_shape(ops, kv):
    """4096 tokens x 32 layers: takes the 512-lane x 2-chunk kernel shape used for long
    prefill launches; compared in full against the oracle."""
    case = make_bulk_case(T=4096, L=32, H=8, D=128, bs=16, NB=512, kv_cache_dtype=kv, seed=12, std=1.5,
                          pad_fraction=0.05)
    run_both(ops, case)


@pytest.mark.parametrize("T,L,kv", [
    (300, 41, "fp8"),    # three layer groups per token, the last one a layer short (14 + 14 + 13)
    (300, 41, "auto"),
    (96, 70, "fp8"),     # two launches (64 + 6 layers); the first splits into four groups of 16
    (2100, 23, "fp8_e5m2"),   # two groups of 12 and 11 layers
])
def test_layer_groups_with_a_ragged_tail(ops, T, L, kv):
    """Layers of one token split over several workgroups of the 512-lane shape, layer count not a
    multiple of the group size; compared in full against the oracle."""
    case = make_bulk_case(T=T, L=L, H=8, D=128, bs=16, NB=(T + 15) // 16 + 3, kv_cache_dtype=kv, seed=31, std=1.5,
                          pad_fraction=0.1)
    run_both(ops, case)


def test_random_configurations(ops):
    """Seeded sweep over shapes, dtypes, layouts, pitches and padding: exercises the layer
    grouping, the power-of-two and general row decompositions, the multi-launch split and
    the element-wise fallback against the oracle."""
    import random
    rnd = random.Random(2024)
    for it in range(40):
        H = rnd.choice([1, 2, 3, 4, 8])
        D = rnd.choice([16, 32, 64, 80, 96, 128, 20])
        cfg = dict(T=rnd.choice([1, 2, 7, 33, 130, 600]), L=rnd.choice([1, 2, 5, 16, 33, 64, 65, 100]), H=H, D=D,
                   bs=rnd.choice([1, 4, 16, 32]), NB=0,
                   src_dtype=rnd.choice([torch.bfloat16, torch.float16, torch.float32]),
                   kv_cache_dtype=rnd.choice(["auto", "fp8", "fp8_e5m2"]), seed=1000 + it, std=rnd.choice([0.1, 1.5, 30.0]),
                   pad_fraction=rnd.choice([0.0, 0.1, 0.5]), layout=rnd.choice(["flash", "flashinfer"]),
                   key_pad=rnd.choice([0, 0, 8, 24, 3]))
        cfg["NB"] = (cfg["T"] + cfg["bs"] - 1) // cfg["bs"] + rnd.choice([0, 1, 5])
        if cfg["T"] * cfg["L"] * H * D > 40_000_000:
            cfg["L"] = max(1, 40_000_000 // (cfg["T"] * H * D))
        try:
            run_both(ops, make_bulk_case(**cfg))
        except AssertionError as e:
            raise AssertionError(f"configuration {it}: {cfg}: {e}") from None


def test_config3_shape_properties(ops):
    """The 70B SwiftKV shape at full size (16384 tokens, 40 layers, 10 % padding): too large
    for the CPU oracle in seconds, so it is checked through size-independent properties:
    rows of padded tokens and unaddressed slots keep their sentinel, a random sample of
    tokens matches the oracle bit for bit, and the write is idempotent."""
    T, L, H, D, bs, NB = 16384, 40, 8, 128, 16, 8192
    n = H * D
    dev = torch.device(DEV)
    g = torch.Generator().manual_seed(2)
    gd = torch.Generator(device=dev).manual_seed(2)
    # generated on the GPU (1.3 GB per tensor); the sampled rows are copied back for the oracle
    dkeys = torch.empty(T, L * n, dtype=torch.bfloat16, device=dev)
    dvalues = torch.empty(T, L * n, dtype=torch.bfloat16, device=dev)
    for t0 in range(0, T, 2048):
        dkeys[t0:t0 + 2048] = (torch.randn(2048, L * n, generator=gd, device=dev) * 1.5).to(torch.bfloat16)
        dvalues[t0:t0 + 2048] = (torch.randn(2048, L * n, generator=gd, device=dev) * 1.5).to(torch.bfloat16)
    from helpers import make_slots
    slots = make_slots(T, NB * bs, g, pad_fraction=0.1)
    assert int((slots < 0).sum()) == 1638
    dks = [(dkeys[:, l * n:(l + 1) * n].float().abs().max() / 448.0) for l in range(L)]
    dvs = [(dvalues[:, l * n:(l + 1) * n].float().abs().max() / 448.0) for l in range(L)]
    k_scales, v_scales = [s.cpu() for s in dks], [s.cpu() for s in dvs]
    dslots = slots.to(dev)
    sentinel = 0xA5
    bufs = [torch.full((2, NB, bs, H, D), sentinel, dtype=torch.uint8, device=dev) for _ in range(L)]
    kc, vc = [b[0] for b in bufs], [b[1] for b in bufs]
    ops.reshape_and_cache_flash_bulk(dkeys, dvalues, kc, vc, dslots, "fp8", dks, dvs, H, D)
    torch.cuda.synchronize()

    valid = slots >= 0
    written = torch.zeros(NB * bs, dtype=torch.bool)
    written[slots[valid]] = True
    # (1) untouched rows: every row not addressed by a valid slot is still all-sentinel
    for l in (0, 17, 39):
        for c in (kc[l], vc[l]):
            rows = c.view(NB * bs, n)
            untouched = rows[(~written).to(dev)]
            assert bool((untouched == sentinel).all())
    # (2) sampled tokens against the oracle
    sample = torch.randperm(T, generator=g)[:96]
    sub_slots = slots[sample]
    remap = torch.full_like(sub_slots, -1)
    nvalid = int((sub_slots >= 0).sum())
    remap[sub_slots >= 0] = torch.arange(nvalid)
    obufs = [torch.zeros(2, (nvalid + bs - 1) // bs, bs, H, D, dtype=torch.uint8) for _ in range(L)]
    dsample = sample.to(dev)
    oracle.reshape_and_cache_flash_bulk(dkeys[dsample].cpu().contiguous(), dvalues[dsample].cpu().contiguous(),
                                        [b[0] for b in obufs], [b[1] for b in obufs], remap, "fp8",
                                        k_scales, v_scales, H, D)
    src_rows = sub_slots[sub_slots >= 0].to(dev)
    for l in range(L):
        for which in (0, 1):
            got = bufs[l][which].view(NB * bs, n)[src_rows].cpu()
            want = obufs[l][which].view(-1, n)[:nvalid]
            assert torch.equal(got, want), f"layer {l} {'KV'[which]} sample mismatch"
    # (3) idempotence: a second identical write changes nothing
    sums = [int(b.view(-1).to(torch.int64).sum()) for b in bufs[:4]]
    ops.reshape_and_cache_flash_bulk(dkeys, dvalues, kc, vc, dslots, "fp8", dks, dvs, H, D)
    torch.cuda.synchronize()
    assert sums == [int(b.view(-1).to(torch.int64).sum()) for b in bufs[:4]]


def test_errors(ops):
    case = make_bulk_case(T=4, L=2, H=2, D=64, bs=16, NB=2, seed=1)
    d = bulk_case_to(case, DEV)
    a = list(bulk_args(d))
    with pytest.raises(RuntimeError, match="Unsupported data type of kv cache"):
        ops.reshape_and_cache_flash_bulk(*a[:5], "int4", *a[6:])
    with pytest.raises(RuntimeError, match="Unsupported input type of kv cache"):
        ops.reshape_and_cache_flash_bulk(a[0].to(torch.float64), a[1].to(torch.float64), *a[2:])
    with pytest.raises(RuntimeError):
        ops.reshape_and_cache_flash_bulk(*a[:3], a[3][:1], *a[4:])          # list length mismatch
    with pytest.raises(RuntimeError, match="Long"):
        ops.reshape_and_cache_flash_bulk(*a[:4], a[4].to(torch.int32), *a[5:])
    with pytest.raises(RuntimeError, match="element size"):
        ops.reshape_and_cache_flash_bulk(*a[:5], "fp8", *a[6:])            # bf16 cache passed as fp8
    torch.cuda.synchronize()
    assert_bulk_equal(d["bufs"], case["bufs"])                              # nothing was written


def test_layers_that_do_not_look_like_layer_0_are_turned_away(ops):
    """The kernel takes one block stride, block count and block size for all layers; a layer that differs, or a scale
    that is not an fp32 device tensor, is an error here (the reference would write out of bounds).  Every layer is
    looked at on every call: the same wrong set must fail each time, and a good set must still work after a bad one."""
    case = make_bulk_case(T=6, L=3, H=2, D=64, bs=16, NB=4, kv_cache_dtype="fp8", seed=21)
    d = bulk_case_to(case, DEV)
    a = list(bulk_args(d))
    small = torch.zeros(2, 2, 16, 2, 64, dtype=torch.uint8, device=DEV)          # 2 blocks instead of 4
    for _ in range(2):
        with pytest.raises(RuntimeError, match="must share dtype, block stride, number of blocks"):
            ops.reshape_and_cache_flash_bulk(a[0], a[1], [a[2][0], small[0], a[2][2]], [a[3][0], small[1], a[3][2]], *a[4:])
        with pytest.raises(RuntimeError, match="must be float32"):
            ops.reshape_and_cache_flash_bulk(*a[:6], [a[6][0], a[6][1].double(), a[6][2]], *a[7:])
        with pytest.raises(RuntimeError, match="same device"):
            ops.reshape_and_cache_flash_bulk(*a[:7], [a[7][0].cpu(), a[7][1], a[7][2]], *a[8:])
        with pytest.raises(RuntimeError, match="at least 6 rows"):
            ops.reshape_and_cache_flash_bulk(a[0][:4], *a[1:])
        with pytest.raises(RuntimeError, match="384 columns"):
            ops.reshape_and_cache_flash_bulk(a[0][:, :256].contiguous(), *a[1:])
    run_both(ops, case)


def test_same_addresses_under_another_geometry_are_turned_away(ops):
    """A set of per-layer tensors that was accepted once says nothing about the next call: the same addresses can come
    back under another shape (a pool rebuilt after sleep / wake lands where the old one lay).  Layer 1 is a view of
    a LARGER allocation with twice the blocks at half the block stride, at the address a valid call has just used, so
    every write would stay inside its allocation whatever the check did; the call must be refused on the host."""
    L, H, D, bs, NB = 3, 2, 64, 16, 4
    case = make_bulk_case(T=6, L=L, H=H, D=D, bs=bs, NB=NB, kv_cache_dtype="fp8", seed=22)
    d = bulk_case_to(case, DEV)
    big = torch.zeros(4 * 2 * NB * bs * H * D, dtype=torch.uint8, device=DEV)       # twice what a layer needs
    as_layer = big[: 2 * NB * bs * H * D].view(2, NB, bs, H, D)
    as_layer.copy_(d["bufs"][1])
    d["bufs"][1], d["key_caches"][1], d["value_caches"][1] = as_layer, as_layer[0], as_layer[1]
    case_args = list(bulk_args(d))
    ops.reshape_and_cache_flash_bulk(*case_args)                                       # the valid call
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    torch.cuda.synchronize()
    assert_bulk_equal(d["bufs"], case["bufs"])
    before = big.clone()
    other = big[: 2 * 2 * NB * (bs // 2) * H * D].view(2, 2 * NB, bs // 2, H, D)      # same data_ptr, other geometry
    assert other[0].data_ptr() == as_layer[0].data_ptr()
    kc, vc = list(case_args[2]), list(case_args[3])
    kc[1], vc[1] = other[0], other[1]
    for _ in range(2):
        with pytest.raises(RuntimeError, match="must share dtype, block stride, number of blocks"):
            ops.reshape_and_cache_flash_bulk(case_args[0], case_args[1], kc, vc, *case_args[4:])
    # a scale of another type at the address of an accepted one
    ks = list(case_args[6])
    ks[1] = ks[1].view(torch.int32)
    with pytest.raises(RuntimeError, match="must be float32"):
        ops.reshape_and_cache_flash_bulk(*case_args[:6], ks, *case_args[7:])
    torch.cuda.synchronize()
    assert torch.equal(big, before)                                                     # nothing was launched
    ops.reshape_and_cache_flash_bulk(*case_args)                                       # and the valid set still works
    torch.cuda.synchronize()
    assert_bulk_equal(d["bufs"], case["bufs"])


def test_rows_narrower_than_the_layers_as_in_the_reference_unit_test(ops):
    """The reference reads row t at t * keys.stride(0) whatever keys.size(1) says, and its own unit test
    (tests/unit_tests/test_custom_ops.py:63-104) passes keys of shape [L * T, H * D] with 2-D caches [T, H * D]: 4 layers,
    2 tokens, 2 heads of 16, fp32, "auto".  Accepted here too (the last row read ends inside the tensor's storage)
    and equal to the oracle's flat formula; a tensor whose storage ends earlier is refused."""
    L, T, H, D = 4, 2, 2, 16
    g = torch.Generator().manual_seed(5)
    keys, values = torch.randn(L * T, H * D, generator=g), torch.randn(L * T, H * D, generator=g)
    kc = [torch.randn(T, H * D, generator=g) for _ in range(L)]
    vc = [torch.randn(T, H * D, generator=g) for _ in range(L)]
    slots = torch.randint(0, T, (T,), generator=g)
    scales = [torch.tensor(0.1) for _ in range(L)]
    dkc, dvc = [t.to(DEV) for t in kc], [t.to(DEV) for t in vc]
    dscales = [t.to(DEV) for t in scales]
    ops.reshape_and_cache_flash_bulk(keys.to(DEV), values.to(DEV), dkc, dvc, slots.to(DEV), "auto", dscales, dscales, H, D)
    oracle.reshape_and_cache_flash_bulk(keys, values, kc, vc, slots, "auto", scales, scales, H, D)
    torch.cuda.synchronize()
    for got, want in zip(dkc + dvc, kc + vc):
        assert torch.equal(got.cpu(), want)
    with pytest.raises(RuntimeError, match="128 columns"):
        ops.reshape_and_cache_flash_bulk(keys[:4].to(DEV), values.to(DEV), dkc, dvc, slots.to(DEV), "auto", dscales, dscales,
                                         H, D)


def test_prepared_layers_write_the_same_bytes_and_keep_their_tensors(ops):
    """prepare_bulk_kv_layers(...).write(...) against the plain operator and the oracle; the object holds its tensors
    (the caller's lists and views may go), sees scales updated in place, and refuses at construction what the operator
    refuses per call."""
    case = make_bulk_case(T=300, L=6, H=8, D=128, bs=16, NB=32, kv_cache_dtype="fp8", seed=80, std=1.5, pad_fraction=0.1)
    d = bulk_case_to(case, DEV)
    a = bulk_args(d)
    layers = ops.prepare_bulk_kv_layers(a[2], a[3], a[6], a[7])
    assert layers.num_layers == 6
    keep = [b.clone() for b in d["bufs"]]
    d["key_caches"], d["value_caches"] = None, None          # only the pool's own tensors stay with the caller
    del a
    layers.write(d["keys"], d["values"], d["slot_mapping"], "fp8", 8, 128)
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    assert_bulk_equal(d["bufs"], case["bufs"])
    # a scale changed in place is read by the next write (the kernel reads scales on the device)
    for b, k in zip(d["bufs"], keep):
        b.copy_(k)
    case2 = make_bulk_case(T=300, L=6, H=8, D=128, bs=16, NB=32, kv_cache_dtype="fp8", seed=80, std=1.5, pad_fraction=0.1)
    d["k_scales"][2].mul_(2.0)
    case2["k_scales"][2] = case2["k_scales"][2] * 2.0
    layers.write(d["keys"], d["values"], d["slot_mapping"], "fp8", 8, 128)
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case2))
    assert_bulk_equal(d["bufs"], case2["bufs"])
    # the per-call checks are the operator's
    with pytest.raises(RuntimeError, match="element size"):
        layers.write(d["keys"], d["values"], d["slot_mapping"], "auto", 8, 128)
    with pytest.raises(RuntimeError, match="Long"):
        layers.write(d["keys"], d["values"], d["slot_mapping"].int(), "fp8", 8, 128)
    with pytest.raises(RuntimeError, match="at least 300 rows"):
        layers.write(d["keys"][:10], d["values"], d["slot_mapping"], "fp8", 8, 128)
    # and so are the per-layer ones, at construction
    bufs = d["bufs"]
    small = torch.zeros(2, 2, 16, 8, 128, dtype=torch.uint8, device=DEV)
    with pytest.raises(RuntimeError, match="must share dtype, block stride, number of blocks"):
        ops.prepare_bulk_kv_layers([bufs[0][0], small[0]], [bufs[0][1], small[1]], d["k_scales"][:2], d["v_scales"][:2])
    with pytest.raises(RuntimeError, match="value_caches"):
        ops.prepare_bulk_kv_layers([bufs[0][0]], [], d["k_scales"][:1], d["v_scales"][:1])
    bad = ops.prepare_bulk_kv_layers([bufs[0][0]], [bufs[0][1]], [d["k_scales"][0].double()], d["v_scales"][:1])
    with pytest.raises(RuntimeError, match="must be float32"):          # the scales only matter to an fp8 write
        bad.write(d["keys"], d["values"], d["slot_mapping"], "fp8", 8, 128)
    # with the selection folded in: the rows index_select would give
    idx = torch.tensor([5, 299, 0, 5], device=DEV)
    k_out = torch.zeros(4, 6 * 1024, dtype=torch.bfloat16, device=DEV)
    v_out = torch.zeros_like(k_out)
    layers.write_select(d["keys"], d["values"], d["slot_mapping"], "fp8", 8, 128, idx, k_out, v_out)
    torch.cuda.synchronize()
    assert torch.equal(k_out, d["keys"].index_select(0, idx)) and torch.equal(v_out, d["values"].index_select(0, idx))
