#!/usr/bin/env python3
"""Benchmark of the csrc/custom_ops hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one bulk KV-cache write (one launch of the hot path) over the 70B
SwiftKV shape (the benchmark's headline workload): 16384 tokens, 40 layers, 8 KV heads
x 128, block 16, fp8-e4m3 cache with per-tensor amax/448 scales, 10 % of the
slots are padding.  Inputs are resident in HBM before the timed region.

The caches sit where they sit in the serving process the shape comes from
(Llama-3.3-70B SwiftKV, fp8, one MI355X): the resident weights are allocated first
(66 GiB, a placeholder that is never touched), then vLLM's paged KV pool, one
[2, num_blocks, 16, 8, 128] tensor per layer for all 80 layers (65536 blocks =
2 GiB per layer), and the bulk write fills the upper 40 layers, as
llama_swiftkv.py:599-622 does.  This matters on MI355X: its HBM answers in three
address regions of 96 GiB, stores into one region top out near 4.9 TB/s while stores
spread over two or three reach 6.9 TB/s, so the same kernel is 15-20 % slower when
every cache is packed into the first 13 GiB of an otherwise empty GPU.  That
compact placement is measured too and reported under extras.

The last stdout line is ONE JSON object:

  value / ms_per_step   wall clock around exactly K steps (sync on both sides)
  roofline              the kernel's own duration from HIP events recorded on the
                        stream it is launched on, against the 8 TB/s HBM peak
  cpu_baseline          the CPU oracle (a C port of the reference kernel, OpenMP)
                        timed on this machine's host cores on a bounded sample
  extras                the other workloads (8B prefill chunk, speculator ops, decode mix)

Only one GPU is used; --gpus N with N > 1 is refused.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import subprocess
import sys
import time

import torch

HBM_PEAK_GBS = 8000.0
ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_slots(num_tokens, num_slots, gen, pad_fraction):
    n_pad = int(pad_fraction * num_tokens)
    slots = torch.full((num_tokens,), -1, dtype=torch.int64)
    order = torch.randperm(num_tokens, generator=gen)
    valid = order[n_pad:]
    slots[valid] = torch.randperm(num_slots, generator=gen)[: valid.numel()]
    return slots


class BulkWorkload:
    """One bulk KV-write configuration, resident on the GPU."""

    def __init__(self, name, T, L, H, D, bs, NB, kv, pad_fraction, seed, std, dev, bufs=None, make_bufs=None):
        self.name, self.T, self.L, self.H, self.D, self.bs, self.NB, self.kv = name, T, L, H, D, bs, NB, kv
        n = H * D
        self.n = n
        g = torch.Generator().manual_seed(seed)
        gd = torch.Generator(device=dev).manual_seed(seed)
        self.keys = torch.empty(T, L * n, dtype=torch.bfloat16, device=dev)
        self.values = torch.empty(T, L * n, dtype=torch.bfloat16, device=dev)
        step = max(1, min(T, (1 << 24) // (L * n)))
        for t0 in range(0, T, step):
            t1 = min(T, t0 + step)
            self.keys[t0:t1] = (torch.randn(t1 - t0, L * n, generator=gd, device=dev) * std).to(torch.bfloat16)
            self.values[t0:t1] = (torch.randn(t1 - t0, L * n, generator=gd, device=dev) * std).to(torch.bfloat16)
        self.slots_cpu = make_slots(T, NB * bs, g, pad_fraction)
        self.slots = self.slots_cpu.to(dev)
        self.valid = int((self.slots_cpu >= 0).sum())
        quant = kv != "auto"
        cdt = torch.uint8 if quant else torch.bfloat16
        # bufs: the layers' [2, NB, bs, H, D] cache tensors when they already exist (a serving pool); make_bufs: a
        # function that allocates them now, behind the source
        if bufs is None:
            bufs = make_bufs() if make_bufs else [torch.zeros(2, NB, bs, H, D, dtype=cdt, device=dev) for _ in range(L)]
        self.bufs = bufs
        assert len(self.bufs) == L and tuple(self.bufs[0].shape) == (2, NB, bs, H, D) and self.bufs[0].dtype == cdt
        self.key_caches = [b[0] for b in self.bufs]
        self.value_caches = [b[1] for b in self.bufs]
        if quant:
            self.k_scales = [(self.keys[:, l * n:(l + 1) * n].float().abs().max() / 448.0) for l in range(L)]
            self.v_scales = [(self.values[:, l * n:(l + 1) * n].float().abs().max() / 448.0) for l in range(L)]
        else:
            self.k_scales = [torch.ones((), device=dev) for _ in range(L)]
            self.v_scales = [torch.ones((), device=dev) for _ in range(L)]
        # algorithmic bytes: read K+V once (2 B each), write the cache once (1 or 2 B each)
        self.bytes_per_unit = n * (4 + (2 if quant else 4))
        self.bytes = self.valid * L * self.bytes_per_unit

    def args(self):
        return (self.keys, self.values, self.key_caches, self.value_caches, self.slots, self.kv,
                self.k_scales, self.v_scales, self.H, self.D)


class ServingMemoryMap:
    """Device memory laid out as the serving process lays it out: resident weights first (a placeholder
    that is never touched), then one [2, num_blocks, block, heads, head_size] cache tensor per model
    layer, the way vLLM's FlashAttention backend allocates its paged pool.  SwiftKV's bulk write fills
    the layers from num_key_value_layers up (llama_swiftkv.py:599-622)."""

    def __init__(self, dev, weight_gib, model_layers, first_written_layer, NB, bs, H, D, cdt):
        self.weight_gib, self.model_layers, self.first_written_layer, self.NB = weight_gib, model_layers, first_written_layer, NB
        self.weights = torch.empty(weight_gib << 30, dtype=torch.uint8, device=dev)
        self.pool = [torch.empty(2, NB, bs, H, D, dtype=cdt, device=dev) for _ in range(model_layers)]
        self.pool_gib = sum(b.numel() * b.element_size() for b in self.pool) / 2 ** 30

    def written_layers(self):
        return self.pool[self.first_written_layer:]

    def describe(self):
        return (f"{self.weight_gib} GiB resident weights (placeholder) allocated first, then the paged KV pool of all "
                f"{self.model_layers} layers, {self.NB} blocks = {self.pool_gib / self.model_layers:.0f} GiB per layer "
                f"({self.pool_gib:.0f} GiB); layers {self.first_written_layer}-{self.model_layers - 1} are written; "
                f"K/V source allocated after the pool")


def kernel_stats(fn, steps, nbytes):
    us = event_times_us(fn, steps)
    m = statistics.median(us)
    return {"kernel_us": round(m, 2), "GBps": round(nbytes / m / 1e3, 1), "hbm_frac": round(nbytes / m / 1e3 / HBM_PEAK_GBS, 4)}


def warm_replays(replay, min_ms=15.0, max_replays=3000):
    """Replays until the GPU has been busy for min_ms.  The first milliseconds of back-to-back work behind an idle GPU
    run several per cent slower than the steady state (23.8 against 25.1 us for the 131 MB argmax), and every extra
    starts behind host-bound set-up; a serving loop is never in that state.  Bounded by time, so that a run under a
    counter-collecting profiler, where a replay takes milliseconds, stops after the first few."""
    t0, n = time.perf_counter(), 0
    while n < max_replays:
        for _ in range(5):
            replay()
        n += 5
        torch.cuda.synchronize()
        if (time.perf_counter() - t0) * 1e3 >= min_ms:
            break


def event_times_us(fn, iters):
    """Duration of each call of fn() from HIP events on the current stream."""
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(iters)]
    for i in range(iters):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    return [s.elapsed_time(e) * 1e3 for s, e in zip(starts, ends)]


def read_traffic(path):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE + WRITE_SIZE, scaled by
    a copy kernel of known size); the figure is kept next to the profile it came from, with the day it was
    measured and the commit of the library it was measured on.  Returns (bytes or None, {key: text})."""
    fields = {}
    try:
        with open(path) as f:
            for line in f:
                if "=" in line and not line.lstrip().startswith("#"):
                    key, value = line.split("=", 1)
                    fields[key.strip()] = value.strip()
    except OSError:
        return None, fields
    try:
        return int(float(fields["hbm_bytes_per_launch"].split()[0])), fields
    except (KeyError, ValueError):
        return None, fields


def cpu_baseline_bulk(w: BulkWorkload, target_seconds=10.0):
    """Time the CPU oracle on a sample of the workload's tokens (all layers)."""
    import oracle
    threads = oracle.num_threads()
    n, L = w.n, w.L

    def prepare(sample_tokens):
        g = torch.Generator().manual_seed(99)
        sample = torch.randperm(w.T, generator=g)[:sample_tokens]
        sub = w.slots_cpu[sample]
        nvalid = int((sub >= 0).sum())
        remap = torch.full_like(sub, -1)
        remap[sub >= 0] = torch.arange(nvalid)
        keys = w.keys[sample.to(w.keys.device)].cpu().contiguous()
        values = w.values[sample.to(w.keys.device)].cpu().contiguous()
        nb = (nvalid + w.bs - 1) // w.bs
        bufs = [torch.zeros(2, nb, w.bs, w.H, w.D, dtype=w.bufs[0].dtype) for _ in range(L)]
        ks = [s.cpu() for s in w.k_scales]
        vs = [s.cpu() for s in w.v_scales]

        def run():
            t0 = time.perf_counter()
            oracle.reshape_and_cache_flash_bulk(keys, values, [b[0] for b in bufs], [b[1] for b in bufs], remap,
                                                w.kv, ks, vs, w.H, w.D)
            return time.perf_counter() - t0

        return run, nvalid * L * w.bytes_per_unit

    run, nbytes = prepare(min(w.T, 128))          # calibration pass (also warms the library)
    rate = nbytes / run()
    tokens = int(min(w.T, max(128, target_seconds * rate / (L * w.bytes_per_unit))))
    run, nbytes = prepare(tokens)
    # passes over the sample until about target_seconds of CPU work have been timed
    total_dt, passes = 0.0, 0
    while total_dt < target_seconds and passes < 50:
        total_dt, passes = total_dt + run(), passes + 1
    return {
        "value": round(passes * nbytes / total_dt / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
        "sample": f"{passes} passes over {tokens} of {w.T} tokens x {L} layers of the same workload "
                  f"({passes * nbytes / 1e6:.0f} MB algorithmic) in {total_dt:.2f} s, C oracle with OpenMP",
        "cpu_model": cpu_model(),
        "note": "the reference has no CPU implementation of the bulk write (its fallback, llama_swiftkv.py:623-650, is "
                "vLLM's CUDA operator), so a port of its kernel is the only CPU form there is; the speculator operators, "
                "which do have a PyTorch fallback in the reference, are timed both ways in extras.speculator.cpu_baseline",
    }


def cpu_baseline_bulk_pytorch(w: BulkWorkload, layers=4, target_seconds=3.0):
    """The bulk write as PyTorch CPU operations on a sample: per layer
    cache_l.view(-1, n).index_copy_(0, slots[valid], cvt(keys[valid, l*n:(l+1)*n])) and the same for the values,
    cvt = (x.float() / scale).clamp(-448, 448).to(float8_e4m3fn).  The reference has no CPU form of this operator;
    this is how one would write it with library routines (it is the closed form the oracle is pinned against)."""
    n, L = w.n, min(layers, w.L)
    threads = torch.get_num_threads()

    def prepare(sample_tokens):
        g = torch.Generator().manual_seed(98)
        sample = torch.randperm(w.T, generator=g)[:sample_tokens]
        sub = w.slots_cpu[sample]
        valid = sub >= 0
        nvalid = int(valid.sum())
        dst = torch.randperm(nvalid, generator=g)
        keys = w.keys[:, : L * n][sample.to(w.keys.device)].cpu().contiguous()
        values = w.values[:, : L * n][sample.to(w.keys.device)].cpu().contiguous()
        nb = (nvalid + w.bs - 1) // w.bs
        caches = [torch.zeros(2, nb * w.bs, n, dtype=torch.uint8) for _ in range(L)]
        ks = [float(s) for s in w.k_scales[:L]]
        vs = [float(s) for s in w.v_scales[:L]]

        def cvt(x, scale):
            return (x.float() / scale).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)

        def run():
            t0 = time.perf_counter()
            for l in range(L):
                caches[l][0].index_copy_(0, dst, cvt(keys[valid, l * n:(l + 1) * n], ks[l]))
                caches[l][1].index_copy_(0, dst, cvt(values[valid, l * n:(l + 1) * n], vs[l]))
            return time.perf_counter() - t0

        return run, nvalid * L * w.bytes_per_unit

    run, nbytes = prepare(min(w.T, 256))
    run()
    rate = nbytes / run()
    tokens = int(min(w.T, max(256, 0.5 * rate / (L * w.bytes_per_unit))))     # about half a second per pass
    run, nbytes = prepare(tokens)
    total_dt, passes = 0.0, 0
    while total_dt < target_seconds and passes < 50:
        total_dt, passes = total_dt + run(), passes + 1
    return {
        "value": round(passes * nbytes / total_dt / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "pytorch",
        "sample": f"{passes} passes over {tokens} of {w.T} tokens x {L} of {w.L} layers of the same workload "
                  f"({passes * nbytes / 1e6:.0f} MB algorithmic) in {total_dt:.2f} s; per-layer fancy-index read, "
                  f"float division, clamp, float8_e4m3fn cast and index_copy_ with torch's intra-op threads",
        "cpu_model": cpu_model(),
    }


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline_speculator():
    """CPU baselines of the speculator operators at 512 x 4096 bf16, two kinds side by side:
    "pytorch": the reference's own PyTorch fallback (arctic_speculator.py:92-99, 784-806, restated in
    oracle/torch_fallback.py), in bf16 on the host cores with torch's intra-op threads - the CPU path the reference has;
    "port": the C oracle (OpenMP), a port of the reference's CUDA kernels."""
    import oracle
    from oracle.torch_fallback import speculator_ln_fallback, sum_lstm_fallback
    T, Hd = 512, 4096
    g = torch.Generator().manual_seed(3)
    rn = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16)
    s4, z4, pc, x = rn(T, 4 * Hd), rn(T, 4 * Hd), rn(T, Hd), rn(T, Hd)
    w, b = (1 + 0.02 * torch.randn(Hd, generator=g)).to(torch.bfloat16), (0.02 * torch.randn(Hd, generator=g)).to(torch.bfloat16)
    sw = 0.5 ** (0.5 / 3)
    alpha = ((1 - sw * sw) * (Hd / 2)) ** 0.5 / sw

    def time_calls(fn, seconds):
        fn()
        times = []
        t_end = time.perf_counter() + seconds
        while time.perf_counter() < t_end or len(times) < 5:
            t0 = time.perf_counter()
            fn()
            times.append(time.perf_counter() - t0)
        return round(statistics.median(times) * 1e6, 1), len(times)

    out = {"cpu_model": cpu_model(), "host_cores_visible": os.cpu_count()}
    port = {"kind": "port", "cores": oracle.num_threads(), "what": "C oracle with OpenMP (a port of the reference's kernels)"}
    for name, fn in (("sum_lstm", lambda: oracle.sum_lstm(s4, z4, pc, w, b, w, b, alpha, 1e-6, 1e-6, False)),
                     ("speculator_ln", lambda: oracle.speculator_ln(x, w, b, 1e-6))):
        port[name + "_us_per_call"], _ = time_calls(fn, 1.0)
    out["port"] = port
    threads = torch.get_num_threads()
    pt = {"kind": "pytorch", "cores": threads, "dtype": "bf16",
          "what": "the reference's PyTorch fallback (arctic_speculator.py:92-99, 784-806) on CPU tensors, "
                  f"torch {torch.__version__}, {threads} intra-op threads"}
    with torch.no_grad():
        for name, fn in (("sum_lstm", lambda: sum_lstm_fallback(s4, z4, pc, w, b, w, b, alpha, 1e-6, 1e-6, False)),
                         ("speculator_ln", lambda: speculator_ln_fallback(x, w, b, 1e-6))):
            pt[name + "_us_per_call"], calls = time_calls(fn, 4.0)
            pt[name + "_calls_timed"] = calls
    pt["sample"] = "whole calls at the full 512 x 4096 shape, median of the calls made in about 4 s per operator"
    out["pytorch"] = pt
    return out


def bench_decode_sizes(ops, dev, mem, steps):
    """The bulk write at decode batch sizes on the same memory map (40 layers, fp8, no padding): 640 MB of
    source sets rotated inside one HIP graph so that the K/V rows come from HBM, not from the last-level cache."""
    out = {}
    for T in (64, 256, 512, 2048):
        source_bytes = 2 * T * 40 * 1024 * 2
        sets = min(64, max(4, -(-640 * 2 ** 20 // source_bytes)))   # 640 MB of K/V rows in rotation
        ws = [BulkWorkload(f"decode-{T}", T, 40, 8, 128, 16, mem.NB, "fp8", 0.0, 20 + k, 1.5, dev,
                           bufs=mem.written_layers()) for k in range(sets)]
        rounds = max(1, (8192 // T) // sets)   # enough launches per replay that the replay's own start-up does not show

        def run():
            for _ in range(rounds):
                for w in ws:
                    ops.reshape_and_cache_flash_bulk(*w.args())
        run()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run()
        warm_replays(graph.replay)
        us = statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / (len(ws) * rounds)
        out[f"{T}_tokens"] = {"us_per_call_graph": round(us, 2), "GBps": round(ws[0].bytes / us / 1e3, 1),
                              "hbm_frac": round(ws[0].bytes / us / 1e3 / HBM_PEAK_GBS, 4)}
        del ws, graph
    return out


def bench_block_contiguous_slots(ops, dev, w, steps):
    """The headline launch with the slot pattern a paged allocator produces for a prefill chunk instead of the
    benchmark's random distinct slots: the chunk's tokens fill whole blocks in order (16 consecutive tokens = 16
    consecutive slots = 16 KiB of one layer's K cache), the blocks themselves lie anywhere in the pool; the same
    10 % of the tokens are padding.  Same source, same caches, same bytes."""
    g = torch.Generator().manual_seed(12)
    blocks = torch.randperm(w.NB, generator=g)[: (w.T + w.bs - 1) // w.bs]
    slots = (blocks[:, None] * w.bs + torch.arange(w.bs)[None, :]).reshape(-1)[: w.T].clone()
    slots[w.slots_cpu < 0] = -1
    slots_dev = slots.to(dev)
    args = list(w.args())
    args[4] = slots_dev
    f = lambda: ops.reshape_and_cache_flash_bulk(*args)
    for _ in range(5):
        f()
    return kernel_stats(f, steps, w.bytes)


def bench_reference_decomposition(ops, dev, w, mem, steps, library_us):
    """The same fp8 write in the launch decomposition of the reference's kernel (one workgroup per (layer, token), one
    element per lane per step, reshape_and_cache_flash_bulk.cu:12-60,133-135), written for this GPU in bench_floor.hip:
    what that decomposition costs on an MI355X, next to the library's kernel, on the same tensors.  First its bytes
    are compared with the library's on two of the written caches; then the headline launch is timed, and the launch
    of a 512-token decode batch with the K/V rows of 8 source sets in rotation inside a HIP graph (as
    bulk_fp8_70b_decode_sizes_serving_map measures the library)."""
    floor = load_floor_kernels()
    if floor is None:
        return "bench_floor.so is not built"

    def tables(v):
        table = lambda ts: torch.tensor([t.data_ptr() for t in ts], dtype=torch.int64, device=dev)
        return table(v.key_caches), table(v.value_caches), table(v.k_scales), table(v.v_scales)

    def launch(v, tabs):
        rc = floor.floor_write_per_layer_and_token(
            v.keys.data_ptr(), v.values.data_ptr(), tabs[0].data_ptr(), tabs[1].data_ptr(), v.slots.data_ptr(), v.T, v.L,
            v.key_caches[0].stride(0), v.keys.stride(0), v.values.stride(0), v.H, v.D, v.bs, tabs[2].data_ptr(),
            tabs[3].data_ptr(), torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc

    tabs = tables(w)
    # two of the caches, cleared (the pool is uninitialised memory), written by the library and kept; cleared again,
    # written by the other kernel and compared
    w.key_caches[0].zero_()
    w.value_caches[w.L - 1].zero_()
    ops.reshape_and_cache_flash_bulk(*w.args())
    want_k, want_v = w.key_caches[0].clone(), w.value_caches[w.L - 1].clone()
    w.key_caches[0].zero_()
    w.value_caches[w.L - 1].zero_()
    launch(w, tabs)
    identical = bool(torch.equal(w.key_caches[0], want_k) and torch.equal(w.value_caches[w.L - 1], want_v))
    del want_k, want_v
    out = {"identical_bytes": identical}
    for _ in range(3):
        launch(w, tabs)
    ref = kernel_stats(lambda: launch(w, tabs), max(5, steps // 4), w.bytes)
    out["70b_prefill_16384_tokens_serving_map"] = {"reference_decomposition": ref, "library_kernel_us": round(library_us, 2),
                                                   "library_is_faster_by": round(ref["kernel_us"] / library_us, 2)}
    T, sets = 512, 8
    ws = [BulkWorkload(f"decode-{T}", T, 40, 8, 128, 16, mem.NB, "fp8", 0.0, 20 + k, 1.5, dev, bufs=mem.written_layers())
          for k in range(sets)]
    per_set = [tables(v) for v in ws]
    rounds = 2
    times = {}
    for name, call in (("library", lambda v, t: ops.reshape_and_cache_flash_bulk(*v.args())),
                       ("reference_decomposition", launch)):
        def run():
            for _ in range(rounds):
                for v, t in zip(ws, per_set):
                    call(v, t)
        run()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run()
        warm_replays(graph.replay)
        times[name] = statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / (sets * rounds)
        del graph
    out["decode_512_tokens_40_layers_serving_map"] = {
        "reference_decomposition": {"us_per_call_graph": round(times["reference_decomposition"], 2),
                                    "GBps": round(ws[0].bytes / times["reference_decomposition"] / 1e3, 1),
                                    "hbm_frac": round(ws[0].bytes / times["reference_decomposition"] / 1e3 / HBM_PEAK_GBS, 4)},
        "library_us_per_call_graph": round(times["library"], 2),
        "library_is_faster_by": round(times["reference_decomposition"] / times["library"], 2)}
    out["note"] = ("kernel time only: the reference's launcher also copies four pointer tables to the device with a "
                   "synchronous copy each on every call (reshape_and_cache_flash_bulk.cu:121-131), which this comparison "
                   "leaves out")
    return out


def load_floor_kernels():
    """bench_floor.so: bare kernels that move the same bytes as the library's and compute nothing
    (built by __graft_entry__.build()).  None when it has not been built."""
    import ctypes
    path = os.path.join(ROOT, "bench_floor.so")
    if not os.path.exists(path):
        return None
    lib = ctypes.CDLL(path)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    lib.floor_lstm_traffic.argtypes = [vp, vp, vp, vp, vp, i64, i32, vp]
    lib.floor_lstm_traffic_staged.argtypes = [vp, vp, vp, vp, vp, i64, i32, vp]
    lib.floor_ln_traffic.argtypes = [vp, vp, i64, i32, vp]
    lib.floor_fp4_traffic.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i32, vp]
    lib.floor_stream_resident.argtypes = [vp, vp, i32, i64, i32, i32, i32, i32, vp]
    lib.floor_stream.argtypes = [vp, i32, vp, i32, i64, i32, vp, vp]
    lib.floor_valu_rate.argtypes = [i32, i32, i32, vp, vp]
    lib.floor_node.argtypes = [vp, vp, i32, i32, i32, vp]
    lib.floor_row_read.argtypes = [vp, i64, i64, i32, vp, vp]
    lib.floor_write_per_layer_and_token.argtypes = [vp, vp, vp, vp, vp, i64, i32, i64, i64, i64, i32, i32, i32, vp, vp, vp]
    f32 = ctypes.c_float
    lib.floor_sum_lstm_three_passes.argtypes = [vp] * 9 + [i64, i32, i64, i64, i64, i64, f32, f32, f32, vp]
    lib.floor_ln_two_passes.argtypes = [vp, vp, vp, vp, i64, i32, i64, f32, vp]
    return lib


def bench_speculator(ops, dev, steps, warmup):
    """Speculator workload: sum_lstm (3 chained steps) and the standalone LayerNorm at
    T=512, H=4096, bf16.  Eight buffer sets (> 256 MB in total) are rotated so that
    the inputs do not stay resident in the last-level cache between launches."""
    T, Hd, sets = 512, 4096, 8
    g = torch.Generator(device=dev).manual_seed(3)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev).to(torch.bfloat16)
    S = [[rn(T, 4 * Hd) for _ in range(3)] for _ in range(sets)]
    Z = [[rn(T, 4 * Hd) for _ in range(3)] for _ in range(sets)]
    C0 = [rn(T, Hd) for _ in range(sets)]
    X = [rn(T, Hd) for _ in range(sets)]
    vec = lambda m: (m + 0.02 * torch.randn(Hd, generator=g, device=dev)).to(torch.bfloat16)
    w_cell, b_cell, w_state, b_state = vec(1.0), vec(0.0), vec(1.0), vec(0.0)
    sw = 0.5 ** (0.5 / 3)
    alpha = ((1 - sw * sw) * (Hd / 2)) ** 0.5 / sw

    def lstm3(i):
        cell = C0[i % sets]
        for k in range(3):
            _, cell = ops.sum_lstm(S[i % sets][k], Z[i % sets][k], cell, w_cell, b_cell, w_state, b_state,
                                   alpha, 1e-6, 1e-6, False)

    def lstm3_shared_z(i):
        # the same three steps with the embedding row passed once ([T, H]) instead of repeated four times
        cell = C0[i % sets]
        for k in range(3):
            _, cell = ops.sum_lstm_shared_z(S[i % sets][k], Z[i % sets][k][:, :Hd], cell, w_cell, b_cell, w_state,
                                            b_state, alpha, 1e-6, 1e-6, False)

    # the embedding lookup in front of every step: forget_emb(last_tokens) of a 32000 x 4096 table
    table = rn(32000, Hd)
    IDS = [torch.randint(0, 32000, (T, 1), generator=g, device=dev) for _ in range(sets)]

    def lstm3_lookup_repeat(i):
        # as the reference's caller runs it: lookup, repeat(1, 1, 4), sum_lstm
        cell = C0[i % sets]
        for k in range(3):
            z4 = torch.nn.functional.embedding(IDS[(i + k) % sets], table).repeat(1, 1, 4)
            _, cell = ops.sum_lstm(S[i % sets][k], z4.flatten(0, 1), cell, w_cell, b_cell, w_state, b_state,
                                   alpha, 1e-6, 1e-6, False)

    def lstm3_embedded(i):
        cell = C0[i % sets]
        for k in range(3):
            _, cell = ops.sum_lstm_embedded(S[i % sets][k], table, IDS[(i + k) % sets], cell, w_cell, b_cell, w_state,
                                            b_state, alpha, 1e-6, 1e-6, False)

    def ln(i):
        ops.speculator_ln(X[i % sets], w_cell, b_cell, 1e-6)

    def add_ln_gelu(i):
        # the MLP / sum_rnn speculator's states.add_(z, alpha); gelu(ln(states)) in one launch
        ops.speculator_add_ln_gelu(X[i % sets], C0[i % sets], w_cell, b_cell, alpha, 1e-6)

    def add_ln_gelu_separate(i):
        s = X[i % sets]
        s.add_(C0[i % sets], alpha=1e-3)
        torch.nn.functional.gelu(ops.speculator_ln(s, w_cell, b_cell, 1e-6))

    floor = load_floor_kernels()
    OS = [torch.empty(T, Hd, dtype=torch.bfloat16, device=dev) for _ in range(2)]

    def lstm3_traffic_only(i):
        # the loads and stores of the three sum_lstm calls with no arithmetic between them
        stream = torch.cuda.current_stream().cuda_stream
        for k in range(3):
            floor.floor_lstm_traffic(S[i % sets][k].data_ptr(), Z[i % sets][k].data_ptr(), C0[i % sets].data_ptr(),
                                     OS[0].data_ptr(), OS[1].data_ptr(), T, Hd, stream)

    def lstm3_traffic_staged(i):
        # the same bytes requested in the stages of the library's kernel (each stage waits for what it would read)
        stream = torch.cuda.current_stream().cuda_stream
        for k in range(3):
            floor.floor_lstm_traffic_staged(S[i % sets][k].data_ptr(), Z[i % sets][k].data_ptr(), C0[i % sets].data_ptr(),
                                            OS[0].data_ptr(), OS[1].data_ptr(), T, Hd, stream)

    OC = [torch.empty(T, Hd, dtype=torch.bfloat16, device=dev) for _ in range(3)]

    def lstm3_three_passes(i, state_out=None):
        # the reference's kernel decomposition written for this GPU (bench_floor.hip): 128 lanes per row, three passes
        stream = torch.cuda.current_stream().cuda_stream
        cell = C0[i % sets]
        for k in range(3):
            rc = floor.floor_sum_lstm_three_passes(
                (state_out if state_out is not None else OS[0]).data_ptr(), OC[k].data_ptr(), S[i % sets][k].data_ptr(),
                Z[i % sets][k].data_ptr(), cell.data_ptr(), w_cell.data_ptr(), b_cell.data_ptr(), w_state.data_ptr(),
                b_state.data_ptr(), T, Hd, 4 * Hd, 4 * Hd, Hd, Hd, alpha, 1e-6, 1e-6, stream)
            assert rc == 0, rc
            cell = OC[k]

    def ln_two_passes(i, out=None):
        # the reference's kernel decomposition written for this GPU (bench_floor.hip): 256 lanes per row, two passes
        rc = floor.floor_ln_two_passes((out if out is not None else OS[0]).data_ptr(), X[i % sets].data_ptr(),
                                       w_cell.data_ptr(), b_cell.data_ptr(), T, Hd, Hd, 1e-6,
                                       torch.cuda.current_stream().cuda_stream)
        assert rc == 0, rc

    def ln_traffic_only(i):
        floor.floor_ln_traffic(X[i % sets].data_ptr(), OS[0].data_ptr(), T, Hd, torch.cuda.current_stream().cuda_stream)

    cases = [("sum_lstm", lstm3, 22 * Hd * T, 3),
             ("sum_lstm_shared_z", lstm3_shared_z, 16 * Hd * T, 3),
             ("lookup_repeat_sum_lstm_as_three_ops", lstm3_lookup_repeat, 16 * Hd * T, 3),
             ("sum_lstm_embedded", lstm3_embedded, 16 * Hd * T, 3),
             ("speculator_ln", ln, 4 * Hd * T, 1),
             ("speculator_add_ln_gelu", add_ln_gelu, 6 * Hd * T, 1),
             ("add_ln_gelu_as_three_ops", add_ln_gelu_separate, 6 * Hd * T, 1)]
    if floor is not None:
        cases.insert(1, ("sum_lstm_traffic_only_floor", lstm3_traffic_only, 22 * Hd * T, 3))
        cases.insert(2, ("sum_lstm_traffic_only_in_stages", lstm3_traffic_staged, 22 * Hd * T, 3))
        cases.append(("speculator_ln_traffic_only_floor", ln_traffic_only, 4 * Hd * T, 1))
        cases.insert(3, ("sum_lstm_reference_decomposition", lstm3_three_passes, 22 * Hd * T, 3))
        cases.append(("speculator_ln_reference_decomposition", ln_two_passes, 4 * Hd * T, 1))
    out = {}
    for name, fn, per_call, calls in cases:
        for i in range(warmup):
            fn(i)
        torch.cuda.synchronize()
        counter = iter(range(10 ** 9))
        us = event_times_us(lambda: fn(next(counter)), steps)
        med = statistics.median(us) / calls
        out[name] = {"us_per_call_eager": round(med, 2), "bytes_per_call": per_call}
        # the same loop inside one HIP graph: kernel time without host launch gaps
        graph = torch.cuda.CUDAGraph()
        reps = sets
        with torch.cuda.graph(graph):
            for i in range(reps):
                fn(i)
        warm_replays(graph.replay)
        us = event_times_us(graph.replay, max(10, steps))
        med = statistics.median(us) / (reps * calls)
        out[name].update({"us_per_call_graph": round(med, 2),
                          "GBps_graph": round(per_call / med / 1e3, 1),
                          "hbm_frac_graph": round(per_call / med / 1e3 / HBM_PEAK_GBS, 4)})
    if floor is not None:
        # the comparison kernel computes the same function: third step's state and cell against the library's, within
        # the operators' tolerance (1e-2 relative + 2e-2 absolute)
        cell = C0[0]
        for k in range(3):
            state, cell = ops.sum_lstm(S[0][k], Z[0][k], cell, w_cell, b_cell, w_state, b_state, alpha, 1e-6, 1e-6, False)
        lstm3_three_passes(0, state_out=OS[1])
        close = lambda a, b: bool(torch.allclose(a.float(), b.float(), rtol=1e-2, atol=2e-2))
        out["sum_lstm_reference_decomposition"]["within_tolerance_of_the_library"] = close(OS[1], state) and close(OC[2], cell)
        out["sum_lstm_reference_decomposition"]["library_is_faster_by"] = round(
            out["sum_lstm_reference_decomposition"]["us_per_call_graph"] / out["sum_lstm"]["us_per_call_graph"], 2)
        ln_two_passes(0, out=OS[1])
        out["speculator_ln_reference_decomposition"]["within_tolerance_of_the_library"] = close(
            OS[1], ops.speculator_ln(X[0], w_cell, b_cell, 1e-6))
        out["speculator_ln_reference_decomposition"]["library_is_faster_by"] = round(
            out["speculator_ln_reference_decomposition"]["us_per_call_graph"] / out["speculator_ln"]["us_per_call_graph"], 2)
    return out


def bench_fp4(ops, dev, steps):
    """NVFP4-style cache write, one call per layer as the model would issue them: 8192 tokens,
    8 KV heads x 128, 16 layers (16 key/value tensors and caches, so nothing is re-used from cache).
    Algorithmic bytes per token and layer: 2 x 2n read + 2 x (n/2 + n/16) written = 5248 B."""
    T, H, D, bs, NB, L = 8192, 8, 128, 16, 8192, 16
    g = torch.Generator(device=dev).manual_seed(5)
    keys = [(torch.randn(T, H, D, generator=g, device=dev) * 0.5).to(torch.bfloat16) for _ in range(L)]
    values = [(torch.randn(T, H, D, generator=g, device=dev) * 0.5).to(torch.bfloat16) for _ in range(L)]
    kc = [torch.zeros(NB, bs, H, D // 2, dtype=torch.uint8, device=dev) for _ in range(L)]
    vc = [torch.zeros(NB, bs, H, D // 2, dtype=torch.uint8, device=dev) for _ in range(L)]
    ks = [torch.zeros(NB, bs, H, D // 16, dtype=torch.uint8, device=dev) for _ in range(L)]
    vs = [torch.zeros(NB, bs, H, D // 16, dtype=torch.uint8, device=dev) for _ in range(L)]
    slots = torch.randperm(NB * bs, generator=torch.Generator().manual_seed(5))[:T].to(dev)
    z = torch.zeros((), device=dev)

    def step():
        for l in range(L):
            ops.reshape_and_cache_flash_fp4(keys[l], values[l], kc[l], vc[l], ks[l], vs[l], slots, "fp4", z, z)

    def per_layer(fn):
        for _ in range(3):
            fn()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            fn()
        warm_replays(graph.replay)
        return statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / L

    med = per_layer(step)
    nbytes = T * (4 * H * D + 2 * (H * D // 2 + H * D // 16))
    out = {"us_per_layer_graph": round(med, 2), "bytes_per_layer": nbytes, "GBps": round(nbytes / med / 1e3, 1),
           "hbm_frac": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4)}
    floor = load_floor_kernels()
    if floor is not None:   # the same loads and stores (both caches contiguous), nothing computed
        def traffic():
            st = torch.cuda.current_stream().cuda_stream
            for l in range(L):
                rc = floor.floor_fp4_traffic(keys[l].data_ptr(), values[l].data_ptr(), kc[l].data_ptr(), vc[l].data_ptr(),
                                             ks[l].data_ptr(), vs[l].data_ptr(), slots.data_ptr(), T, H * D // 16, st)
                assert rc == 0, rc
        out["traffic_only_us_per_layer_graph"] = round(per_layer(traffic), 2)
    return out


def bench_row_gather(ops, dev, steps):
    """swiftkv_select of a decode-only batch at the 70B shape (llama_swiftkv.py:663-679): 512 rows of
    hidden_states and residual (8192 bf16), positions (int64), k_states and v_states (40 layers x 1024 bf16)
    gathered by logits_indices into the decode buffers; one launch against torch's five index_select calls.
    Four rotating sets (800 MB) keep the rows out of the last-level cache."""
    T, hidden, kvw, sets = 512, 8192, 40 * 1024, 4
    g = torch.Generator(device=dev).manual_seed(6)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev).to(torch.bfloat16)
    src = [[rn(T, hidden), rn(T, hidden), torch.arange(T, device=dev), rn(T, kvw), rn(T, kvw)] for _ in range(sets)]
    dst = [[torch.empty_like(t) for t in s] for s in src]
    idx = torch.arange(T, device=dev)
    nbytes = 2 * sum(t.numel() * t.element_size() for t in src[0])

    def fused(i):
        ops.gather_rows(src[i % sets], idx, dst[i % sets])

    def separate(i):
        for t, o in zip(src[i % sets], dst[i % sets]):
            torch.index_select(t, 0, idx, out=o)

    out = {"bytes_per_call": nbytes}
    for name, fn in (("gather_rows", fused), ("five_index_select", separate)):
        for i in range(3):
            fn(i)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(sets):
                fn(i)
        warm_replays(graph.replay)
        med = statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / sets
        out[name] = {"us_per_call_graph": round(med, 2), "GBps": round(nbytes / med / 1e3, 1),
                     "hbm_frac": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4)}
    return out


def bench_bulk_select(ops, dev, steps):
    """The bulk write and swiftkv_select of a decode-only batch together (llama_swiftkv.py:617-622, 663-679):
    512 tokens, 40 layers x 8 x 128, fp8 cache of 8192 blocks per layer; hidden_states and residual 8192 bf16.
    As the reference's caller runs them (bulk write + five index_select), with gather_rows for the five, and
    with the K/V selection folded into the bulk write (k_states / v_states read once).  Four rotating sets."""
    T, L, H, D, bs, NB, hidden, sets = 512, 40, 8, 128, 16, 8192, 8192, 4
    n = H * D
    g = torch.Generator(device=dev).manual_seed(8)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev).to(torch.bfloat16)
    bufs = [torch.zeros(2, NB, bs, H, D, dtype=torch.uint8, device=dev) for _ in range(L)]
    kc, vc = [b[0] for b in bufs], [b[1] for b in bufs]
    sc = [torch.tensor([0.02], device=dev) for _ in range(L)]
    K, V = [rn(T, L * n) for _ in range(sets)], [rn(T, L * n) for _ in range(sets)]
    Hs, Rs = [rn(T, hidden) for _ in range(sets)], [rn(T, hidden) for _ in range(sets)]
    P = torch.arange(T, device=dev)
    S = [torch.randperm(NB * bs, generator=g, device=dev)[:T] for _ in range(sets)]
    idx = torch.arange(T, device=dev)
    ob = [torch.empty(T, hidden, dtype=torch.bfloat16, device=dev), torch.empty(T, hidden, dtype=torch.bfloat16, device=dev),
          torch.empty(T, dtype=torch.int64, device=dev), torch.empty(T, L * n, dtype=torch.bfloat16, device=dev),
          torch.empty(T, L * n, dtype=torch.bfloat16, device=dev)]

    def reference_sequence(i):
        ops.reshape_and_cache_flash_bulk(K[i], V[i], kc, vc, S[i], "fp8", sc, sc, H, D)
        for src, o in zip([Hs[i], Rs[i], P, K[i], V[i]], ob):
            torch.index_select(src, 0, idx, out=o)

    def with_gather_rows(i):
        ops.reshape_and_cache_flash_bulk(K[i], V[i], kc, vc, S[i], "fp8", sc, sc, H, D)
        ops.gather_rows([Hs[i], Rs[i], P, K[i], V[i]], idx, ob)

    def with_bulk_select(i):
        ops.reshape_and_cache_flash_bulk_select(K[i], V[i], kc, vc, S[i], "fp8", sc, sc, H, D, idx, ob[3], ob[4])
        ops.gather_rows([Hs[i], Rs[i], P], idx, ob[:3])

    out = {}
    for name, fn in (("bulk_write_then_five_index_select", reference_sequence),
                     ("bulk_write_then_gather_rows", with_gather_rows),
                     ("bulk_select_then_gather_rows_of_three", with_bulk_select)):
        for i in range(sets):
            fn(i)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(sets):
                fn(i)
        warm_replays(graph.replay)
        out[name] = {"us_per_step_graph": round(statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / sets, 2)}
    return out


def host_overhead_route(route, calls=3000):
    """Host wall time per eager call with the GPU out of the picture: tiny inputs (4 tokens, 8 rows), so that a
    kernel is over long before the host has issued the next one; `calls` calls are issued back to back and the
    wall clock is divided by their number (one synchronisation in front, one behind, outside the clock).
    route "py_custom_ops": this package's module functions (the C++ host layer called directly).  route
    "torch_ops": the same host layer through torch.ops.arctic_inference.* as this package registers it (what
    torch.compile and callers of the registered operators take).  route "torch_ext": the same library behind the
    reference's own torch_bindings.cpp compiled with this package's forwards (the file named by ARCTIC_TORCH_EXT).
    Runs in a process of its own: the last route defines the arctic_inference namespace a second time."""
    dev = torch.device("cuda:0")
    if route in ("py_custom_ops", "torch_ops"):
        from arcticinference_amd import py_custom_ops as ops
        assert ops.try_load_torch_library()
        if route == "py_custom_ops":
            bulk, lstm, ln = ops.reshape_and_cache_flash_bulk, ops.sum_lstm, ops.speculator_ln
        else:
            ns = torch.ops.arctic_inference
            bulk, lstm, ln = ns.reshape_and_cache_flash_bulk, ns.sum_lstm_cuda, ns.speculator_ln_cuda
    else:
        torch.ops.load_library(os.environ["ARCTIC_TORCH_EXT"])
        ns = torch.ops.arctic_inference
        bulk, lstm, ln = ns.reshape_and_cache_flash_bulk, ns.sum_lstm_cuda, ns.speculator_ln_cuda

    def per_call_us(f):
        for _ in range(200):
            f()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(calls):
                f()
            t1 = time.perf_counter()
            torch.cuda.synchronize()
            us = (t1 - t0) * 1e6 / calls
            best = us if best is None else min(best, us)
        return round(best, 2)

    out = {}
    x = torch.randn(8, 4096, device=dev).to(torch.bfloat16)
    s4 = torch.randn(8, 16384, device=dev).to(torch.bfloat16)
    w = torch.ones(4096, device=dev, dtype=torch.bfloat16)
    out["speculator_ln"] = per_call_us(lambda: ln(x, w, w, 1e-6))
    out["sum_lstm"] = per_call_us(lambda: lstm(s4, s4, x, w, w, w, w, 1.0, 1e-6, 1e-6, False))
    T, H, D, NB, bs = 4, 8, 128, 64, 16
    for L in (16, 40):
        keys = torch.randn(T, L * H * D, device=dev).to(torch.bfloat16)
        values = torch.randn(T, L * H * D, device=dev).to(torch.bfloat16)
        pool = [torch.zeros(2, NB, bs, H, D, dtype=torch.uint8, device=dev) for _ in range(L)]
        kc, vc = [b[0] for b in pool], [b[1] for b in pool]
        ks = [torch.ones((), device=dev) for _ in range(L)]
        vs = [torch.ones((), device=dev) for _ in range(L)]
        slots = torch.arange(T, device=dev)
        out[f"reshape_and_cache_flash_bulk_{L}_layers"] = per_call_us(
            lambda: bulk(keys, values, kc, vc, slots, "fp8", ks, vs, H, D))
        if route == "py_custom_ops":   # the per-layer arguments checked once and held (prepare_bulk_kv_layers)
            write = ops.prepare_bulk_kv_layers(kc, vc, ks, vs).write
            out[f"prepared_layers_write_{L}_layers"] = per_call_us(lambda: write(keys, values, slots, "fp8", H, D))

        # what the caller itself spends per step on the four lists it passes (llama_swiftkv.py:594-615: two views of
        # every layer's cache tensor and two attribute reads), for scale
        def caller_lists():
            a, b, c, d = [], [], [], []
            for l in range(L):
                kv = pool[l]
                a.append(kv[0])
                b.append(kv[1])
                c.append(ks[l])
                d.append(vs[l])
            return a, b, c, d
        t0 = time.perf_counter()
        for _ in range(300):
            caller_lists()
        out[f"caller_builds_its_four_lists_{L}_layers"] = round((time.perf_counter() - t0) * 1e6 / 300, 2)
    return out


def bench_host_overhead():
    """Host microseconds per eager call through both integration routes, each measured in a child process."""
    ext = os.path.join(ROOT, "oracle", "_ref", "arctic_torch_ext.so")
    routes = {"route_1_py_custom_ops": ("py_custom_ops", {}), "route_1_through_torch_ops": ("torch_ops", {})}
    if os.path.exists(ext):
        routes["route_2_reference_torch_bindings"] = ("torch_ext", {"ARCTIC_TORCH_EXT": ext})
    out = {"what": "host wall time per eager call in microseconds, tiny inputs (4 tokens / 8 rows), 3000 calls issued "
                   "back to back, best of 3 rounds; the GPU work of a call is shorter than the host's"}
    for name, (route, env) in routes.items():
        proc = subprocess.run([sys.executable, os.path.abspath(__file__), "--host-overhead-route", route],
                              capture_output=True, text=True, env=dict(os.environ, **env), timeout=300)
        if proc.returncode != 0:
            out[name] = "failed: " + (proc.stderr.strip().splitlines() or ["no output"])[-1]
            continue
        out[name] = json.loads(proc.stdout.strip().splitlines()[-1])
    if "route_2_reference_torch_bindings" not in routes:
        out["route_2_reference_torch_bindings"] = "oracle/_ref/arctic_torch_ext.so is not built (make -C oracle torch_ext)"
    return out


def bench_suffix_decoding():
    """Suffix-tree speculation on the host cores (no GPU): libarctic_suffix.so next to the reference's own
    code (oracle/_ref, compiled from the reference's sources, when it is there), both driven through the
    same raw ctypes calls with preallocated buffers.  One global tree of depth 64 over 256 responses of 1024
    tokens made of recurring phrases (so contexts do match); then decoding steps of 32 requests: speculate
    from the last 64 tokens (path and tree drafts), append token by token; then eviction of half the cache."""
    import ctypes
    import numpy as np
    from arcticinference_amd.suffix_decoding import _tree
    from oracle.suffix_ref import RefTree

    rng = np.random.default_rng(11)
    phrases = [rng.integers(0, 32000, int(rng.integers(8, 40))).astype(np.int32) for _ in range(400)]

    def text(n):
        out = []
        while sum(len(p) for p in out) < n:
            out.append(phrases[int(rng.zipf(1.3)) % len(phrases)] if rng.random() < 0.9
                       else rng.integers(0, 32000, 5).astype(np.int32))
        return np.ascontiguousarray(np.concatenate(out)[:n])

    responses = [text(1024) for _ in range(256)]
    decode = [text(64 + 128) for _ in range(32)]
    tok, par = np.empty(64, np.int32), np.empty(64, np.int32)
    prob = np.empty(64, np.float32)
    score, mlen = ctypes.c_float(), ctypes.c_int()
    outs = (tok.ctypes.data, par.ctypes.data, prob.ctypes.data, ctypes.byref(score), ctypes.byref(mlen))

    def run(create, extend, speculate, remove):
        h = create(64)
        out = {}
        t0 = time.perf_counter()
        for i, r in enumerate(responses):
            extend(h, i, r.ctypes.data, r.size)
        out["extend_Mtokens_per_s"] = round(len(responses) * 1024 / (time.perf_counter() - t0) / 1e6, 3)
        for mode, use_tree in (("speculate_path", 0), ("speculate_tree", 1)):
            jobs = [(d.ctypes.data + 4 * (pos - 64)) for d in decode for pos in range(64, len(d), 4)]
            t0, drafted = time.perf_counter(), 0
            for ptr in jobs:
                drafted += speculate(h, ptr, 64, 16, 2.0, 0.0, 0.1, use_tree, *outs)
            dt = time.perf_counter() - t0
            out[mode + "_kcalls_per_s"] = round(len(jobs) / dt / 1e3, 2)
            out[mode + "_tokens_per_call"] = round(drafted / len(jobs), 2)
        jobs = [(1000 + j, d.ctypes.data + 4 * pos) for j, d in enumerate(decode) for pos in range(64, len(d))]
        t0 = time.perf_counter()
        for sid, ptr in jobs:                                # token-by-token growth of live responses
            extend(h, sid, ptr, 1)
        out["append_Mtokens_per_s"] = round(len(jobs) / (time.perf_counter() - t0) / 1e6, 3)
        t0 = time.perf_counter()
        for i in range(0, len(responses), 2):
            remove(h, i)
        out["remove_sequences_per_s"] = round(len(responses) / 2 / (time.perf_counter() - t0), 1)
        return out

    lib = _tree._lib
    mine = run(lib.arctic_suffix_tree_create, lib.arctic_suffix_tree_extend, lib.arctic_suffix_tree_speculate,
               lib.arctic_suffix_tree_remove)
    result = {"library": mine, "cores": 1}
    if RefTree.available():
        ref_lib = RefTree.lib()
        ref = run(ref_lib.ref_suffix_tree_create, ref_lib.ref_suffix_tree_extend, ref_lib.ref_suffix_tree_speculate,
                  ref_lib.ref_suffix_tree_remove)
        result["reference"] = ref
        result["speedup"] = {k: round(mine[k] / ref[k], 2) for k in mine if not k.endswith("tokens_per_call")}
    else:
        result["reference"] = "oracle/_ref/libsuffix_ref.so not present"
    return result


def bench_argmax(ops, dev, steps):
    """Token selection at the end of a speculator step (arctic_speculator.py:846-848, 862): argmax over a
    128256-wide vocabulary for 512 rows of bf16 logits (131 MB), clamped; one launch against torch's
    argmax + clamp_.  Three rotating sets keep the logits out of the last-level cache."""
    T, V, sets = 512, 128256, 3
    g = torch.Generator(device=dev).manual_seed(8)
    logits = [torch.randn(T, V, generator=g, device=dev).to(torch.bfloat16) for _ in range(sets)]
    nbytes = T * V * 2 + T * 8
    out = {"bytes_per_call": nbytes}
    floor = load_floor_kernels()
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    cases = [("speculator_argmax", lambda i: ops.speculator_argmax(logits[i % sets], V)),
             ("torch_argmax_clamp", lambda i: torch.argmax(logits[i % sets], dim=-1).clamp_(0, V - 1))]
    if floor is not None:
        # the kernel's loads with nothing computed: what reading the rows costs in this launch shape
        cases.append(("row_read_only_floor", lambda i: floor.floor_row_read(
            logits[i % sets].data_ptr(), T, V * 2, 1024, sink.data_ptr(), torch.cuda.current_stream().cuda_stream)))
    for name, fn in cases:
        for i in range(3):
            fn(i)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(sets):
                fn(i)
        warm_replays(graph.replay)
        med = statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / sets
        out[name] = {"us_per_call_graph": round(med, 2), "GBps": round(nbytes / med / 1e3, 1),
                     "hbm_frac": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4)}
    return out


def box_reference(dev):
    """What plain library kernels reach on this very GPU (boxes of one pool differ by up to 20 %):
    a contiguous bf16 -> fp8 cast of 1.3 GB (the same 2:1 read:write mix as the bulk fp8 write, no
    scatter, no scaling) and a 1 GiB device-to-device copy.  About 25 ms of GPU work."""
    x = torch.randn(1 << 26, device=dev).to(torch.bfloat16).repeat(10)
    f = lambda: x.to(torch.float8_e4m3fn)
    for _ in range(3):
        f()
    cast = statistics.median(event_times_us(f, 30))
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    g = lambda: dst.copy_(src)
    for _ in range(3):
        g()
    copy = statistics.median(event_times_us(g, 30))
    return {"torch_bf16_to_fp8_cast_GBps": round(x.numel() * 3 / cast / 1e3, 1),
            "torch_copy_1GiB_GBps": round(2 * (1 << 30) / copy / 1e3, 1)}


def bench_decode_mix(ops, dev, steps):
    """Decode-step workload: 512 decode tokens; bulk fp8 KV write over 16 layers into 32768-block caches, ln0, three
    sum_lstm steps; one HIP graph per step.  Eight sets of everything that is read (K/V rows, slots, ln0 input,
    pre-activations; 1.2 GB in all) rotate between replays so that no input is served from the 256 MB last-level
    cache; the caches (17 GB) are shared, they are only written.  The first sum_lstm takes prev_cell=None (the cell
    of zeros a proposal round starts from) unless `as_the_caller_issues_it`, where a zero tensor is cleared and
    passed as the reference's caller does.  `kv_write_on_a_second_stream` forks the KV write, which nothing in the
    step depends on, onto a second stream inside the captured graph."""
    sets, T, Hd = 8, 512, 4096
    ws = [BulkWorkload("decode", 512, 16, 8, 128, 16, 32768, "fp8", 0.0, 4 + i, 1.5, dev) for i in range(1)]
    for i in range(1, sets):
        ws.append(BulkWorkload("decode", 512, 16, 8, 128, 16, 32768, "fp8", 0.0, 4 + i, 1.5, dev, bufs=ws[0].bufs))
    g = torch.Generator(device=dev).manual_seed(4)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev).to(torch.bfloat16)
    S = [[rn(T, 4 * Hd) for _ in range(3)] for _ in range(sets)]
    Z = [[rn(T, 4 * Hd) for _ in range(3)] for _ in range(sets)]
    X = [rn(T, Hd) for _ in range(sets)]
    vec = lambda m: (m + 0.02 * torch.randn(Hd, generator=g, device=dev)).to(torch.bfloat16)
    w_cell, b_cell, w_state, b_state = vec(1.0), vec(0.0), vec(1.0), vec(0.0)
    sw = 0.5 ** (0.5 / 3)
    alpha = ((1 - sw * sw) * (Hd / 2)) ** 0.5 / sw
    nbytes = ws[0].bytes + 4 * Hd * T + 3 * 22 * Hd * T

    side = torch.cuda.Stream()   # default priority

    def step(i, mode):
        main = torch.cuda.current_stream()
        if mode == "fork":
            # the KV write on a second captured stream, beside the speculator's kernels
            side.wait_stream(main)
            with torch.cuda.stream(side):
                ops.reshape_and_cache_flash_bulk(*ws[i].args())
        else:
            ops.reshape_and_cache_flash_bulk(*ws[i].args())
        ops.speculator_ln(X[i], None, None, 1e-6)
        cell = torch.zeros(T, Hd, dtype=torch.bfloat16, device=dev) if mode == "zeros" else None
        for k in range(3):
            _, cell = ops.sum_lstm(S[i][k], Z[i][k], cell, w_cell, b_cell, w_state, b_state, alpha, 1e-6, 1e-6,
                                   False)
        if mode == "fork":
            main.wait_stream(side)

    out = {"bytes_per_step": nbytes, "sets_in_rotation": sets}
    for name, zero_tensor in (("", "chain"), ("_as_the_caller_issues_it", "zeros"),
                              ("_kv_write_on_a_second_stream", "fork")):
        step(0, zero_tensor)
        torch.cuda.synchronize()
        graphs = []
        for i in range(sets):
            gr = torch.cuda.CUDAGraph()
            with torch.cuda.graph(gr):
                step(i, zero_tensor)
            graphs.append(gr)
        def all_graphs():
            for gr in graphs:
                gr.replay()
        warm_replays(all_graphs)
        counter = iter(range(10 ** 9))
        us = event_times_us(lambda: graphs[next(counter) % sets].replay(), max(200, steps))
        med = statistics.median(us)
        # the same graphs replayed back to back, one pair of events around all of them: per step, without the
        # idle gap in front of a lone replay
        def all_sets():
            for gr in graphs:
                gr.replay()
        b2b = statistics.median(event_times_us(all_sets, max(25, steps // 4))) / sets
        us.sort()
        out.update({f"us_per_step_graph{name}": round(med, 2),
                    f"us_per_step_graph_p10_p90{name}": [round(us[len(us) // 10], 2), round(us[len(us) * 9 // 10], 2)],
                    f"replays{name}": len(us), f"GBps{name}": round(nbytes / med / 1e3, 1),
                    f"hbm_frac{name}": round(nbytes / med / 1e3 / HBM_PEAK_GBS, 4),
                    f"us_per_step_graphs_back_to_back{name}": round(b2b, 2),
                    f"hbm_frac_back_to_back{name}": round(nbytes / b2b / 1e3 / HBM_PEAK_GBS, 4)})
        del graphs
    return out


def bench_bulk_auto(ops, dev, steps):
    """The bf16 (`auto`) cache path: 8192 algorithmic bytes per valid token and layer (4n read, 4n written).
    config_1: 256 tokens x 16 layers into 512-block caches (33.5 MB per launch), eight sets of sources and caches
    (4.4 GB) rotating inside one HIP graph so that nothing is cache resident; 70B shape: 16384 tokens x 40 layers, 10 %
    padding, 8192-block bf16 caches (21 GB), compact placement, event-timed launches."""
    out = {}
    sets = 8
    ws = [BulkWorkload("config-1", 256, 16, 8, 128, 16, 512, "auto", 0.0, 100 + i, 1.0, dev) for i in range(sets)]

    def run():
        for w in ws:
            ops.reshape_and_cache_flash_bulk(*w.args())
    run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    warm_replays(graph.replay)
    us = statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / sets
    out["config_1_256_tokens_16_layers"] = {"us_per_call_graph": round(us, 2), "bytes_per_call": ws[0].bytes,
                                            "GBps": round(ws[0].bytes / us / 1e3, 1),
                                            "hbm_frac": round(ws[0].bytes / us / 1e3 / HBM_PEAK_GBS, 4)}
    del ws, graph
    torch.cuda.empty_cache()
    w = BulkWorkload("70B-auto", 16384, 40, 8, 128, 16, 8192, "auto", 0.10, 2, 1.5, dev)
    f = lambda: ops.reshape_and_cache_flash_bulk(*w.args())
    for _ in range(5):
        f()
    out["70b_shape_compact_pool"] = dict(kernel_stats(f, steps, w.bytes), bytes_per_call=w.bytes)
    del w, f
    torch.cuda.empty_cache()
    # the same launch on the serving map of the headline: 66 GiB of weights, then a bf16 pool of the same size in
    # bytes (80 layers x [2, 32768, 16, 8, 128] bf16 = 2 GiB each), layers 40-79 written
    try:
        mem = ServingMemoryMap(dev, 66, 80, 40, 32768, 16, 8, 128, torch.bfloat16)
        w = BulkWorkload("70B-auto-serving", 16384, 40, 8, 128, 16, 32768, "auto", 0.10, 2, 1.5, dev, bufs=mem.written_layers())
        f = lambda: ops.reshape_and_cache_flash_bulk(*w.args())
        for _ in range(5):
            f()
        out["70b_shape_serving_map"] = dict(kernel_stats(f, steps, w.bytes), bytes_per_call=w.bytes,
                                            memory_map=mem.describe())
        del mem, w, f
    except torch.OutOfMemoryError:
        out["70b_shape_serving_map"] = "not enough free device memory"
    torch.cuda.empty_cache()
    return out


def bench_bulk_tp_heads(ops, dev, steps):
    """The 70B shape as one GPU of a tensor-parallel group sees it: num_kv_heads / TP heads per GPU
    (llama_swiftkv.py:598), i.e. cache rows of 128, 256 or 512 bytes instead of 1 KiB; fp8, 16384 tokens x 40 layers,
    10 % padding, 8192-block caches, compact placement."""
    out = {}
    for H in (1, 2, 4, 8):
        w = BulkWorkload(f"70B-{H}-heads", 16384, 40, H, 128, 16, 8192, "fp8", 0.10, 2, 1.5, dev)
        f = lambda: ops.reshape_and_cache_flash_bulk(*w.args())
        for _ in range(5):
            f()
        out[f"{H}_kv_heads"] = dict(kernel_stats(f, steps, w.bytes), bytes_per_call=w.bytes, cache_row_bytes=H * 128)
        del w, f
        torch.cuda.empty_cache()
    return out


def bench_source_before_pool(ops, dev, steps):
    """The headline launch with the K/V source allocated BETWEEN the weights and the KV pool instead of behind the
    pool.  A vLLM worker profiles a forward pass of its largest batch before it sizes and allocates the pool, and
    torch's caching allocator keeps those activation blocks, so the k_states / v_states of an eager prefill chunk come
    out of memory that lies in front of the pool; the loads of the launch (two thirds of its traffic) then come from
    another HBM region than most of its stores.  Meant for a process of its own on an idle GPU (--only), where
    allocation order is physical order."""
    weights = torch.empty(66 << 30, dtype=torch.uint8, device=dev)
    pool = []

    def written_layers_of_a_new_pool():
        torch.cuda.empty_cache()      # the source generator's temporaries go back; keys and values stay where they are
        pool.extend(torch.empty(2, 65536, 16, 8, 128, dtype=torch.uint8, device=dev) for _ in range(80))
        return pool[40:]

    w = BulkWorkload("70B-SwiftKV-source-first", 16384, 40, 8, 128, 16, 65536, "fp8", 0.10, 2, 1.5, dev,
                     make_bufs=written_layers_of_a_new_pool)
    f = lambda: ops.reshape_and_cache_flash_bulk(*w.args())
    box_reference(dev)                # the GPU out of its idle state, as in front of the headline
    for _ in range(20):
        f()
    out = dict(kernel_stats(f, max(steps, 50), w.bytes),
               memory_map="66 GiB resident weights (placeholder), then the K/V source (2.5 GiB), then the paged KV pool of "
                          "all 80 layers, 65536 blocks = 2 GiB per layer; layers 40-79 are written")
    del weights
    return out


def bench_lstm_rows(ops, dev, steps):
    """sum_lstm at 4096 against the number of rows (tokens) per call: the fixed cost of a launch against the
    90 112 bytes per row.  Enough buffer sets rotate inside one HIP graph that every call reads from HBM (at least
    300 MB in rotation, at least eight sets)."""
    Hd = 4096
    g = torch.Generator(device=dev).manual_seed(9)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev).to(torch.bfloat16)
    vec = lambda m: (m + 0.02 * torch.randn(Hd, generator=g, device=dev)).to(torch.bfloat16)
    w_cell, b_cell, w_state, b_state = vec(1.0), vec(0.0), vec(1.0), vec(0.0)
    out = {}
    for T in (8, 32, 128, 256, 512, 1024, 2048, 4096):
        per_call = 22 * Hd * T
        sets = max(8, -(-300 * 2 ** 20 // per_call))
        sets = min(sets, 256)
        S, Z, C = [rn(T, 4 * Hd) for _ in range(sets)], [rn(T, 4 * Hd) for _ in range(sets)], [rn(T, Hd) for _ in range(sets)]

        def run():
            for i in range(sets):
                ops.sum_lstm(S[i], Z[i], C[i], w_cell, b_cell, w_state, b_state, 23.07, 1e-6, 1e-6, False)
        run()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run()
        warm_replays(graph.replay)
        us = statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / sets
        out[f"{T}_rows"] = {"us_per_call_graph": round(us, 2), "GBps": round(per_call / us / 1e3, 1),
                            "hbm_frac": round(per_call / us / 1e3 / HBM_PEAK_GBS, 4), "sets_in_rotation": sets}
        del S, Z, C, graph
    return out


def bench_lstm_widths(ops, dev, steps):
    """sum_lstm at 512 rows against the row width: the kernel that requests a row in stages (all four scale / shift
    vectors given, rows of up to 8192 elements, spare lanes in the last wave when the width is no multiple of 512)
    next to the general kernel, which the same call takes when a vector is missing (here: the cell norm's pair)."""
    T = 512
    g = torch.Generator(device=dev).manual_seed(9)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev).to(torch.bfloat16)
    out = {}
    for Hd in (2048, 2880, 4000, 4096, 5120, 6144, 8192, 12288):
        per_call = 22 * Hd * T
        sets = max(8, -(-300 * 2 ** 20 // per_call))
        S, Z, C = [rn(T, 4 * Hd) for _ in range(sets)], [rn(T, 4 * Hd) for _ in range(sets)], [rn(T, Hd) for _ in range(sets)]
        w = [rn(Hd) for _ in range(4)]
        row = {}
        for name, cell_pair in (("all_four_vectors", (w[0], w[1])), ("without_the_cell_norm_vectors", (None, None))):
            def run():
                for i in range(sets):
                    ops.sum_lstm(S[i], Z[i], C[i], cell_pair[0], cell_pair[1], w[2], w[3], 23.07, 1e-6, 1e-6, False)
            run()
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                run()
            warm_replays(graph.replay)
            us = statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / sets
            row[name] = {"us_per_call_graph": round(us, 2), "hbm_frac": round(per_call / us / 1e3 / HBM_PEAK_GBS, 4)}
            del graph
        out[f"{Hd}_wide"] = row
        del S, Z, C
    return out


def bench_argmax_shapes(ops, dev, steps):
    """speculator_argmax over vocabulary sizes (512 rows; 50257 and 128257 put every row at another offset from a
    16-byte boundary) and over small batches (128256 logits per row), bf16, enough rotating sets to read from HBM."""
    g = torch.Generator(device=dev).manual_seed(10)
    out = {}
    for T, V in ((512, 32000), (512, 50257), (512, 65536), (512, 128257), (512, 151936), (512, 262144),
                 (1, 128256), (8, 128256), (64, 128256), (128, 128256), (256, 128256)):
        sets = max(3, min(64, (400 << 20) // (T * V * 2) + 1))
        logits = [torch.randn(T, V, generator=g, device=dev).to(torch.bfloat16) for _ in range(sets)]

        def run():
            for x in logits:
                ops.speculator_argmax(x, V)
        run()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run()
        warm_replays(graph.replay)
        us = statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / sets
        out[f"{T}_rows_x_{V}"] = {"us_per_call_graph": round(us, 2), "hbm_frac": round(2 * T * V / us / 1e3 / HBM_PEAK_GBS, 4)}
        del logits, graph
    return out


def bench_speculator_round_glue(ops, dev, steps):
    """Everything but the matrix products of one proposal round of the LSTM speculator (three heads, 512 rows,
    width 4096, 128256-entry vocabulary; arctic_speculator.py:733-862): ln0 / sqrt 2, then per head the embedding
    lookup, the gate update and the token selection.  Once as the reference's caller issues it with its own two
    operators (speculator_ln + division; embedding + repeat + sum_lstm; argmax + clamp_), once with the fused
    operators (speculator_ln_scaled; sum_lstm_embedded; speculator_argmax).  The projections and the LM head sit
    between these steps in the real loop; their outputs are stand-ins here.  One HIP graph each, two rotating sets."""
    T, Hd, V, heads, sets = 512, 4096, 128256, 3, 2
    g = torch.Generator(device=dev).manual_seed(9)
    rn = lambda *s: torch.randn(*s, generator=g, device=dev).to(torch.bfloat16)
    X = [rn(T, 1, Hd) for _ in range(sets)]
    S = [[rn(T, 1, 4 * Hd) for _ in range(heads)] for _ in range(sets)]          # projection outputs
    LOG = [[rn(T, V) for _ in range(heads)] for _ in range(sets)]                # LM-head outputs
    table = rn(V, Hd)
    tokens0 = torch.randint(0, V, (T, 1), generator=g, device=dev)
    cell0 = rn(T, 1, Hd)
    vec = lambda m: (m + 0.02 * torch.randn(Hd, generator=g, device=dev)).to(torch.bfloat16)
    w_cell, b_cell, w_state, b_state = vec(1.0), vec(0.0), vec(1.0), vec(0.0)
    sw = 0.5 ** (0.5 / 3)
    alpha = ((1 - sw * sw) * (Hd / 2)) ** 0.5 / sw
    sqrt2 = 2 ** 0.5

    def as_the_caller(i):
        prev = ops.speculator_ln(X[i], None, None, 1e-6) / sqrt2
        tokens, cell = tokens0.clamp(0, V - 1), cell0
        for k in range(heads):
            z4 = torch.nn.functional.embedding(tokens, table).repeat(1, 1, 4)
            state, cell = ops.sum_lstm(S[i][k].flatten(0, 1).contiguous(), z4.flatten(0, 1).contiguous(),
                                       cell.flatten(0, 1).contiguous(), w_cell, b_cell, w_state, b_state, alpha, 1e-6,
                                       1e-6, False)
            state, cell = state.reshape(T, 1, Hd), cell.reshape(T, 1, Hd)
            tokens = torch.argmax(LOG[i][k], dim=-1).reshape(T, -1)
            tokens.clamp_(0, V - 1)
        return prev, state, tokens

    def fused(i):
        prev = ops.speculator_ln_scaled(X[i], None, None, 1e-6, 1.0 / sqrt2)
        tokens, cell = tokens0, cell0
        for k in range(heads):
            state, cell = ops.sum_lstm_embedded(S[i][k], table, tokens, cell, w_cell, b_cell, w_state, b_state, alpha,
                                                1e-6, 1e-6, False)
            tokens = ops.speculator_argmax(LOG[i][k], V).reshape(T, -1)
        return prev, state, tokens

    a, b = as_the_caller(0), fused(0)
    torch.cuda.synchronize()
    same = bool(torch.equal(a[2], b[2]) and torch.equal(a[1], b[1]))
    out = {"outputs_identical": same}
    for name, fn in (("as_the_reference_caller", as_the_caller), ("fused_operators", fused)):
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(sets):
                fn(i)
        warm_replays(graph.replay)
        out[name] = {"us_per_round_graph": round(statistics.median(event_times_us(graph.replay, max(10, steps // 2))) / sets, 2)}
    return out


def placement_sweep(ops, dev, steps):
    """Where the caches sit in HBM against how fast the same launch runs.  The GPU's memory is taken in 32
    chunks of 8 GiB (allocation order follows physical order on an otherwise empty GPU); the 70B-shape
    source sits in one chunk and the 80 caches (4096 blocks each, 5 GiB) in another.  Scan 1 keeps the
    source in chunk 0 and moves the caches through every chunk: the chunks that run slow share chunk 0's
    region.  Scan 2 repeats that from the first fast chunk, which separates the other two regions.  The
    last cases spread the caches of one launch over the regions found."""
    T, L, H, D, bs, NB = 16384, 40, 8, 128, 16, 4096
    n = H * D
    nchunks, chunk_bytes = 32, 8 << 30
    chunks = [torch.empty(chunk_bytes, dtype=torch.uint8, device=dev) for _ in range(nchunks)]
    src_bytes, cache_bytes = T * L * n * 2, NB * bs * n
    gd = torch.Generator(device=dev).manual_seed(2)
    slots_cpu = make_slots(T, NB * bs, torch.Generator().manual_seed(2), 0.10)
    slots = slots_cpu.to(dev)
    nbytes = int((slots_cpu >= 0).sum()) * L * n * 6
    scales = [torch.full((), 0.0134, device=dev) for _ in range(L)]

    def source(c):
        kv = chunks[c][:2 * src_bytes].view(torch.bfloat16).view(2, T, L * n)
        for t0 in range(0, T, 512):
            kv[:, t0:t0 + 512] = (torch.randn(2, 512, L * n, generator=gd, device=dev) * 1.5).to(torch.bfloat16)
        return kv[0], kv[1]

    def cache(c, index, base):
        off = base + index * cache_bytes
        return chunks[c][off:off + cache_bytes].view(NB, bs, H, D)

    def timed(k, v, kc, vc):
        f = lambda: ops.reshape_and_cache_flash_bulk(k, v, kc, vc, slots, "fp8", scales, scales, H, D)
        for _ in range(3):
            f()
        return round(statistics.median(event_times_us(f, steps)), 1)

    def scan(src_chunk):
        k, v = source(src_chunk)
        row = []
        for c in range(nchunks):
            base = 2 * src_bytes if c == src_chunk else 0
            row.append(timed(k, v, [cache(c, 2 * l, base) for l in range(L)], [cache(c, 2 * l + 1, base) for l in range(L)]))
        return row

    scan0 = scan(0)
    cut = (min(scan0) + max(scan0)) / 2
    region_a = [c for c in range(nchunks) if scan0[c] > cut]
    first_fast = next(c for c in range(nchunks) if scan0[c] <= cut)
    scan1 = scan(first_fast)
    cut1 = (min(scan1) + max(scan1)) / 2
    region_b = [c for c in range(nchunks) if scan1[c] > cut1]
    region_c = [c for c in range(nchunks) if c not in region_a and c not in region_b]
    out = {"chunk_gib": 8, "us_source_in_chunk_0": scan0, f"us_source_in_chunk_{first_fast}": scan1,
           "regions": [region_a, region_b, region_c], "bytes_per_launch": nbytes}
    if region_a and region_b and region_c:
        k, v = source(0)
        reps = [region_a[len(region_a) // 2], region_b[len(region_b) // 2], region_c[len(region_c) // 2]]
        base = 2 * src_bytes
        cases = {
            "one_region (source's own)": [reps[0]] * L,
            "one_region (another)": [reps[1]] * L,
            "layers_alternate_over_2_regions": [reps[l % 2] for l in range(L)],
            "layers_alternate_over_3_regions": [reps[l % 3] for l in range(L)],
            "lower_half_in_one_upper_half_in_another": [reps[1] if l < L // 2 else reps[2] for l in range(L)],
        }
        out["spread_cases_us"] = {
            name: timed(k, v, [cache(where[l], 2 * l, base) for l in range(L)],
                        [cache(where[l], 2 * l + 1, base) for l in range(L)])
            for name, where in cases.items()}
        out["spread_cases_GBps"] = {name: round(nbytes / us / 1e3) for name, us in out["spread_cases_us"].items()}
        floor = load_floor_kernels()
        if floor is not None:
            # bare streams of 64 KiB pieces dealt over one, two or three regions: 3 GiB loaded, stored, or
            # loaded with half as much stored (the byte mix of the fp8 write)
            import ctypes
            pieces = 3 * 16384
            sink = torch.zeros(1, dtype=torch.int32, device=dev)
            ptrs = lambda offs: (ctypes.c_void_p * 3)(*[chunks[c].data_ptr() + offs for c in reps])
            low, high = ptrs(0), ptrs(4 << 30)
            stream = torch.cuda.current_stream().cuda_stream

            def stream_GBps(mode, nsrc, ndst, moved):
                f = lambda: floor.floor_stream(low, nsrc, high, ndst, pieces, mode, sink.data_ptr(), stream)
                for _ in range(2):
                    f()
                return round(moved / statistics.median(event_times_us(f, steps)) / 1e3)

            out["bare_stream_GBps"] = {
                "load_only": {f"{n}_regions": stream_GBps(0, n, 1, pieces * 65536) for n in (1, 2, 3)},
                "store_only": {f"{n}_regions": stream_GBps(1, 1, n, pieces * 65536) for n in (1, 2, 3)},
                "load_2_store_1, loads from one region": {
                    f"stores_to_{n}_regions": stream_GBps(2, 1, n, pieces * 98304) for n in (1, 2, 3)},
                "load_2_store_1 with the stores scattered as rows of 1 KiB (the bulk write's pattern)": {
                    f"stores_to_{n}_regions": stream_GBps(3, 1, n, pieces * 98304) for n in (1, 2, 3)},
                "the same with 16-byte stores (a lane loads 32 adjacent bytes)": {
                    f"stores_to_{n}_regions": stream_GBps(4, 1, n, pieces * 98304) for n in (1, 2, 3)},
            }

            # the scattered stream by resident workgroups of 1024 lanes (the best of four shapes): what the pattern
            # costs when nothing but bandwidth shapes the kernel
            def resident_GBps(ndst, slices=((0, 0),), shapes=((4, 256), (4, 768), (8, 256), (8, 512))):
                best = 0
                for loads, groups in shapes:
                    for period_us, read_share in slices:
                        # a period in which every workgroup moves one piece at `period_us`'s assumed rate (bytes / us)
                        period = int(groups * loads * 16384 * 1.5 / period_us * 100) if period_us else 0
                        f = lambda: floor.floor_stream_resident(chunks[reps[0]].data_ptr(), high, ndst, 3 << 30, loads, groups,
                                                                period, int(period * read_share), stream)
                        for _ in range(2):
                            assert f() == 0
                        best = max(best, round((3 << 30) * 1.5 / statistics.median(event_times_us(f, max(5, steps // 10))) / 1e3))
                return best

            out["bare_stream_GBps"]["scattered 2:1 stream by resident workgroups (1024 lanes, 4 or 8 loads per lane in flight)"] = {
                f"stores_to_{n}_regions": resident_GBps(n) for n in (1, 2, 3)}
            # ... with reads and writes in turns: periods sized for 5.0 to 6.5 TB/s, 50 to 70 % of a period for the loads
            slices = [(rate, share) for rate in (5.0e6, 5.5e6, 6.0e6, 6.5e6) for share in (0.5, 0.6, 0.7)]
            out["bare_stream_GBps"]["the same with all loads in one window of the shared clock and all stores in the other (best of 12 schedules)"] = {
                "stores_to_1_regions": resident_GBps(1, slices, ((8, 256), (4, 512)))}
    return out


def bench_node_floor(dev, steps):
    """What one kernel node of a HIP graph costs on this GPU when it moves next to nothing: 64 nodes of 512 workgroups x
    512 lanes (the speculator operators' launch shape) in one graph, empty, and with one memory round trip each.  The
    fixed part of every small operator's time."""
    floor = load_floor_kernels()
    if floor is None:
        return "bench_floor.so is not built"
    blocks, nodes = 512, 64
    a = torch.zeros(nodes, blocks * 1024, dtype=torch.uint8, device=dev)
    b = torch.zeros(nodes, blocks * 1024, dtype=torch.uint8, device=dev)
    out = {}
    for name, touch in (("empty_kernel", 0), ("one_16_byte_load_and_store_per_workgroup_wave", 1)):
        def run():
            stream = torch.cuda.current_stream().cuda_stream
            for i in range(nodes):
                floor.floor_node(a[i].data_ptr(), b[i].data_ptr(), blocks, 512, touch, stream)
        run()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            run()
        warm_replays(graph.replay)
        us = statistics.median(event_times_us(graph.replay, max(10, steps // 2)))
        out[name] = {"us_per_node_in_a_graph": round(us / nodes, 2)}
        us = event_times_us(lambda: floor.floor_node(a[0].data_ptr(), b[0].data_ptr(), blocks, 512, touch,
                                                     torch.cuda.current_stream().cuda_stream), max(20, steps))
        out[name]["us_per_eager_launch_between_events"] = round(statistics.median(us), 2)
    return out


def bench_valu_rates(dev, steps):
    """Issue cost of vector-ALU operations on this GPU, in nanoseconds per wave-instruction per SIMD, from chains of one
    operation at 1, 2 and 4 waves per SIMD (bench_floor.hip).  What sum_lstm's arithmetic costs follows from these:
    a reciprocal or exp2 that stands between full-rate operations costs an issue slot like they do (the
    transcendental pipe runs beside the main one), so the kernel's arithmetic time is its instruction count, not its
    count of transcendentals."""
    floor = load_floor_kernels()
    if floor is None:
        return "bench_floor.so is not built"
    out_buf = torch.zeros(16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    cus = torch.cuda.get_device_properties(dev).multi_processor_count
    iters = 4096
    names = {0: "v_mul_f32", 1: "v_fma_f32", 2: "v_rcp_f32", 3: "v_exp_f32",
             4: "v_rcp_f32 + 3 dependent full-rate operations (per instruction)", 5: "v_lshlrev_b32",
             6: "v_cvt_f64_f32 . v_mul_f64 . v_cvt_f32_f64 (per instruction)", 7: "v_med3_f32"}
    per_round = {0: 1, 1: 1, 2: 1, 3: 1, 4: 4, 5: 1, 6: 3, 7: 1}
    out = {"compute_units": cus}
    for op, name in names.items():
        row = {}
        for waves in (1, 2, 4):
            f = lambda: floor.floor_valu_rate(op, cus * waves, iters, out_buf.data_ptr(), stream)
            f()
            us = statistics.median(event_times_us(f, max(5, steps // 10)))
            row[f"{waves}_waves_per_simd"] = round(us * 1e3 / (iters * 8 * per_round[op] * waves), 2)
        out[name] = row
    return out


def calibration_copy(dev):
    """A plain 1 GiB device copy: known bytes that a counter run of the same command scales FETCH_SIZE / WRITE_SIZE by."""
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev).fill_(1)
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


# extras that can be run alone with --only
ONLY = {
    "graph_node_floor": lambda ops, dev, a: bench_node_floor(dev, a.steps),
    "valu_issue_ns_per_wave_instruction": lambda ops, dev, a: bench_valu_rates(dev, a.steps),
    "decode_mix": lambda ops, dev, a: bench_decode_mix(ops, dev, a.steps),
    "speculator": lambda ops, dev, a: bench_speculator(ops, dev, a.steps, a.warmup),
    "sum_lstm_rows_sweep": lambda ops, dev, a: bench_lstm_rows(ops, dev, a.steps),
    "sum_lstm_width_sweep": lambda ops, dev, a: bench_lstm_widths(ops, dev, a.steps),
    "speculator_argmax_shapes": lambda ops, dev, a: bench_argmax_shapes(ops, dev, a.steps),
    "bulk_auto_bf16_cache": lambda ops, dev, a: bench_bulk_auto(ops, dev, a.steps),
    "speculator_argmax_512x128256": lambda ops, dev, a: bench_argmax(ops, dev, a.steps),
    "fp4_write_8b_layer": lambda ops, dev, a: bench_fp4(ops, dev, a.steps),
    "bulk_write_and_select_decode_70b": lambda ops, dev, a: bench_bulk_select(ops, dev, a.steps),
    "swiftkv_select_decode_70b": lambda ops, dev, a: bench_row_gather(ops, dev, a.steps),
    "bulk_fp8_70b_tp_sharded_heads_compact_pool": lambda ops, dev, a: bench_bulk_tp_heads(ops, dev, a.steps),
    "host_us_per_call": lambda ops, dev, a: bench_host_overhead(),
    "bulk_fp8_70b_source_before_pool": lambda ops, dev, a: bench_source_before_pool(ops, dev, a.steps),
}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--weight-gib", type=int, default=66, help="resident-weights placeholder allocated before the KV pool")
    ap.add_argument("--pool-blocks", type=int, default=65536, help="blocks per layer of the 80-layer KV pool")
    ap.add_argument("--no-extras", action="store_true", help="skip the speculator / decode-mix measurements")
    ap.add_argument("--no-cpu", action="store_true",
                    help="skip the CPU baselines and the host time per call (which runs child processes)")
    ap.add_argument("--placement-sweep", action="store_true",
                    help="instead of the benchmark, time the 70B-shape launch with the caches in each 8 GiB chunk "
                         "of the GPU's memory and spread over its regions; prints one JSON object")
    ap.add_argument("--only", choices=sorted(ONLY), default=None,
                    help="instead of the benchmark, run one of the extra measurements alone (for profiling it); "
                         "prints one JSON object")
    ap.add_argument("--host-overhead-route", choices=["py_custom_ops", "torch_ops", "torch_ext"], default=None, help=argparse.SUPPRESS)
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device copy (known bytes) so that a counter run of this "
                         "command can scale FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this path is built and measured on ONE GPU (every token, layer and row is "
                 "independent, so more GPUs only run the same kernel on their own share); use --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    if args.host_overhead_route:   # the child process of bench_host_overhead()
        print(json.dumps(host_overhead_route(args.host_overhead_route)), flush=True)
        return

    from arcticinference_amd import py_custom_ops as ops
    if not ops.try_load_torch_library():
        sys.exit("bench.py: libarctic_mi355x.so is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    log(f"device: {torch.cuda.get_device_name(0)}; host cores: {os.cpu_count()}")

    if args.placement_sweep:
        print(json.dumps({"placement_sweep": placement_sweep(ops, dev, max(5, args.steps // 5))}), flush=True)
        return
    if args.only:
        if args.calibrate_copy:
            calibration_copy(dev)
        print(json.dumps({args.only: ONLY[args.only](ops, dev, args)}), flush=True)
        return

    extras = {}
    # the same shape with nothing else on the GPU: 40 caches of 8192 blocks (10 GiB) right behind the
    # source, all inside one HBM region.  Always measured: the headline's roofline carries both placements.
    wc = BulkWorkload("70B-SwiftKV-compact", 16384, 40, 8, 128, 16, 8192, "fp8", 0.10, 2, 1.5, dev)
    fc = lambda: ops.reshape_and_cache_flash_bulk(*wc.args())
    for _ in range(args.warmup):
        fc()
    region_start, region_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    region_start.record()
    for _ in range(args.steps):
        fc()
    region_end.record()
    torch.cuda.synchronize()
    compact_mean = region_start.elapsed_time(region_end) * 1e3 / args.steps
    compact_us = event_times_us(fc, args.steps)
    compact = {"kernel_us_mean": round(compact_mean, 2), "kernel_us_median": round(statistics.median(compact_us), 2),
               "GBps": round(wc.bytes / compact_mean / 1e3, 1),
               "hbm_frac": round(wc.bytes / compact_mean / 1e3 / HBM_PEAK_GBS, 4),
               "placement": "source and 40 caches of 8192 blocks allocated first in the process (13 GiB; inside one HBM "
                            "region when the GPU was idle before)"}
    extras["bulk_fp8_70b_compact_pool"] = compact
    log(f"compact placement: {compact}")
    del wc, fc
    torch.cuda.empty_cache()

    # the map needs 66 + 160 GiB of the 268; should less be free, halve the pool rather than fail
    mem, pool_blocks = None, args.pool_blocks
    while mem is None:
        try:
            mem = ServingMemoryMap(dev, args.weight_gib, 80, 40, pool_blocks, 16, 8, 128, torch.uint8)
        except torch.OutOfMemoryError:
            if pool_blocks <= 2048:
                raise
            pool_blocks //= 2
            log(f"not enough free device memory for the pool; retrying with {pool_blocks} blocks per layer")
        if mem is None:
            torch.cuda.empty_cache()   # after the handler, when the half-built map is no longer referenced
    args.pool_blocks = pool_blocks
    log(f"memory map: {mem.describe()}")
    w = BulkWorkload("70B-SwiftKV", 16384, 40, 8, 128, 16, args.pool_blocks, "fp8", 0.10, 2, 1.5, dev,
                     bufs=mem.written_layers())
    fn = lambda: ops.reshape_and_cache_flash_bulk(*w.args())
    # The same-box reference points are measured here, right in front of the headline, on the same memory map.  They
    # also leave the GPU in the state a serving process keeps it in: behind an idle second the power management runs a
    # launch of this size 5-10 % slower for some twenty launches (per launch after 1 s of idle: 646, 585, 589, 599,
    # 610, 649, 655, 654, 654, 647, 637 ... 588 us), which a timed region of W = 5 and K = 20 would sit right inside
    # (620 us after an idle second, 588 us behind 12 ms of copies, 581 us in the steady state).
    extras["box_reference"] = box_reference(dev)
    for _ in range(args.warmup):
        fn()
    # the timed region: exactly K launches between two synchronisations; a pair of HIP events on the launch stream
    # brackets the same K launches, so the kernel's average duration comes from the region that `value` comes from
    # (the launches queue up behind each other: the host needs 20-odd us to issue one, the GPU 600 to run it)
    region_start, region_end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    region_start.record()
    for _ in range(args.steps):
        fn()
    region_end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall / args.steps * 1e3
    value = w.bytes / (wall / args.steps) / 1e9
    kernel_us = region_start.elapsed_time(region_end) * 1e3 / args.steps
    achieved = w.bytes / kernel_us / 1e3

    us = event_times_us(fn, args.steps)   # per launch, for the spread (a host hiccup between a launch's events shows here)
    if not args.no_extras:
        extras["bulk_fp8_70b_block_contiguous_slots_serving_map"] = bench_block_contiguous_slots(ops, dev, w, args.steps)
        extras["bulk_fp8_70b_decode_sizes_serving_map"] = bench_decode_sizes(ops, dev, mem, args.steps)
        extras["bulk_fp8_reference_decomposition"] = bench_reference_decomposition(ops, dev, w, mem, args.steps, kernel_us)
        # The speculator's operators and the decode step are measured here, while the serving map is held: their
        # tensors (activations of a few GB at most) are then allocated behind weights and KV pool, as in a serving
        # process, and in the physical order of a fresh process.  Allocated late, after the map has been handed back
        # and re-used, the same tensors land on other pages and the same kernels run 2-5 % slower or faster from run
        # to run (`--only NAME` measures in a process of its own).
        extras["speculator"] = bench_speculator(ops, dev, args.steps, args.warmup)
        extras["sum_lstm_rows_sweep"] = bench_lstm_rows(ops, dev, args.steps)
        torch.cuda.empty_cache()
        extras["decode_mix"] = bench_decode_mix(ops, dev, args.steps)
        torch.cuda.empty_cache()
        extras["speculator_argmax_512x128256"] = bench_argmax(ops, dev, args.steps)
        torch.cuda.empty_cache()
        extras["speculator_round_without_matrix_products"] = bench_speculator_round_glue(ops, dev, args.steps)
        torch.cuda.empty_cache()
    if args.calibrate_copy:
        calibration_copy(dev)
    traffic, traffic_fields = read_traffic(os.path.join(ROOT, "profiles", "kv_write_bulk_fp8_70b.traffic.txt"))
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic,
                "traffic_source": "not measured in this run (a process cannot read the HBM counters of its own kernels): "
                                  "carried over from profiles/kv_write_bulk_fp8_70b.traffic.txt, two rocprofv3 --pmc runs "
                                  "of this command, FETCH_SIZE and WRITE_SIZE scaled by a 1 GiB copy, measured on "
                                  f"{traffic_fields.get('measured_on', 'an unrecorded day')} with the library at commit "
                                  f"{traffic_fields.get('library_commit', 'unrecorded')}",
                "placement": "serving memory map (config.memory_map): the written caches span two of the HBM's three "
                             "address regions",
                "achieved_compact": compact["GBps"], "frac_compact": compact["hbm_frac"],
                "kernel_us_mean_compact": compact["kernel_us_mean"],
                "placement_compact": "the same launch with only the source and 40 caches of 8192 blocks on the GPU (13 GiB, "
                                     "one HBM region)",
                "kernel": "kv_write_bulk_kernel<bf16, e4m3>", "kernel_us_mean": round(kernel_us, 2),
                "kernel_us_mean_is": "HIP events around the K timed launches / K",
                "kernel_us_per_launch_mean": round(statistics.mean(us), 2),
                "kernel_us_median": round(statistics.median(us), 2),
                "kernel_us_p10": round(sorted(us)[len(us) // 10], 2),
                "kernel_us_p90": round(sorted(us)[(9 * len(us)) // 10], 2), "kernel_us_max": round(max(us), 2),
                "algorithmic_bytes": w.bytes}
    log(f"bulk fp8 70B shape: {ms_per_step:.3f} ms/step wall, kernel {kernel_us:.1f} us, {achieved:.0f} GB/s")

    cpu = cpu_pytorch = None
    if not args.no_cpu:
        cpu = cpu_baseline_bulk(w)
        log(f"cpu baseline: {cpu}")
        cpu_pytorch = cpu_baseline_bulk_pytorch(w)
        log(f"cpu baseline, PyTorch formulation: {cpu_pytorch}")

    workload_text = (f"bulk KV write at the 70B SwiftKV shape: {w.T} tokens x {w.L} layers x {w.H} KV heads x {w.D}, "
                     f"block {w.bs}, fp8-e4m3 cache, amax/448 scales, 10% slots = -1, the rest distinct random "
                     f"slots of a {w.NB}-block pool")
    cfg = {"workload": workload_text, "tokens": w.T, "valid_tokens": w.valid, "layers": w.L, "kv_heads": w.H,
           "head_size": w.D, "block_size": w.bs, "num_blocks": w.NB, "memory_map": mem.describe(),
           "parallelism": "single GPU"}
    del w, fn, mem
    torch.cuda.empty_cache()

    if not args.no_extras:
        w2 = BulkWorkload("8B-prefill", 8192, 16, 8, 128, 16, 8192, "fp8", 0.0, 1, 1.5, dev)
        f2 = lambda: ops.reshape_and_cache_flash_bulk(*w2.args())
        for _ in range(5):
            f2()
        m = statistics.median(event_times_us(f2, args.steps))
        extras["bulk_fp8_8b_prefill"] = {"kernel_us": round(m, 2), "GBps": round(w2.bytes / m / 1e3, 1),
                                         "hbm_frac": round(w2.bytes / m / 1e3 / HBM_PEAK_GBS, 4),
                                         "placement": "source and 16 caches of 8192 blocks allocated together (2.4 GiB)"}
        del w2, f2
        torch.cuda.empty_cache()
        # the same shape on the memory map of an 8B serving process: 8 GiB of weights, then the pool of all 32
        # layers sized like the 70B one, to fill 90 % of the HBM (229376 blocks = 7 GiB per layer); layers 16-31
        # are written
        try:
            mem8 = ServingMemoryMap(dev, 8, 32, 16, 229376, 16, 8, 128, torch.uint8)
            w3 = BulkWorkload("8B-prefill-serving", 8192, 16, 8, 128, 16, 229376, "fp8", 0.0, 1, 1.5, dev,
                              bufs=mem8.written_layers())
            f3 = lambda: ops.reshape_and_cache_flash_bulk(*w3.args())
            for _ in range(5):
                f3()
            extras["bulk_fp8_8b_prefill_serving_map"] = dict(kernel_stats(f3, args.steps, w3.bytes),
                                                             memory_map=mem8.describe())
            del mem8, w3, f3
        except torch.OutOfMemoryError:
            extras["bulk_fp8_8b_prefill_serving_map"] = "not enough free device memory"
        torch.cuda.empty_cache()
        extras["fp4_write_8b_layer"] = bench_fp4(ops, dev, args.steps)
        torch.cuda.empty_cache()
        if not args.no_cpu:
            extras["speculator"]["cpu_baseline"] = cpu_baseline_speculator()
        extras["bulk_auto_bf16_cache"] = bench_bulk_auto(ops, dev, args.steps)
        extras["bulk_fp8_70b_tp_sharded_heads_compact_pool"] = bench_bulk_tp_heads(ops, dev, args.steps)
        extras["swiftkv_select_decode_70b"] = bench_row_gather(ops, dev, args.steps)
        extras["bulk_write_and_select_decode_70b"] = bench_bulk_select(ops, dev, args.steps)
        torch.cuda.empty_cache()
        extras["suffix_decoding_cpu"] = bench_suffix_decoding()
        if not args.no_cpu:   # child processes: left out with the other host-side measurements
            extras["host_us_per_call"] = bench_host_overhead()
        log(f"extras: {extras}")

    result = {
        "metric": "bulk KV-write HBM GB/s (fp8-e4m3, 70B SwiftKV shape)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "fp8_e4m3",
        "data": "synthetic",
        "config": cfg,
        "roofline": roofline, "cpu_baseline": cpu, "cpu_baseline_pytorch": cpu_pytorch, "extras": extras,
    }
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
