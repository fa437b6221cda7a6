"""Writes the golden fixtures in this directory.

    python tests/golden/make_golden.py

The reference ships no golden vectors for this path (its tests compare two live
GPU implementations), so these fixtures are produced here from the closed forms
of the three operators, evaluated with torch library routines only - index
assignment and the CPU float8 casts for the KV write, float64 rsqrt / mean /
sigmoid / gelu for the speculator operators.  Nothing under oracle/ and nothing
from the shipped package is used: the fixtures are an independent statement of
the expected results, for both the CPU oracle and the GPU kernels to be checked
against.

Closed forms (reference: csrc/custom_ops/reshape_and_cache_flash_bulk.cu:12-60,
quant_utils.cuh:456-489, speculator_ln.cu:21-107, sum_lstm.cu:28-191 and the
in-test restatements tests/unit_tests/test_speculator_ln.py:41-48,
tests/unit_tests/test_sum_lstm.py:22-70).
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
F64 = torch.float64


def bits16(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy()


# --------------------------------------------------------------------------- #
def bulk_case(name, out, *, T, L, H, D, bs, NB, src_dtype, kv, seed, pad):
    g = torch.Generator().manual_seed(seed)
    n = H * D
    keys = (torch.randn(T, L * n, generator=g) * 1.5).to(src_dtype)
    values = (torch.randn(T, L * n, generator=g) * 1.5).to(src_dtype)
    slots = torch.randperm(NB * bs, generator=g)[:T].to(torch.int64)
    slots[torch.randperm(T, generator=g)[:pad]] = -1
    quant = kv != "auto"
    row_bytes = n * (1 if quant else 2)
    init = torch.randint(0, 256, (L, 2, NB * bs, row_bytes), generator=g, dtype=torch.uint8)
    final = init.clone()
    k_scales, v_scales = [], []
    for l in range(L):
        for which, src, scales in ((0, keys, k_scales), (1, values, v_scales)):
            x = src[:, l * n:(l + 1) * n]
            if quant:
                tdt, mx = (torch.float8_e5m2, 57344.0) if kv == "fp8_e5m2" else (torch.float8_e4m3fn, 448.0)
                s = (x.float().abs().max() / mx).to(torch.float32)
                scales.append(float(s))
                rows = (x.float() / s).clamp(-mx, mx).to(tdt).view(torch.uint8)
            else:
                scales.append(1.0)
                rows = x.contiguous().view(torch.uint8).view(T, row_bytes)
            for t in range(T):
                if slots[t] >= 0:
                    final[l, which, slots[t]] = rows[t]
    out[f"{name}.dims"] = np.array([H, D, bs, NB, L], dtype=np.int64)
    out[f"{name}.keys"] = bits16(keys)
    out[f"{name}.values"] = bits16(values)
    out[f"{name}.slots"] = slots.numpy()
    out[f"{name}.cache_init"] = init.view(L, -1).numpy()
    out[f"{name}.cache_out"] = final.view(L, -1).numpy()
    out[f"{name}.k_scales"] = np.array(k_scales, dtype=np.float32)
    out[f"{name}.v_scales"] = np.array(v_scales, dtype=np.float32)


# --------------------------------------------------------------------------- #
def rms_norm64(x, eps, w, b):
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
    if w is not None:
        y = y * w
    if b is not None:
        y = y + b
    return y


def ln_cases(out):
    names = []
    seed = 300
    for dtype, dn in ((torch.float16, "f16"), (torch.bfloat16, "bf16")):
        for affine in (False, True):
            for shape in ((4, 128), (3, 260), (2, 513), (2, 2, 1024)):
                seed += 1
                g = torch.Generator().manual_seed(seed)
                x = torch.randn(*shape, generator=g).to(dtype)
                w = torch.randn(shape[-1], generator=g).to(dtype) if affine else None
                b = torch.randn(shape[-1], generator=g).to(dtype) if affine else None
                y = rms_norm64(x.to(F64), 1e-6, None if w is None else w.to(F64), None if b is None else b.to(F64))
                name = f"{dn}_{'affine' if affine else 'plain'}_{'x'.join(map(str, shape))}"
                names.append(name)
                out[f"{name}.x"] = bits16(x)
                if affine:
                    out[f"{name}.w"] = bits16(w)
                    out[f"{name}.b"] = bits16(b)
                out[f"{name}.want"] = y.to(torch.float32).numpy()
    out["names"] = np.array(names)


def lstm_cases(out):
    names = []
    cases = [dict(rows=1, D=64, pad4=0, padD=0), dict(rows=4, D=128, pad4=7, padD=3),
             dict(rows=3, D=256, pad4=0, padD=0), dict(rows=2, D=512, pad4=16, padD=8)]
    for dtype, dn in ((torch.float16, "f16"), (torch.bfloat16, "bf16")):
        for ci, c in enumerate(cases):
            for fast in (False, True):
                wb_cell, wb_state = (ci % 2 == 0), (ci < 2) or fast
                rows, D = c["rows"], c["D"]
                g = torch.Generator().manual_seed(1000 * ci + 10 * fast + (dtype == torch.float16))
                states = torch.randn(rows, 4 * D + c["pad4"], generator=g).to(dtype)[:, :4 * D]
                z4 = torch.randn(rows, 4 * D + c["pad4"], generator=g).to(dtype)[:, :4 * D]
                pc = torch.randn(rows, D + c["padD"], generator=g).to(dtype)[:, :D]
                vec = lambda m, on: (m + 0.5 * torch.randn(D, generator=g)).to(dtype) if on else None
                w_cell, b_cell = vec(1.0, wb_cell), vec(0.0, wb_cell)
                w_state, b_state = vec(1.0, wb_state), vec(0.0, wb_state)
                alpha, eps_c, eps_s = 0.35, 1e-6, 1e-5
                alpha32 = float(torch.tensor(alpha, dtype=torch.float32))
                d = lambda t: None if t is None else t.to(F64)
                s, z = states.to(F64), z4.to(F64)
                pre = s + alpha32 * z
                pf, pi, po, pcell = pre.split(D, dim=-1)
                act = lambda v: torch.nn.functional.gelu(v, approximate="tanh" if fast else "none")
                c_new = pc.to(F64) * torch.sigmoid(pf) + act(rms_norm64(pcell, eps_c, d(w_cell), d(b_cell))) * torch.sigmoid(pi)
                cell_rounded = c_new.to(dtype)              # what out_cell holds and the state phase reads back
                inv_s = torch.rsqrt(c_new.pow(2).mean(-1, keepdim=True) + eps_s)   # from the UNROUNDED cell
                sn = cell_rounded.to(F64) * inv_s
                if w_state is not None:
                    sn = sn * d(w_state)
                if b_state is not None:
                    sn = sn + d(b_state)
                state = act(sn) * torch.sigmoid(po)
                name = f"{dn}_case{ci}_{'tanh' if fast else 'erf'}"
                names.append(name)
                out[f"{name}.meta"] = np.array([rows, D, c["pad4"], c["padD"], int(fast)], dtype=np.int64)
                out[f"{name}.scalars"] = np.array([alpha, eps_c, eps_s], dtype=np.float64)
                out[f"{name}.states"] = bits16(states)
                out[f"{name}.z4"] = bits16(z4)
                out[f"{name}.prev_cell"] = bits16(pc)
                for k, v in (("w_cell", w_cell), ("b_cell", b_cell), ("w_state", w_state), ("b_state", b_state)):
                    if v is not None:
                        out[f"{name}.{k}"] = bits16(v)
                out[f"{name}.want_cell"] = c_new.to(torch.float32).numpy()
                out[f"{name}.want_state"] = state.to(torch.float32).numpy()
    out["names"] = np.array(names)


def main():
    bulk = {}
    bulk_case("bf16_auto", bulk, T=24, L=2, H=2, D=32, bs=4, NB=8, src_dtype=torch.bfloat16, kv="auto", seed=21, pad=0)
    bulk_case("bf16_fp8", bulk, T=24, L=3, H=2, D=32, bs=4, NB=8, src_dtype=torch.bfloat16, kv="fp8", seed=22, pad=5)
    bulk_case("f16_fp8_e5m2", bulk, T=16, L=2, H=1, D=64, bs=8, NB=4, src_dtype=torch.float16, kv="fp8_e5m2",
              seed=23, pad=3)
    np.savez_compressed(os.path.join(HERE, "bulk_kv_write.npz"), **bulk)
    ln = {}
    ln_cases(ln)
    np.savez_compressed(os.path.join(HERE, "speculator_ln.npz"), **ln)
    lstm = {}
    lstm_cases(lstm)
    np.savez_compressed(os.path.join(HERE, "sum_lstm.npz"), **lstm)
    for f in ("bulk_kv_write.npz", "speculator_ln.npz", "sum_lstm.npz"):
        print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
