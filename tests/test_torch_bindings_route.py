"""The second integration route: the reference's own TORCH_LIBRARY block (csrc/custom_ops/torch_bindings.cpp, compiled
unchanged from where the reference lies) registered over libarctic_mi355x.so through the forwards of
arcticinference_amd/csrc/torch_forwards.cpp.  `make -C oracle torch_ext` builds the extension into oracle/_ref (it holds
compiled reference code, so it stays out of version control).  Each check runs in a process of its own: the extension
and the Python module both define the arctic_inference namespace, and one process can hold only one definition."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXT = os.path.join(ROOT, "oracle", "_ref", "arctic_torch_ext.so")
REFERENCE = "/root/reference"


def ensure_built():
    if os.path.exists(EXT):
        return
    if not os.path.isdir(os.path.join(REFERENCE, "csrc", "custom_ops")):
        pytest.skip("oracle/_ref/arctic_torch_ext.so is not built and the reference's sources are not here to build it")
    from arcticinference_amd import _native
    if _native.library_path() is None:
        _native.build()
    subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "torch_ext", f"REFERENCE={REFERENCE}"], check=True,
                   capture_output=True)


def run_script(body: str) -> str:
    script = (f"import sys\nsys.path.insert(0, {ROOT!r})\nsys.path.insert(0, {os.path.join(ROOT, 'tests')!r})\n"
              f"import torch\ntorch.ops.load_library({EXT!r})\n" + body)
    proc = subprocess.run([sys.executable, "-c", script], capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    return proc.stdout


def test_the_reference_binding_file_registers_the_same_schemas():
    ensure_built()
    out = run_script(
        "for name in ('reshape_and_cache_flash_bulk', 'reshape_and_cache_flash_fp4', 'speculator_ln_cuda', 'sum_lstm_cuda'):\n"
        "    print(name, '|', getattr(torch.ops.arctic_inference, name).default._schema)\n")
    got = dict(line.split(" | ", 1) for line in out.strip().splitlines())
    from arcticinference_amd import py_custom_ops
    import torch
    for name, text in py_custom_ops._SCHEMAS.items():
        want = str(torch._C.parse_schema("arctic_inference::" + text))
        assert got[name].strip() == want, f"{name}: {got[name]} != {want}"


GPU_BODY = r'''
import oracle
from helpers import assert_bulk_equal, assert_close, bulk_args, bulk_case_to, make_bulk_case, make_lstm_case
ops = torch.ops.arctic_inference
DEV = "cuda:0"
# bulk write: fp8 and bf16 caches, padding
for kv in ("fp8", "auto"):
    case = make_bulk_case(T=300, L=6, H=8, D=128, bs=16, NB=32, kv_cache_dtype=kv, seed=70, std=1.5, pad_fraction=0.1)
    d = bulk_case_to(case, DEV)
    ops.reshape_and_cache_flash_bulk(*bulk_args(d))
    torch.cuda.synchronize()
    oracle.reshape_and_cache_flash_bulk(*bulk_args(case))
    assert_bulk_equal(d["bufs"], case["bufs"])
# norm and LSTM step: the reference's output conventions and the oracle's values
c = make_lstm_case(rows=48, D=1024, seed=71, padD=8)
dc = {k: None if v is None else v.to(DEV) for k, v in c.items()}
pc = torch.empty(48, 1032, dtype=torch.bfloat16, device=DEV)[:, :1024]
pc.copy_(dc["prev_cell"])
state, cell = ops.sum_lstm_cuda(dc["states"], dc["z4"], pc, dc["w_cell"], dc["b_cell"], dc["w_state"], dc["b_state"],
                                0.35, 1e-6, 1e-6, False)
assert state.stride() == pc.stride() and cell.stride() == pc.stride()
want_state, want_cell = oracle.sum_lstm(c["states"], c["z4"], c["prev_cell"], c["w_cell"], c["b_cell"], c["w_state"],
                                        c["b_state"], 0.35, 1e-6, 1e-6, False)
assert_close(state, want_state, what="state")
assert_close(cell, want_cell, what="cell")
x = c["prev_cell"].contiguous()
y = ops.speculator_ln_cuda(x.to(DEV).view(6, 8, 1024), dc["w_cell"], None, 1e-6)
assert y.shape == (6, 8, 1024)
assert_close(y.view(48, 1024), oracle.speculator_ln(x, c["w_cell"], None, 1e-6), what="norm")
try:
    ops.speculator_ln_cuda(x.float().to(DEV), None, None, 1e-6)
    raise SystemExit("an fp32 input was accepted")
except RuntimeError as e:
    assert "only fp16 and bf16" in str(e)
# NVFP4-style write: bytes equal to the oracle's
T, H, D, bs, NB = 64, 4, 64, 16, 8
g = torch.Generator().manual_seed(72)
key, value = torch.randn(T, H, D, generator=g).bfloat16(), torch.randn(T, H, D, generator=g).bfloat16()
slots = torch.randperm(NB * bs, generator=g)[:T]
caches = [torch.zeros(NB, bs, H, D // 2, dtype=torch.uint8) for _ in range(2)] + \
         [torch.zeros(NB, bs, H, D // 16, dtype=torch.uint8) for _ in range(2)]
dcaches = [t.to(DEV) for t in caches]
one = torch.ones(())
ops.reshape_and_cache_flash_fp4(key.to(DEV), value.to(DEV), dcaches[0], dcaches[1], slots.to(DEV), "fp4", one.to(DEV),
                                one.to(DEV), dcaches[2], dcaches[3])
torch.cuda.synchronize()
oracle.reshape_and_cache_flash_fp4(key, value, caches[0], caches[1], caches[2], caches[3], slots, "fp4", one, one)
for a, b in zip(dcaches, caches):
    assert torch.equal(a.cpu(), b)
print("route ok")
'''


@pytest.mark.gpu
def test_one_call_per_operator_through_the_reference_binding_file():
    if not os.path.exists(EXT):
        pytest.skip("oracle/_ref/arctic_torch_ext.so is not built (it is built where the reference's sources are)")
    assert "route ok" in run_script(GPU_BODY)
