"""The C-ABI library: loads without a GPU, exports exactly what include/arctic_mi355x.h
declares, depends on no torch library, and rejects bad arguments before any launch."""
import ctypes
import os
import re
import subprocess

import pytest

from arcticinference_amd import _native

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "arctic_mi355x.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)          # drop comments
    return sorted(set(re.findall(r"\b(arctic_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    path = _native.library_path()
    assert path is not None, "libarctic_mi355x.so is not built (python -c 'import __graft_entry__ as g; g.build()')"
    return _native.load()


def test_header_and_binding_list_agree():
    assert declared_functions() == sorted(_native.EXPORTED_SYMBOLS)


def test_every_declared_symbol_is_exported(lib):
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    out = subprocess.run(["nm", "-D", "--defined-only", _native.library_path()], capture_output=True, text=True).stdout
    exported_c = {l.split()[-1] for l in out.splitlines() if " T " in l and not l.split()[-1].startswith("_Z")}
    assert set(declared_functions()) <= exported_c


def test_abi_version_matches_header(lib):
    m = re.search(r"#define\s+ARCTIC_ABI_VERSION\s+(\d+)", open(HEADER).read())
    assert lib.arctic_abi_version() == int(m.group(1)) == _native.ABI_VERSION


def test_no_torch_dependency():
    # the NEEDED entries of the ELF file itself (ldd would also resolve transitive paths)
    out = subprocess.run(["readelf", "-d", _native.library_path()], capture_output=True, text=True).stdout
    needed = [l.split("[")[-1].rstrip("]") for l in out.splitlines() if "(NEEDED)" in l]
    assert needed, out
    assert not any(("torch" in n) or ("c10" in n) or ("python" in n.lower()) for n in needed), needed
    assert any("amdhip64" in n for n in needed), needed


def test_header_compiles_as_plain_c(tmp_path):
    src = tmp_path / "t.c"
    src.write_text('#include "arctic_mi355x.h"\nint main(void) { return ARCTIC_ABI_VERSION >= 1 ? 0 : 1; }\n')
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-c", str(src), "-o",
                    str(tmp_path / "t.o")], check=True)


def test_argument_errors_return_codes_without_launching(lib):
    # every call below fails validation, so nothing is enqueued and no GPU is needed
    rc = lib.arctic_speculator_ln(None, None, None, None, 4, 128, 128, 1e-6, _native.DTYPE_F32, None)
    assert rc == 2 and b"only fp16 and bf16" in lib.arctic_last_error()
    rc = lib.arctic_speculator_ln(None, None, None, None, 4, 0, 0, 1e-6, _native.DTYPE_BF16, None)
    assert rc == 1 and b"hidden size must be > 0" in lib.arctic_last_error()
    rc = lib.arctic_speculator_ln(None, None, None, None, 4, 128, 128, 1e-6, _native.DTYPE_BF16, None)
    assert rc == 1 and b"null" in lib.arctic_last_error()
    rc = lib.arctic_sum_lstm(*([None] * 9), 4, 64, 256, 256, 64, 64, 1.0, 1e-6, 1e-6, 0, _native.DTYPE_F32, None)
    assert rc == 2 and b"sum_lstm: only fp16 and bf16" in lib.arctic_last_error()
    rc = lib.arctic_reshape_and_cache_flash_bulk(None, None, 0, 0, None, None, None, None, None, 4, 2, 2, 64, 16, 0,
                                                 0, _native.DTYPE_BF16, 7, None)
    assert rc == 2 and b"Unsupported data type of kv cache" in lib.arctic_last_error()
    rc = lib.arctic_reshape_and_cache_flash_bulk(None, None, 0, 0, None, None, None, None, None, 4, 2, 2, 64, 16, 0,
                                                 0, 9, _native.KV_AUTO, None)
    assert rc == 2 and b"Unsupported input type of kv cache" in lib.arctic_last_error()
    rc = lib.arctic_reshape_and_cache_flash_bulk(None, None, 0, 0, None, None, None, None, None, 4, 100000, 2, 64, 16,
                                                 0, 0, _native.DTYPE_BF16, _native.KV_AUTO, None)
    assert rc == 1 and b"num_layers" in lib.arctic_last_error()
    # empty problems are successful no-ops (reference: reshape_and_cache_flash_bulk.cu:87-89)
    assert lib.arctic_reshape_and_cache_flash_bulk(None, None, 0, 0, None, None, None, None, None, 4, 0, 2, 64, 16, 0,
                                                   0, _native.DTYPE_BF16, _native.KV_AUTO, None) == 0
    assert lib.arctic_speculator_ln(None, None, None, None, 0, 128, 128, 1e-6, _native.DTYPE_BF16, None) == 0
    # the entry points of the "next" rows validate the same way
    bulk = (None, None, 0, 0, None, None, None, None, None, 4, 2, 2, 64, 16, 0, 0, _native.DTYPE_BF16, _native.KV_AUTO)
    rc = lib.arctic_reshape_and_cache_flash_bulk_select(*bulk, None, None, 8, 4, 4, None, None, 0, 0, None)
    assert rc == 1 and b"null tensor pointer" in lib.arctic_last_error()
    fake = ctypes.c_void_p(256)        # never dereferenced: the calls below are refused on their other arguments
    held = (fake, fake, 0, 0, fake, fake, None, None, fake) + bulk[9:]
    rc = lib.arctic_reshape_and_cache_flash_bulk_select(*held, None, fake, 8, 4, 4, None, None, 0, 0, None)
    assert rc == 1 and b"null keys_out or values_out" in lib.arctic_last_error()
    rc = lib.arctic_reshape_and_cache_flash_bulk_select(*held, None, None, 8, 4, 4, fake, fake, 0, 0, None)
    assert rc == 1 and b"index list is missing" in lib.arctic_last_error()
    rc = lib.arctic_reshape_and_cache_flash_bulk_select(*held, None, fake, 8, 5000, 5000, fake, fake, 0, 0, None)
    assert rc == 1 and b"longer than 2048 entries" in lib.arctic_last_error()
    rc = lib.arctic_reshape_and_cache_flash_bulk_select(*held, None, fake, 2, 4, 4, fake, fake, 0, 0, None)
    assert rc == 2 and b"int32 or int64" in lib.arctic_last_error()
    assert lib.arctic_reshape_and_cache_flash_bulk_select(*bulk[:10], 0, *bulk[11:], None, None, 8, 4, 4, None, None, 0, 0,
                                                          None) == 0
    static = (*bulk[:9], 1 << 20, *bulk[10:], None, 8, 4, 1 << 20, None, None, 0, 0, None)
    rc = lib.arctic_reshape_and_cache_flash_bulk_select_static(*static)
    assert rc == 1 and b"exceeds the 262144 tokens" in lib.arctic_last_error()
    rc = lib.arctic_build_row_map(None, 8, None, 2, 0, None)
    assert rc == 2 and b"int32 or int64" in lib.arctic_last_error()
    rc = lib.arctic_build_row_map(None, 8, None, 8, 0, None)
    assert rc == 1 and b"null" in lib.arctic_last_error()
    assert lib.arctic_build_row_map(None, 0, None, 8, 0, None) == 0
    rc = lib.arctic_sum_lstm_embedded(*([None] * 10), 4, 64, 256, 64, 64, 64, 100, 1.0, 1e-6, 1e-6, 0, _native.DTYPE_BF16, None)
    assert rc == 1 and b"null token ids" in lib.arctic_last_error()
    rc = lib.arctic_speculator_embed_add_ln_act(None, None, None, None, None, None, 4, 128, 128, 128, 10, 1.0, 1e-6, 1, 1.0,
                                                _native.DTYPE_BF16, None)
    assert rc == 1 and b"null embedding table or token ids" in lib.arctic_last_error()
    rc = lib.arctic_argmax_clamp(None, None, 4, 0, 0, 0, _native.DTYPE_BF16, None)
    assert rc == 1 and b"cols > 0" in lib.arctic_last_error()
    rc = lib.arctic_gather_rows(9, None, None, None, None, None, None, 8, 1, 1, 0, None)
    assert rc == 1 and b"between 0 and 8 tensors" in lib.arctic_last_error()


def test_product_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "arcticinference_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".cpp", ".h")) or f == "Makefile":
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), f"{f} mentions the oracle"
