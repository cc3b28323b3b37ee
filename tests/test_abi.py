"""The C-ABI library loads and exports every symbol include/fieldfare_moe.h declares (no GPU needed)."""
import ctypes
import re
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def declared_symbols():
    text = (ROOT / "include" / "fieldfare_moe.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ffmoe_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    syms = declared_symbols()
    for name in ("ffmoe_create", "ffmoe_destroy", "ffmoe_upload_layer", "ffmoe_router", "ffmoe_verify",
                 "ffmoe_verify_partials", "ffmoe_reduce_token_major", "ffmoe_gemv_int4", "ffmoe_dequant_expert"):
        assert name in syms


def test_library_exports_every_declared_symbol():
    import fieldfare_moe
    assert fieldfare_moe.LIB_PATH.exists(), "the session fixture builds the library when it is missing"
    lib = ctypes.CDLL(str(fieldfare_moe.LIB_PATH))
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, f"not exported: {missing}"
    assert sorted(fieldfare_moe.EXPORTS) == declared_symbols()


def test_create_without_gpu_fails_loudly():
    import torch
    import fieldfare_moe
    if torch.cuda.is_available():
        return
    L = fieldfare_moe.lib()
    shape = fieldfare_moe.Shape(128, 64, 16, 8, 1, 16)
    h = ctypes.c_void_p()
    err = ctypes.c_char_p()
    rc = L.ffmoe_create(0, ctypes.byref(shape), ctypes.byref(h), ctypes.byref(err))
    assert rc != 0 and err.value
    try:
        fieldfare_moe.Context(128, 64, 16)
        raise AssertionError("Context() must not succeed without a GPU")
    except RuntimeError:
        pass
