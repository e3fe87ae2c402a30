"""CPU-only checks of the drop-in boundary: the built library exports every symbol that
include/sliced_hip.h declares, the Python binding covers exactly that set, and without a GPU
the library fails loudly instead of computing anything on the host."""
import ctypes as C
import os
import re

import pytest

from sliced_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "sliced_hip.h")


def declared_symbols():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    return sorted(set(re.findall(r"\b(slhip_[a-z0-9_]+)\s*\(", src)))


def test_header_declares_symbols():
    syms = declared_symbols()
    assert len(syms) >= 50
    for must in ("slhip_sgemm", "slhip_softmax", "slhip_softmax_grad", "slhip_transpose", "slhip_sum_rows",
                 "slhip_max_cols_grad", "slhip_add_row", "slhip_ew_chain", "slhip_sgd_step"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_lib.LIB_PATH), "build first: python -m sliced_amd.build"
    lib = C.CDLL(_lib.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, missing


def test_binding_matches_header():
    assert sorted(_lib.PROTOTYPES) == declared_symbols()
    _lib.load()


def test_fails_loudly_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = _lib.load()
    h = C.c_void_p()
    rc = lib.slhip_init(0, C.byref(h))
    assert rc != 0 and not h.value
    assert b"device" in lib.slhip_last_error_string().lower()
    with pytest.raises(_lib.SlicedHipError):
        from sliced_amd.device import Context
        Context(0)


def test_argument_validation_needs_no_gpu():
    lib = _lib.load()
    # a null context is rejected before anything touches the device
    assert lib.slhip_sgemm(None, 0, 0, 4, 4, 4, None, None, None, 0.0) == -1
    assert lib.slhip_softmax(None, 2, 3, None, None) == -1
    assert lib.slhip_transpose(None, 2, 3, None, None, 0.0) == -1
    assert b"null" in lib.slhip_last_error_string().lower()
