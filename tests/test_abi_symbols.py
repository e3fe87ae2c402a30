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


# ---- the header and the library from plain C (tests/abi_consumer/consumer.c)
CONSUMER_SRC = os.path.join(ROOT, "tests", "abi_consumer", "consumer.c")


def consumer_binary():
    from sliced_amd import build
    if not os.path.exists(build.CONSUMER):
        build.build_consumer()
    return build.CONSUMER


def test_header_is_c99():
    import subprocess
    r = subprocess.run(["gcc", "-std=c99", "-pedantic", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I",
                        os.path.join(ROOT, "include"), CONSUMER_SRC], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout


def test_c_consumer_links_and_fails_loudly_without_a_gpu():
    import subprocess
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    r = subprocess.run([consumer_binary()], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=60)
    assert r.returncode == 2, (r.returncode, r.stdout, r.stderr)
    assert "device" in r.stderr.lower() and "PASS" not in r.stdout


@pytest.mark.gpu
def test_c_consumer_runs_a_layer_through_the_abi():
    """The C99 program calls init, malloc, h2d, sgemm, add_row, relu, softmax, Tgemm, sum_rows, transpose, d2h
    and compares with its own loops: no Python between the caller and the library."""
    import subprocess
    r = subprocess.run([consumer_binary()], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    print(r.stdout, r.stderr, flush=True)
    assert r.returncode == 0, (r.returncode, r.stdout, r.stderr)
    assert r.stdout.strip().splitlines()[-1] == "PASS"


def test_ctypes_prototypes_match_the_header_type_by_type():
    """Every argument of sliced_amd/_lib.py's table against the C type the header declares: a pointer where the
    header has a pointer (of whatever kind: the table passes addresses), size_t, int32_t, uint64_t and float where it
    has those, and the return types."""
    from test_rust_binding import header_signatures
    # (size_t and uint64_t are one ctypes class on this ABI, 64 bits both: one kind)
    kinds = {"int32_t": "i32", "uint32_t": "u32", "uint64_t": "u64", "size_t": "u64", "float": "f32"}
    assert C.sizeof(C.c_size_t) == 8

    def c_kind(t):
        t = t.strip()
        if "*" in t:
            return "ptr"
        return kinds[t.replace("const ", "")]

    def ct_kind(t):
        if t in (C.c_void_p, C.c_char_p) or (isinstance(t, type) and issubclass(t, C._Pointer)):
            return "ptr"
        return {C.c_int32: "i32", C.c_uint32: "u32", C.c_uint64: "u64", C.c_size_t: "u64", C.c_float: "f32"}[t]

    sigs = header_signatures()
    assert sorted(sigs) == sorted(_lib.PROTOTYPES)
    wrong = []
    for name, (ret, params) in sigs.items():
        want = [c_kind(p) for p in params]
        got = [ct_kind(t) for t in _lib.PROTOTYPES[name]]
        want_ret = "ptr" if "*" in ret else kinds[ret]
        got_ret = ct_kind(_lib._RESTYPE.get(name, C.c_int32))
        if want != got or want_ret != got_ret:
            wrong.append((name, want, got, want_ret, got_ret))
    assert not wrong, wrong[:5]
