"""The Rust binding crate (bindings/rust) cannot be compiled here (no rustc, no custos), so what CAN
be checked is checked mechanically: its `extern "C"` block declares exactly the functions of
include/sliced_hip.h with the same number of arguments, its constants carry the header's values,
and every op trait of the hot path has an impl in src/ops.rs."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "sliced_hip.h")
CRATE = os.path.join(ROOT, "bindings", "rust")


def header_functions():
    src = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    out = {}
    for name, args in re.findall(r"\b(slhip_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", src, flags=re.S):
        args = args.strip()
        out[name] = 0 if args in ("", "void") else len(args.split(","))
    return out


def rust_functions():
    src = open(os.path.join(CRATE, "src", "ffi.rs")).read()
    block = src[src.index('extern "C" {'):]
    out = {}
    for name, args in re.findall(r"pub fn (slhip_[a-z0-9_]+)\s*\((.*?)\)\s*->", block, flags=re.S):
        args = [a for a in args.split(",") if a.strip()]
        out[name] = len(args)
    return out


def test_ffi_declares_every_function_of_the_header_with_its_arity():
    h, r = header_functions(), rust_functions()
    assert len(h) >= 80
    assert sorted(h) == sorted(r), (sorted(set(h) - set(r)), sorted(set(r) - set(h)))
    assert {k: v for k, v in r.items() if h[k] != v} == {}


def test_ffi_constants_match_the_header():
    hdr = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    rs = open(os.path.join(CRATE, "src", "ffi.rs")).read()
    header_consts = {}
    for body in re.findall(r"enum\s*\{(.*?)\}", hdr, flags=re.S):
        for name, val in re.findall(r"(SLHIP_[A-Z0-9_]+)\s*=\s*(-?(?:0x)?[0-9a-fA-F]+)", body):
            header_consts[name] = int(val, 0)
    assert len(header_consts) >= 30
    rust_consts = {n: int(v, 0) for n, v in re.findall(r"pub const (SLHIP_[A-Z0-9_]+): \w+ = (-?(?:0x)?[0-9a-fA-F]+);", rs)}
    assert rust_consts == header_consts


def test_every_hot_path_trait_has_an_impl():
    ops = open(os.path.join(CRATE, "src", "ops.rs")).read()
    traits = ["Gemm", "GemmGrad", "Sum", "SumRows", "SumCols", "SumRowsGrad", "SumColsGrad", "Max", "MaxRows", "MaxCols",
              "MaxRowsGrad", "MaxColsGrad", "Mean", "MeanRows", "MeanCols", "MeanRowsGrad", "MeanColsGrad", "Softmax",
              "SoftmaxGrad", "Transpose", "TranposeGrad", "RowOp", "RowOpGrad", "ColOp", "ColOpGrad", "BinaryElementWise",
              "BinaryElementWiseGrad", "AddElementWiseGrad", "ApplyFunction", "UnaryGrad", "Diagflat", "DiagflatGrad", "Onehot"]
    for t in traits:
        direct = re.search(r"impl<[^{]*?>\s+%s<f32[^{]*?for HIP<Mods>" % t, ops, flags=re.S)
        by_macro = re.search(r"(reduction|broadcast_grad|max_grad)!\(%s," % t, ops)
        assert direct or by_macro, t
    # the crate says what it is
    readme = open(os.path.join(CRATE, "README.md")).read()
    assert "never been compiled" in readme
    for f in ("Cargo.toml", "build.rs", "src/lib.rs", "src/device.rs", "src/probe.rs", "src/graph.rs"):
        assert os.path.exists(os.path.join(CRATE, f)), f
