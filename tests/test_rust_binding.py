"""The Rust binding crate (bindings/rust) cannot be compiled here (no rustc, no custos), so what CAN
be checked is checked mechanically: its `extern "C"` block declares exactly the functions of
include/sliced_hip.h with the same number of arguments and, argument by argument, the Rust type
that the C type maps to (pointer depth and constness included), its constants carry the header's
values, and every op trait of the hot path has an impl in src/ops.rs."""
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


# ---- argument and return TYPES, one by one
def c_type_to_rust(t):
    """The Rust FFI type that a C parameter type of the header has to be declared as."""
    t = re.sub(r"\s+", " ", t.strip())
    t = t.replace(" *", "*").replace("* ", "*")
    base = {"int32_t": "i32", "uint32_t": "u32", "uint64_t": "u64", "size_t": "usize", "float": "f32", "char": "c_char",
            "void": "c_void", "slhip_ctx": "SlhipCtx", "slhip_graph": "SlhipGraph", "slhip_event": "SlhipEvent",
            "slhip_ew_insn": "SlhipEwInsn"}
    m = re.fullmatch(r"(const )?(struct )?(\w+)((?:\*(?: ?const)?)*)", t)
    assert m, t
    const_base, name, stars = bool(m.group(1)), m.group(3), m.group(4)
    assert name in base, t
    out = base[name]
    # pointer levels from the innermost outwards: `const T*` is *const T; `T* const*` is *const *mut T
    levels = re.findall(r"\*( ?const)?", stars)
    pointee_const = const_base
    for lv in levels:
        out = ("*const " if pointee_const else "*mut ") + out
        pointee_const = bool(lv)
    return out


def split_c_params(args):
    args = args.strip()
    if args in ("", "void"):
        return []
    out = []
    for a in args.split(","):
        a = re.sub(r"/\*.*?\*/", "", a).strip()
        a = re.sub(r"\s+", " ", a)
        m = re.fullmatch(r"(.*?[\*\s])(\w+)", a)     # type, then the parameter's name
        assert m, a
        out.append(m.group(1).strip())
    return out


def header_signatures():
    src = re.sub(r"/\*.*?\*/", "", open(HEADER).read(), flags=re.S)
    sigs = {}
    for ret, name, args in re.findall(r"\n([\w \*]+?)\s*\b(slhip_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", src, flags=re.S):
        sigs[name] = (ret.strip(), split_c_params(args))
    return sigs


def rust_signatures():
    src = open(os.path.join(CRATE, "src", "ffi.rs")).read()
    block = src[src.index('extern "C" {'):]
    block = re.sub(r"//[^\n]*", "", block)
    sigs = {}
    for name, args, ret in re.findall(r"pub fn (slhip_[a-z0-9_]+)\s*\((.*?)\)\s*->\s*([^;]+);", block, flags=re.S):
        types = []
        for a in [x for x in args.split(",") if x.strip()]:
            t = a.split(":", 1)[1]
            t = re.sub(r"\s+", " ", t.strip())
            t = re.sub(r"\b(?:std::os::raw::|std::ffi::|core::ffi::)", "", t)
            types.append(t)
        sigs[name] = (re.sub(r"\s+", " ", re.sub(r"\b(?:std::os::raw::|std::ffi::|core::ffi::)", "", ret.strip())), types)
    return sigs


def test_ffi_argument_and_return_types_match_the_header():
    h, r = header_signatures(), rust_signatures()
    assert sorted(h) == sorted(r)
    wrong = []
    for name, (ret, params) in h.items():
        want_ret = c_type_to_rust(ret)
        want = [c_type_to_rust(p) for p in params]
        got_ret, got = r[name]
        if want_ret != got_ret or want != got:
            wrong.append((name, want_ret, want, got_ret, got))
    assert not wrong, wrong[:5]


def test_the_declarations_shown_in_the_integration_guide_match_the_header():
    """INTEGRATION.md shows a part of the FFI block; what it shows has to be what the header declares."""
    md = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    blocks = re.findall(r"```rust\n(.*?)```", md, flags=re.S)
    shown = {}
    for b in blocks:
        if 'extern "C"' not in b:
            continue
        b = re.sub(r"//[^\n]*", "", b)
        for name, args, ret in re.findall(r"pub fn (slhip_[a-z0-9_]+)\s*\((.*?)\)\s*->\s*([^;]+);", b, flags=re.S):
            strip = lambda t: re.sub(r"\s+", " ", re.sub(r"\b(?:std::os::raw::|std::ffi::|core::ffi::)", "", t.strip()))
            shown[name] = (strip(ret), [strip(a.split(":", 1)[1]) for a in args.split(",") if a.strip()])
    assert len(shown) >= 30
    h = header_signatures()
    wrong = [(n, shown[n], (c_type_to_rust(h[n][0]), [c_type_to_rust(p) for p in h[n][1]])) for n in shown
             if n not in h or shown[n] != (c_type_to_rust(h[n][0]), [c_type_to_rust(p) for p in h[n][1]])]
    assert not wrong, wrong[:3]


def test_every_call_into_the_library_passes_as_many_arguments_as_the_header_declares():
    """The crate's sources cannot be type-checked here; the number of arguments of every ffi call can."""
    arity = header_functions()
    calls = 0
    for f in ("ops.rs", "device.rs", "graph.rs", "probe.rs"):
        src = open(os.path.join(CRATE, "src", f)).read()
        src = re.sub(r"//[^\n]*", "", src)
        for m in re.finditer(r"\b(slhip_[a-z0-9_]+)\s*\(", src):
            name = m.group(1)
            if name not in arity:
                continue
            i, depth, args, cur = m.end(), 1, [], ""
            while depth:
                ch = src[i]
                if ch in "([{":
                    depth += 1
                elif ch in ")]}":
                    depth -= 1
                    if depth == 0:
                        break
                if ch == "," and depth == 1:
                    args.append(cur)
                    cur = ""
                else:
                    cur += ch
                i += 1
            if cur.strip():
                args.append(cur)
            if re.search(r"\bfn\s*$", src[max(0, m.start() - 12):m.start()]):
                continue                      # a wrapper's own definition, not a call
            calls += 1
            assert len(args) == arity[name], (f, name, len(args), arity[name], src[m.start():i + 1][:200])
    assert calls >= 50
