"""The integration guide at the repository root shows the `extern "C"` block a maintainer of the reference crate would add.  No Rust toolchain
exists here to compile it, so this test keeps it mechanically in step with the headers: every function it declares
exists in include/*.h with the same number of arguments and matching argument and return types, and every
function of include/wkf_tensor.h (the level the block says it covers) is declared in it."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GUIDE = "INTEGRATION.md"


def _strip_c(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def _c_type(t):
    """A C parameter or return type, without the parameter's name, reduced to (base, pointer depth)."""
    t = t.replace("const", " ").strip()
    depth = t.count("*")
    t = t.replace("*", " ")
    words = t.split()
    base = {"int": "i32", "size_t": "usize", "float": "f32", "uint32_t": "u32", "uint64_t": "u64", "char": "c_char",
            "void": "void", "wkf_device": "WkfDevice", "wkf_tensor": "WkfTensor", "wkf_slice": "WkfSlice"}
    for i, wd in enumerate(words):
        if wd in base:
            return base[wd], depth
    raise AssertionError("unknown C type: " + t)


def _c_functions():
    funcs = {}
    for header in ("wkf_hip.h", "wkf_tensor.h"):
        text = _strip_c(open(os.path.join(ROOT, "include", header)).read())
        for m in re.finditer(r"(?m)^\s*((?:const\s+)?\w+\s*\**)\s*(wkf_\w+)\s*\(([^;{]*?)\)\s*;", text):
            ret, name, params = m.group(1), m.group(2), m.group(3)
            ps = [] if params.strip() in ("", "void") else [p.strip() for p in params.split(",")]
            funcs[name] = (header, ret.strip(), ps)
    return funcs


def _rust_type(t):
    t = t.strip()
    depth = 0
    while True:
        m = re.match(r"\*(?:mut|const)\s+(.*)", t)
        if not m:
            break
        depth += 1
        t = m.group(1).strip()
    t = t.replace("std::os::raw::", "").replace("std::ffi::", "")
    return {"c_void": "void"}.get(t, t), depth


def _rust_functions():
    text = open(os.path.join(ROOT, GUIDE)).read()
    block = text[text.index('extern "C" {'):]
    block = block[:block.index("\n}\n")]
    block = re.sub(r"//[^\n]*", " ", block)
    funcs = {}
    for m in re.finditer(r"pub fn (wkf_\w+)\s*\(([^)]*)\)\s*(?:->\s*([^;]+))?;", block, flags=re.S):
        name, params, ret = m.group(1), m.group(2), m.group(3)
        ps = [p.split(":", 1)[1] for p in params.split(",") if p.strip()]
        funcs[name] = (ret.strip() if ret else None, ps)
    return funcs


def test_extern_block_matches_the_headers():
    c, rust = _c_functions(), _rust_functions()
    assert len(rust) >= 50
    for name, (ret, params) in rust.items():
        assert name in c, f"the integration guide declares {name}, which no header declares"
        header, cret, cparams = c[name]
        assert len(params) == len(cparams), f"{name}: {len(params)} arguments in the integration guide, {len(cparams)} in {header}"
        for i, (rp, cp) in enumerate(zip(params, cparams)):
            cp_type = re.sub(r"\b\w+\s*$", "", cp) if re.search(r"[\s*]\w+\s*$", cp) else cp   # drop the parameter's name
            assert _rust_type(rp) == _c_type(cp_type), f"{name}, argument {i}: `{rp.strip()}` against `{cp}`"
        if cret == "void":
            assert ret is None, f"{name} returns nothing"
        else:
            assert ret is not None and _rust_type(ret) == _c_type(cret), f"{name}: returns `{ret}` against `{cret}`"


def test_extern_block_covers_the_tensor_level():
    c, rust = _c_functions(), _rust_functions()
    missing = sorted(n for n, (header, _, _) in c.items() if header == "wkf_tensor.h" and n not in rust)
    assert not missing, f"include/wkf_tensor.h declares these, the integration guide does not: {missing}"
