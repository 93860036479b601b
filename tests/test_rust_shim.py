"""The Rust binding under rust/ is written, not compiled (the build image has no Rust toolchain), so its agreement with
the C header is checked textually: every declaration of include/tenferro_hip.h appears in the extern block of
tenferro-hip-sys with the same argument count and the same types, the repr(C) structs have the header's fields in the
header's order, the constants have the header's values, check() has an arm for each of the seven statuses, and the safe
crate uses every symbol it binds."""
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tenferro_hip.h")
SYS = os.path.join(ROOT, "rust", "tenferro-hip-sys", "src", "lib.rs")
SAFE_DIR = os.path.join(ROOT, "rust", "tenferro-hip", "src")

BASE = {"int32_t": "i32", "int64_t": "i64", "uint32_t": "u32", "uint64_t": "u64", "size_t": "usize", "double": "f64",
        "char": "c_char", "void": "c_void"}


def strip_c_comments(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.sub(r"//[^\n]*", "", text)


def c_type_to_rust(ctype):
    """'const int64_t* const*' -> '*const *const i64': a qualifier left of a '*' belongs to what that '*' points at."""
    toks = re.findall(r"const|\*|\w+", ctype)
    words = [t for t in toks if t not in ("const", "*")]
    assert len(words) == 1, ctype
    at = toks.index(words[0])
    out = BASE.get(words[0], words[0])
    const = "const" in toks[:at]
    for t in toks[at + 1:]:
        if t == "const":
            const = True
        elif t == "*":
            out = ("*const " if const else "*mut ") + out
            const = False
    return out


def header_text():
    return strip_c_comments(open(HEADER).read())


def header_functions():
    text = re.sub(r"^\s*#.*$", "", header_text(), flags=re.M)
    text = re.sub(r"typedef\s+(enum|struct)\s+\w+\s*\{.*?\}\s*\w+\s*;", "", text, flags=re.S)
    text = re.sub(r"typedef[^;{]*;", "", text)
    text = text.replace('extern "C" {', "").replace("}", "")
    fns = {}
    for decl in text.split(";"):
        decl = " ".join(decl.split())
        if "(" not in decl:
            continue
        m = re.match(r"(.*?)(\w+)\s*\((.*)\)$", decl)
        ret, name, params = m.group(1).strip(), m.group(2), m.group(3).strip()
        args = []
        if params != "void":
            for p in params.split(","):
                args.append(c_type_to_rust(re.match(r"(.*?)(\w+)$", p.strip()).group(1)))
        fns[name] = (None if ret == "void" else c_type_to_rust(ret), args)
    return fns


def rust_extern_functions():
    text = re.sub(r"//[^\n]*", "", open(SYS).read())
    block = re.search(r'extern "C" \{(.*?)\n\}', text, flags=re.S).group(1)
    fns = {}
    for m in re.finditer(r"pub fn (\w+)\s*\((.*?)\)\s*(?:->\s*([^;]+?))?\s*;", block, flags=re.S):
        name, params, ret = m.group(1), " ".join(m.group(2).split()), m.group(3)
        args = [p.split(":", 1)[1].strip() for p in params.split(",") if p.strip()]
        fns[name] = (ret.strip() if ret else None, args)
    return fns


def test_extern_block_matches_the_header_symbol_by_symbol():
    c, r = header_functions(), rust_extern_functions()
    assert len(c) >= 60
    assert set(c) == set(r), (sorted(set(c) - set(r)), sorted(set(r) - set(c)))
    for name in c:
        assert len(c[name][1]) == len(r[name][1]), (name, c[name], r[name])
        assert c[name] == r[name], (name, c[name], r[name])


def test_extern_block_matches_what_the_library_exports():
    import subprocess
    so = os.path.join(ROOT, "tenferro-rs_amd", "libtenferro_hip.so")
    if not os.path.exists(so):
        pytest.skip("library not built")
    out = subprocess.run(["nm", "-D", "--defined-only", so], capture_output=True, text=True, check=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line and line.split()[-1].startswith("tfh_")}
    assert set(rust_extern_functions()) == exported


def c_struct_fields(name):
    body = re.search(r"typedef struct %s \{(.*?)\} %s;" % (name, name), header_text(), flags=re.S).group(1)
    fields = []
    for decl in body.split(";"):
        decl = " ".join(decl.split())
        if not decl:
            continue
        m = re.match(r"(.*?)([\w\s,\[\]]+)$", decl)
        # "int64_t m, n, k" and "int64_t dims[TFH_MAX_RANK]"
        m = re.match(r"((?:const\s+)?\w+\s*\**)\s*(.*)$", decl)
        ctype, names = m.group(1), m.group(2)
        for n in names.split(","):
            n = n.strip()
            arr = re.match(r"(\w+)\[(\w+)\]$", n)
            if arr:
                fields.append((arr.group(1), "[%s; %s]" % (c_type_to_rust(ctype), arr.group(2))))
            else:
                fields.append((n, c_type_to_rust(ctype)))
    return fields


def rust_struct_fields(name):
    text = re.sub(r"//[^\n]*", "", open(SYS).read())
    body = re.search(r"pub struct %s \{(.*?)\}" % name, text, flags=re.S).group(1)
    return [(m.group(1), " ".join(m.group(2).split())) for m in re.finditer(r"pub (\w+):\s*([^,]+),", body)]


@pytest.mark.parametrize("name", ["tfh_error_info", "tfh_view", "tfh_desc", "tfh_compute_device"])
def test_repr_c_structs_have_the_headers_fields_in_order(name):
    c, r = c_struct_fields(name), rust_struct_fields(name)
    assert c == r, (c, r)
    assert re.search(r"#\[repr\(C\)\]\s*(#\[derive\([^\]]*\)\]\s*)?pub struct %s " % name, open(SYS).read())


def test_constants_have_the_headers_values():
    text = header_text()
    want = {}
    for body in re.findall(r"typedef enum \w+ \{(.*?)\}", text, flags=re.S):
        for m in re.finditer(r"(TFH_\w+)\s*=\s*(\d+)", body):
            want[m.group(1)] = int(m.group(2))
    want["TFH_MAX_RANK"] = int(re.search(r"#define TFH_MAX_RANK (\d+)", open(HEADER).read()).group(1))
    want["TFH_VIEW_CONJ"] = int(re.search(r"#define TFH_VIEW_CONJ (\d+)", open(HEADER).read()).group(1))
    m = re.search(r"#define TFH_STATIC_SCRATCH_BYTES \(\(size_t\)(\d+) << (\d+)\)", open(HEADER).read())
    want["TFH_STATIC_SCRATCH_BYTES"] = int(m.group(1)) << int(m.group(2))
    got = {}
    for m in re.finditer(r"pub const (TFH_\w+): \w+ = ([^;]+);", open(SYS).read()):
        got[m.group(1)] = eval(m.group(2), {"__builtins__": {}})   # "64 << 20"
    assert len(want) >= 39
    assert got == want, (sorted(set(want) ^ set(got)), {k: (want[k], got.get(k)) for k in want if got.get(k) != want[k]})


def test_check_maps_each_of_the_seven_statuses_to_its_own_variant():
    # tenferro-device/src/lib.rs:108-159
    src = open(os.path.join(SAFE_DIR, "lib.rs")).read()
    body = src[src.index("pub fn check(status: i32)"):]
    body = body[:body.index("\n}\n")]
    arms = {
        "TFH_ERR_SHAPE_MISMATCH": r"Error::ShapeMismatch\s*\{\s*expected:.*?got:",
        "TFH_ERR_RANK_MISMATCH": r"Error::RankMismatch\s*\{\s*expected:.*?got:",
        "TFH_ERR_DEVICE": r"Error::DeviceError\(",
        "TFH_ERR_NO_COMPATIBLE_DEVICE": r"Error::NoCompatibleComputeDevice\s*\{\s*space:.*?op:",
        "TFH_ERR_CROSS_MEMORY_SPACE": r"Error::CrossMemorySpaceOperation\s*\{\s*left:.*?right:",
        "TFH_ERR_INVALID_ARGUMENT": r"Error::InvalidArgument\(",
        "TFH_ERR_STRIDED": r"Error::Strided\(",
    }
    for status, variant in arms.items():
        assert re.search(r"sys::%s\s*=>\s*%s" % (status, variant), body, flags=re.S), status


def test_the_safe_crate_uses_every_symbol_it_binds_and_implements_the_trait():
    safe = "".join(open(os.path.join(SAFE_DIR, f)).read() for f in sorted(os.listdir(SAFE_DIR)) if f.endswith(".rs"))
    unused = [name for name in rust_extern_functions() if not re.search(r"sys::%s\b" % name, safe)]
    assert unused == [], unused
    backend = open(os.path.join(SAFE_DIR, "backend.rs")).read()
    assert "impl TensorPrims<Standard> for HipBackend" in backend
    for item in ("type Plan<T: ScalarBase> = HipPlan<T>;", "fn plan<T: ScalarBase>(desc: &PrimDescriptor, shapes: &[&[usize]])",
                 "fn execute<T: ScalarBase>(", "fn has_extension_for<T: ScalarBase>(ext: Extension) -> bool"):
        assert item in backend, item
    for variant in ("BatchedGemm", "Reduce", "Trace", "Permute", "AntiTrace", "AntiDiag", "Contract", "ElementwiseMul"):
        assert "PrimDescriptor::" + variant in backend, variant
    buffer = open(os.path.join(SAFE_DIR, "buffer.rs")).read()
    assert "impl<T> Drop for HipBuffer<T>" in buffer and "sys::tfh_free" in buffer
    assert "impl<T> Drop for HipPlan<T>" in backend and "sys::tfh_plan_destroy" in backend
    event = open(os.path.join(SAFE_DIR, "event.rs")).read()
    assert "pub struct CompletionEvent" in event and "impl Drop for CompletionEvent" in event
