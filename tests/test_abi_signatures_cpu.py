"""CPU-only: one signature per entry point, three places that must agree.

extern "C" functions are linked by name alone: nothing at build time notices when the header declares other
parameters than the source defines, or when the ctypes binding passes other types than the header says.  Here the
prototypes of include/l1attn_hip.h and include/l1attn_cpu.h are parsed and compared, parameter by parameter, with
(1) the definitions in the library sources and (2) the argtypes / restype the Python bindings set."""
import ctypes
import glob
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "l1-attention_amd")


def _strip_comments(text):
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    return re.sub(r"//[^\n]*", " ", text)


def _kind(param):
    """'ptr', 'i64', 'size', 'int', ... of one parameter declaration (its name, const and spacing dropped)."""
    p = re.sub(r"\b(const|restrict|__restrict__)\b", " ", param).strip()
    if "*" in p:
        return "ptr"
    m = re.match(r"((?:unsigned\s+)?[A-Za-z_]\w*)", p)
    base = m.group(1)
    return {"int64_t": "i64", "size_t": "size", "int": "int", "float": "float", "double": "double", "bool": "bool",
            "hipStream_t": "ptr"}.get(base, base)


_PROTO = re.compile(r"\b(int|size_t|void)\s+(l1attn_\w+)\s*\(([^)]*)\)\s*([;{])")


def _prototypes(text, want):
    """name -> (return kind, [parameter kinds]) of every l1attn_* prototype ending in `want` (';' or '{')."""
    out = {}
    for ret, name, params, end in _PROTO.findall(_strip_comments(text)):
        if end != want:
            continue
        ps = [x for x in (y.strip() for y in params.split(",")) if x and x != "void"]
        out[name] = (_kind(ret), [_kind(x) for x in ps])
    return out


def _expand_macros(text):
    """Typed entry points are stamped out by two-parameter macros (a name suffix and an element type): expand
    every use textually so that the definitions read like ordinary functions."""
    text = text.replace("\\\n", " ")
    out = [text]
    for m in re.finditer(r"#define\s+(\w+)\((\w+),\s*(\w+)\)(.*)", text):
        name, sfx, typ, body = m.groups()
        for use in re.finditer(r"^\s*%s\((\w+),\s*([\w ]+)\)" % name, text, flags=re.M):
            out.append(re.sub(r"\b%s\b" % typ, use.group(2), body.replace("##" + sfx, use.group(1))))
    return "\n".join(out)


@pytest.mark.parametrize("header,sources", [
    ("l1attn_hip.h", os.path.join(PKG, "csrc", "*.hip")),
    ("l1attn_cpu.h", os.path.join(PKG, "csrc_cpu", "*.cpp")),
])
def test_definitions_match_the_header(header, sources):
    declared = _prototypes(open(os.path.join(ROOT, "include", header)).read(), ";")
    assert len(declared) >= 19
    defined = {}
    for path in sorted(glob.glob(sources)):
        defined.update(_prototypes(_expand_macros(open(path).read()), "{"))
    for name, sig in declared.items():
        assert name in defined, "declared but not defined: " + name
        assert defined[name] == sig, "%s: header %s, source %s" % (name, sig, defined[name])


_CT = {"ptr": ctypes.c_void_p, "i64": ctypes.c_int64, "size": ctypes.c_size_t, "int": ctypes.c_int}


def _check_binding(L, declared, must_bind):
    bound = 0
    for name, (ret, params) in declared.items():
        f = getattr(L, name)
        if f.argtypes is None:
            if not params:  # nothing to convert
                bound += 1
                continue
            assert name not in must_bind, "called by the Python layer without argtypes: " + name
            continue
        bound += 1
        assert list(f.argtypes) == [_CT[p] for p in params], "%s: header %s, binding %s" % (name, params, f.argtypes)
        if ret == "void":
            assert f.restype is None
        else:
            assert f.restype is _CT[ret], "%s returns %s, binding says %s" % (name, ret, f.restype)
    return bound


def _called(py_files):
    """Names of library functions the Python layer mentions, with the per-type suffix loops expanded."""
    names = set()
    for path in py_files:
        text = open(path).read()
        names.update(re.findall(r"\bl1attn_\w+", text))
    return names


def test_hip_binding_matches_the_header():
    import sys
    sys.path.insert(0, PKG)
    import _l1attn_hip as drv
    if not os.path.exists(drv._LIB_PATH):
        pytest.skip("library not built")
    declared = _prototypes(open(os.path.join(ROOT, "include", "l1attn_hip.h")).read(), ";")
    mentioned = _called([os.path.join(PKG, "_l1attn_hip.py"), os.path.join(ROOT, "bench.py")])
    must = {n for n in declared if n in mentioned}
    # names assembled from a prefix and a type suffix in the binding
    for n in declared:
        if any(n.startswith(p) and p in mentioned for p in ("l1attn_sparse_fwd_", "l1attn_sparse_bwd_", "l1attn_sparse_bidi_fwd_",
                                                            "l1attn_sparse_bidi_bwd_", "l1attn_dense_fwd_", "l1attn_dense_bwd_",
                                                            "l1attn_fused_fwd_", "l1attn_fused_bwd_stage_")):
            must.add(n)
    assert _check_binding(drv.lib(), declared, must) >= 35


def test_cpu_binding_matches_the_header():
    import sys
    sys.path.insert(0, PKG)
    import _l1attn_cpu as cpu
    declared = _prototypes(open(os.path.join(ROOT, "include", "l1attn_cpu.h")).read(), ";")
    assert _check_binding(cpu.lib(), declared, set(declared)) == len(declared) == 19
