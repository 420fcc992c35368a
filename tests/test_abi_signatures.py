"""The ctypes signature table of the Python binding against the declarations in include/et_abi.h:
same number of parameters, and pointer / integer / float / size_t kinds in the same places.  A
pointer bound as a 32-bit int would be truncated on its way into the library."""
import ctypes as C
import importlib.util
import re
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent


def load_table():
    spec = importlib.util.spec_from_file_location("et_binding", ROOT / "scpaper-2021_amd" / "__init__.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod._SIGNATURES


def header_declarations():
    text = "\n".join(h.read_text() for h in sorted((ROOT / "include").glob("*.h")))  # et_abi.h, et_tuning.h
    text = re.sub(r"/\*.*?\*/", " ", text, flags=re.S)
    text = re.sub(r"//[^\n]*", " ", text)
    decls = {}
    for m in re.finditer(r"\b(?:int|const char \*|void)\s*\*?\s*(et_[a-z0-9_]+)\s*\(([^;{]*?)\)\s*;", text, flags=re.S):
        name, params = m.group(1), " ".join(m.group(2).split())
        params = [] if params in ("", "void") else [p.strip() for p in params.split(",")]
        decls[name] = params
    return decls


def kind_of_c(param):
    if "*" in param or re.match(r"(const\s+)?et_(stream|event|graph|model_f32|model|bsr_plan|bsr_pack)\b", param):
        return "ptr"
    if re.match(r"(const\s+)?size_t\b", param):
        return "size"
    if re.match(r"(const\s+)?float\b", param):
        return "float"
    if re.match(r"(const\s+)?(long long|int64_t|uint64_t)\b", param):
        return "i64"
    if re.match(r"(const\s+)?et_f16\b", param):
        return "u16"
    if re.match(r"(const\s+)?(int|int32_t|unsigned|uint32_t)\b", param):
        return "i32"
    return "?" + param


def kind_of_ctypes(t):
    if t in (C.c_void_p, C.c_char_p) or (isinstance(t, type) and issubclass(t, C._Pointer)):
        return "ptr"
    if t is C.c_size_t:
        return "size"
    if t is C.c_float:
        return "float"
    if t in (C.c_longlong, C.c_int64, C.c_uint64, C.c_ulonglong):
        return "i64"
    if t in (C.c_uint16,):
        return "u16"
    if t in (C.c_int, C.c_int32, C.c_uint, C.c_uint32):
        return "i32"
    return "?" + repr(t)


def test_signature_table_matches_header():
    table, decls = load_table(), header_declarations()
    assert len(decls) > 60, "header parse found too few declarations"
    problems = []
    for name, args in table.items():
        if name not in decls:
            problems.append(f"{name}: bound but not declared")
            continue
        want = [kind_of_c(p) for p in decls[name]]
        got = [kind_of_ctypes(t) for t in args]
        # on x86-64 a size_t and a 64-bit integer travel alike
        norm = lambda ks: ["i64" if k == "size" else k for k in ks]
        if norm(want) != norm(got):
            problems.append(f"{name}: header {want} vs binding {got}")
    assert not problems, "\n".join(problems)
