"""The Go binding under bindings/go (uncompiled here: the image has no Go toolchain) names only entry points
that include/mimir_mi355x.h declares, each with the header's parameter list: as many parameters, each of the
kind the C type has (a 32-bit or 64-bit integer, a size, a pointer, a double), and the C return type's."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GO = os.path.join(ROOT, "bindings", "go", "backend", "mi355x")


def _split_top(s):
    out, depth, cur = [], 0, ""
    for ch in s:
        if ch in "([":
            depth += 1
        elif ch in ")]":
            depth -= 1
        if ch == "," and depth == 0:
            out.append(cur.strip()); cur = ""
        else:
            cur += ch
    if cur.strip():
        out.append(cur.strip())
    return out


def _c_kind(t):
    t = t.strip()
    if "*" in t:
        return "ptr"
    base = re.sub(r"\bconst\b", "", t).split()
    base = " ".join(base[:-1]) if len(base) > 1 else base[0]  # drop the parameter's name
    return {"int": "i32", "int32_t": "i32", "int64_t": "i64", "size_t": "size", "double": "f64", "mi355x_status": "u32", "uint32_t": "u32"}[base]


def _header():
    text = open(os.path.join(ROOT, "include", "mimir_mi355x.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    decls = {}
    for m in re.finditer(r"MI355X_API\s+([\w\s\*]+?)\b(mi355x_\w+)\s*\(([^;]*?)\)\s*;", text, flags=re.S):
        ret, name, params = m.group(1).strip(), m.group(2), " ".join(m.group(3).split())
        kinds = [] if params in ("", "void") else [_c_kind(p) for p in _split_top(params)]
        decls[name] = (_c_kind(ret + " x"), kinds)
    return decls


_GO_KINDS = {"int32": {"i32"}, "int64": {"i64"}, "uint64": {"ptr"}, "uintptr": {"ptr", "size"}, "float64": {"f64"}, "string": {"ptr"},
             "unsafe.Pointer": {"ptr"}, "status": {"u32"}, "uint32": {"u32"}}


def _go_params(sig):
    """'dtype int32, w, x, y uint64, m int64' -> ['int32', 'uint64', 'uint64', 'uint64', 'int64']"""
    out, pending = [], 0
    for part in _split_top(" ".join(sig.split())):
        words = part.split()
        if len(words) == 1:
            pending += 1  # a name that shares the type of a later one
        else:
            out += [words[-1]] * (pending + 1)
            pending = 0
    assert pending == 0, sig
    return out


def _go_table():
    src = open(os.path.join(GO, "driver_linux.go")).read()
    src = re.sub(r"//[^\n]*", "", src)
    bound = dict(re.findall(r"\{&(\w+),\s*\"(\w+)\"\}", src))
    sigs = {}
    for m in re.finditer(r"^\s*(mi\w+|hip\w+)\s+func\((.*?)\)\s*([\w\.]*)\s*$", src, flags=re.S | re.M):
        sigs[m.group(1)] = (_go_params(m.group(2)), m.group(3))
    return bound, sigs


def test_every_bound_entry_point_is_declared_with_the_same_parameters():
    decls = _header()
    bound, sigs = _go_table()
    mine = {var: sym for var, sym in bound.items() if sym.startswith("mi355x_")}
    assert len(mine) >= 8
    for var, sym in mine.items():
        assert sym in decls, f"{var} binds {sym}, which the header does not declare"
        assert var in sigs, f"no function variable {var}"
        params, ret = sigs[var]
        want_ret, want = decls[sym]
        assert len(params) == len(want), f"{sym}: {len(params)} Go parameters for {len(want)} in the header"
        for i, (g, c) in enumerate(zip(params, want)):
            kinds = {"ptr"} if g.startswith("*") else _GO_KINDS[g]
            assert c in kinds, f"{sym}: parameter {i} is {g} in Go, {c} in the header"
        ret_kinds = _GO_KINDS[ret]
        assert want_ret in ret_kinds or (want_ret == "size" and ret == "uintptr"), f"{sym}: returns {ret} in Go, {want_ret} in the header"


def test_the_sources_call_only_what_the_table_binds():
    bound, _ = _go_table()
    used = set()
    for name in os.listdir(GO):
        if name.endswith(".go"):
            used |= set(re.findall(r"\b(mi[A-Z]\w+)\(", open(os.path.join(GO, name)).read()))
    assert used and used <= set(bound), used - set(bound)
    # and the library's codes for the dtypes are the header's
    text = open(os.path.join(ROOT, "include", "mimir_mi355x.h")).read()
    src = open(os.path.join(GO, "driver_linux.go")).read()
    for go_name, c_name in (("codeF32", "MI355X_F32"), ("codeI32", "MI355X_I32"), ("codeBF16", "MI355X_BF16"), ("codeF16", "MI355X_F16"),
                            ("codeQ8_0", "MI355X_Q8_0"), ("codeQ4_K", "MI355X_Q4_K"), ("codeQ6_K", "MI355X_Q6_K"), ("codeQ4_0", "MI355X_Q4_0")):
        c = re.search(rf"\b{c_name}\s*=\s*(\w+)", text)
        g = re.search(rf"\b{go_name}\s+int32\s*=\s*(\w+)", src)
        assert c and g and int(c.group(1), 0) == int(g.group(1), 0), (go_name, c_name)
    for go_name, c_name in (("statusShape", "MI355X_ERR_SHAPE"), ("statusDType", "MI355X_ERR_DTYPE"), ("statusIndex", "MI355X_ERR_INDEX"),
                            ("statusInternal", "MI355X_ERR_INTERNAL")):
        c = re.search(rf"\b{c_name}\s*=\s*(\w+)", text)
        g = re.search(rf"\b{go_name}\s+status\s*=\s*(\w+)", src)
        assert c and g and int(c.group(1), 0) == int(g.group(1), 0), (go_name, c_name)


REFERENCE = "/root/reference"


def _go_sources():
    return {name: re.sub(r"//[^\n]*", "", open(os.path.join(GO, name)).read()) for name in os.listdir(GO) if name.endswith(".go")}


def test_every_symbol_of_the_reference_that_the_binding_uses_exists_there_or_is_a_listed_patch():
    """The package cannot be compiled here, so what it takes from github.com/gsoultan/mimir is checked by name:
    every rocm.X, every method called on the embedded rocm backend and every backend.X must be defined in the
    reference's backend/rocm or backend packages, or be one of the additions doc.go asks a maintainer for."""
    import pytest
    if not os.path.isdir(REFERENCE):
        pytest.skip("the reference tree is not here")
    doc = open(os.path.join(GO, "doc.go")).read()
    patches = set(re.findall(r"func \(b \*Backend\) (\w+)\(", doc))
    assert patches == {"DevicePointer", "Stream"}, patches

    def defined(pkg_dir, name, method_of=None):
        for fn in os.listdir(pkg_dir):
            if not fn.endswith(".go") or fn.endswith("_test.go"):
                continue
            text = open(os.path.join(pkg_dir, fn)).read()
            if method_of and re.search(rf"^func \(\w+ \*?{method_of}\) {name}\(", text, flags=re.M):
                return True
            if not method_of and re.search(rf"^(func {name}\(|type {name}\b|var {name}\b|const {name}\b|\t{name}(\s|$))", text, flags=re.M):
                return True
        return False

    rocm_dir, backend_dir = os.path.join(REFERENCE, "backend", "rocm"), os.path.join(REFERENCE, "backend")
    srcs = _go_sources()
    for name, src in srcs.items():
        for sym in set(re.findall(r"\brocm\.(\w+)", src)):
            assert defined(rocm_dir, sym), f"{name}: rocm.{sym} is not in the reference"
        for sym in set(re.findall(r"\b(?:b\.Backend|rb)\.(\w+)\(", src)):
            assert sym in patches or defined(rocm_dir, sym, "Backend"), f"{name}: (*rocm.Backend).{sym} is neither in the reference nor a listed patch"
        for sym in set(re.findall(r"\bbackend\.(\w+)", src)):
            assert defined(backend_dir, sym), f"{name}: backend.{sym} is not in the reference"
    # and the constructor is called the way the reference declares it
    new = re.search(r"^func New\(([^)]*)\)", open(os.path.join(rocm_dir, "rocm_linux.go")).read(), flags=re.M)
    assert new and new.group(1).strip() == ""
    assert re.search(r"rocm\.New\(\)", srcs["mi355x_linux.go"])
