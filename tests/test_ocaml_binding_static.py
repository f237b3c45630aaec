"""The OCaml binding (raven_amd/ocaml) cannot be compiled in this image, so its
three layers are cross-checked as text: every `external` of nx_backend.ml names
a CAMLprim of nx_hip_stubs.c with the same number of arguments, every library
call of the stubs matches its declaration in include/nxhip.h, the module defines
every operation of Backend_intf.S (packages/nx/lib/core/backend_intf.ml), the
dlsym table covers what the stubs call, and every export of the header is
resolved by that table, called by a stub, and reachable from an `external`."""

import re
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
ML = (ROOT / "raven_amd/ocaml/nx_backend.ml").read_text()
STUBS = (ROOT / "raven_amd/ocaml/nx_hip_stubs.c").read_text()
HEADER = (ROOT / "include/nxhip.h").read_text()

# the operations of Backend_intf.S (backend_intf.ml: every `val` of the signature)
S_OPERATIONS = """view dtype context to_host buffer full from_host add sub mul fdiv idiv mod_ pow atan2 cmpeq
cmpne cmplt cmple max min xor or_ and_ neg recip abs sqrt sign exp log sin cos tan asin acos atan sinh cosh tanh
trunc ceil floor round erf where reduce argmax argmin associative_scan sort argsort expand reshape permute shrink
flip pad cat cast contiguous copy assign threefry gather scatter unfold fold matmul fft ifft rfft irfft cholesky
qr svd eigvals eig eigvalsh eigh triangular_solve""".split()


def strip_comments(text, open_, close):
    out, depth, i = [], 0, 0
    while i < len(text):
        if text.startswith(open_, i):
            depth += 1
            i += len(open_)
        elif depth and text.startswith(close, i):
            depth -= 1
            i += len(close)
        else:
            if not depth:
                out.append(text[i])
            i += 1
    return "".join(out)


def top_level_split(text, sep):
    """Pieces of `text` between separators that sit outside every bracket."""
    parts, depth, cur, i = [], 0, [], 0
    while i < len(text):
        ch = text[i]
        if ch in "([{":
            depth += 1
        elif ch in ")]}":
            depth -= 1
        if depth == 0 and text.startswith(sep, i):
            parts.append("".join(cur))
            cur = []
            i += len(sep)
            continue
        cur.append(ch)
        i += 1
    parts.append("".join(cur))
    return parts


def balanced(text, start):
    """The text between the bracket at `start` and its partner."""
    depth = 0
    for i in range(start, len(text)):
        if text[i] == "(":
            depth += 1
        elif text[i] == ")":
            depth -= 1
            if depth == 0:
                return text[start + 1:i]
    raise AssertionError("unbalanced brackets")


def expand_stub_macros(c):
    """UNARY_STUB(name, OP) and its siblings define one CAMLprim each."""
    arity = {"UNARY_STUB": 2, "BINARY_STUB": 3, "COMPARE_STUB": 3}
    prims = {}
    for macro, n in arity.items():
        for name in re.findall(macro + r"\((\w+),\s*NXH_\w+\)", c):
            prims["caml_nx_hip_" + name] = n
    return prims


def c_primitives():
    c = strip_comments(STUBS, "/*", "*/")
    prims = expand_stub_macros(c)
    for m in re.finditer(r"CAMLprim value (caml_nx_hip_\w+)\(", c):
        if "##" in m.group(1):
            continue
        params = balanced(c, m.end() - 1)
        prims[m.group(1)] = "argv" if "argv" in params else len(top_level_split(params, ","))
    return prims


def test_every_external_names_a_primitive_of_the_same_arity():
    ml = strip_comments(ML, "(*", "*)")
    prims = c_primitives()
    externals = re.findall(r"external\s+(\w+)\s*:(.*?)=\s*((?:\"\w+\"\s*)+)", ml, re.S)
    assert len(externals) >= 70
    for name, typ, targets in externals:
        targets = re.findall(r"\"(\w+)\"", targets)
        n_args = len(top_level_split(typ, "->")) - 1
        native = targets[-1]
        assert native in prims, f"{name}: no CAMLprim {native}"
        assert prims[native] == n_args, f"{name}: {n_args} arguments in OCaml, {prims[native]} in C"
        if n_args > 5:  # the bytecode interpreter passes more than five arguments as an array
            assert len(targets) == 2 and prims.get(targets[0]) == "argv", f"{name}: needs a bytecode stub"
        else:
            assert len(targets) == 1


def header_exports():
    """name -> number of parameters, for every function nxhip.h declares."""
    h = strip_comments(HEADER, "/*", "*/")
    h = re.sub(r"//[^\n]*", "", h)
    declared = {}
    for m in re.finditer(r"\b(nxh_\w+)\(", h):
        before = h[:m.start()].rstrip()
        if re.search(r"(int|int64_t|void|\*)\s*$", before):
            declared[m.group(1)] = len(top_level_split(balanced(h, m.end() - 1), ","))
    return declared


def symbol_table(c):
    return set(re.findall(r"X\((\w+)\)", c.split("#define NXH_SYMBOLS(X)")[1].split("static struct")[0]))


def test_library_calls_of_the_stubs_match_the_header():
    declared = header_exports()
    c = strip_comments(STUBS, "/*", "*/")
    table = symbol_table(c)
    calls = list(re.finditer(r"\bL\.(\w+)\(", c))
    assert len(calls) >= 30
    for m in calls:
        fn = m.group(1)
        if fn == "n":  # the table's own macro parameter
            continue
        assert fn in table, f"L.{fn} is not resolved by load_library"
        assert "nxh_" + fn in declared, f"nxh_{fn} is not declared in nxhip.h"
        n = len(top_level_split(balanced(c, m.end() - 1), ","))
        assert n == declared["nxh_" + fn], f"L.{fn}: {n} arguments, nxhip.h declares {declared['nxh_' + fn]}"
    for fn in table:
        assert "nxh_" + fn in declared


def test_the_module_defines_every_operation_of_the_backend_signature():
    ml = strip_comments(ML, "(*", "*)")
    defined = set(re.findall(r"^(?:let|and)\s+(?:rec\s+)?(\w+)", ml, re.M))
    missing = [op for op in S_OPERATIONS if op not in defined]
    assert not missing, f"nx_backend.ml lacks {missing}"
    for op in ("NXH_NEG", "NXH_ERF", "NXH_ADD", "NXH_AND", "NXH_CMPEQ", "NXH_CMPLE"):
        assert op in HEADER and op in STUBS


def test_every_export_of_the_header_is_bound():
    """No entry point of the library is out of the binding's reach: each one is resolved
    at load time, called by at least one stub, and every stub is named by an `external`
    (or is the bytecode twin of one)."""
    declared = header_exports()
    assert len(declared) >= 57
    c = strip_comments(STUBS, "/*", "*/")
    table = symbol_table(c)
    unresolved = sorted(n for n in declared if n[4:] not in table)
    assert not unresolved, f"nx_hip_stubs.c does not resolve {unresolved}"
    called = set(re.findall(r"\bL\.(\w+)\(", c))
    idle = sorted(n for n in table if n not in called)
    assert not idle, f"resolved but never called: {idle}"
    ml = strip_comments(ML, "(*", "*)")
    named = set(re.findall(r"\"(caml_nx_hip_\w+)\"", ml))
    orphans = sorted(p for p in c_primitives() if p not in named)
    assert not orphans, f"CAMLprims that no external names: {orphans}"


def test_the_context_is_destroyed_by_its_last_holder():
    """The context block, every buffer and every graph hold one reference each; the
    finaliser that drops the last one calls nxh_context_destroy."""
    c = strip_comments(STUBS, "/*", "*/")
    assert "custom_finalize_default" not in c
    release = c.split("static void box_release")[1].split("}\n}")[0]
    assert "L.context_destroy" in release
    for fin in ("ctx_finalize", "dev_finalize", "graph_finalize"):
        body = c.split(f"static void {fin}(value v)")[1].split("\n}")[0]
        assert "box_release" in body, fin
    assert c.count("box_retain(Box_val(vctx))") == 2  # buffers and graphs
