"""The reference's known-answer groups (tests/golden/reference_vectors.json, transcribed from
packages/nx/test/backend_contract.ml and test_nx_extended_dtypes.ml), written once over the
backend interface so that the CPU oracle and the HIP backend are put through the very same
cases: every function takes a backend `B` (OracleBackend or raven_amd.nx_backend.Backend) and
raises AssertionError on the first disagreement. Tolerances are the reference's own
(float_close of backend_contract.ml:83-89: equal, or within abs, or within rel of the larger)."""

import json
import math
from pathlib import Path

import numpy as np
import pytest

from helpers import logical
from raven_amd import dtype as dt

GOLD = json.loads((Path(__file__).parent / "golden" / "reference_vectors.json").read_text())


def fl(x):
    return {"inf": math.inf, "-inf": -math.inf, "nan": math.nan}.get(x, x) if isinstance(x, str) else x


def cplx(pairs):
    return np.array([complex(fl(re), fl(im)) for re, im in pairs], dtype=np.complex128)


def float_close(got, want, rel, abs_):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    both_nan = np.isnan(got) & np.isnan(want)
    with np.errstate(invalid="ignore"):
        d = np.abs(got - want)
        ok = both_nan | (got == want) | (d <= abs_) | (d <= rel * np.maximum(np.abs(got), np.abs(want)))
    return ok & ~(np.isnan(got) ^ np.isnan(want))


def assert_close(got, want, rel, abs_, what):
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if np.iscomplexobj(got) or np.iscomplexobj(want):
        ok = float_close(got.real, want.real, rel, abs_) & float_close(got.imag, want.imag, rel, abs_)
    else:
        ok = float_close(got, want, rel, abs_)
    assert ok.all(), f"{what}: got {got.ravel()[~ok.ravel()][:4]}, want {want.ravel()[~ok.ravel()][:4]}"


def T(B, arr, d):
    """A tensor of dtype d holding the storage array `arr` (already in d's storage type)."""
    a = np.ascontiguousarray(arr)
    return B.reshape(B.from_host(a.reshape(-1), d), a.shape)


def from_f32(B, values, d):
    """float32 host values -> dtype d through the backend's own cast."""
    t = T(B, np.asarray(values, dtype=np.float32), dt.float32)
    return t if d is dt.float32 else B.cast(t, d)


def to_f64(B, t):
    if t.dtype in (dt.bfloat16, dt.float8_e4m3, dt.float8_e5m2, dt.float16):
        t = B.cast(t, dt.float32)
    return logical(t).astype(np.float64)


# ── groups already held by the fixture file ─────────────────────────────────
def quantize(B):
    for key, d in (("bf16_quantize", dt.bfloat16), ("f16_quantize", dt.float16)):
        for x, want in GOLD[key]["cases"]:
            got = to_f64(B, from_f32(B, [x], d))[0]
            assert got == want, (key, x, got, want)
    for (m, e), (wm, we) in GOLD["f16_subnormal_exp2"]["cases"]:
        assert to_f64(B, from_f32(B, [math.ldexp(m, e)], dt.float16))[0] == math.ldexp(wm, we)
    for x, want in GOLD["f16_overflow"]["cases"]:
        assert to_f64(B, from_f32(B, [x], dt.float16))[0] == fl(want)
    vals = GOLD["half_exact_roundtrip"]["values"]
    for d in (dt.float16, dt.bfloat16):
        assert to_f64(B, from_f32(B, vals, d)).tolist() == vals


def half_binary(B):
    byname = {"bfloat16": dt.bfloat16, "float16": dt.float16}
    for dn, op, a, b, want in GOLD["half_binary_rounding"]["cases"]:
        d = byname[dn]
        assert to_f64(B, B.binary(op, from_f32(B, [a], d), from_f32(B, [b], d)))[0] == want, (dn, op)
    g = GOLD["half_binary_exact"]
    for d in (dt.float16, dt.bfloat16):
        for op in ("add", "sub", "mul", "fdiv"):
            assert to_f64(B, B.binary(op, from_f32(B, g["a"], d), from_f32(B, g["b"], d))).tolist() == g[op], (d.name, op)


def cast_vectors(B):
    for sname, dname, xs, want in GOLD["cast"]["cases"]:
        s, d = dt.BY_NAME[sname], dt.BY_NAME[dname]
        x = T(B, np.array([fl(v) for v in xs], dtype=s.np_storage), s)
        assert logical(B.cast(x, d)).tolist() == want, (sname, dname)
    for sname, pname, xs in GOLD["cast"]["int4_roundtrip"]:
        s, p = dt.BY_NAME[sname], dt.BY_NAME[pname]
        x = T(B, np.array(xs, dtype=s.np_storage), s)
        packed = B.cast(x, p)
        first = int(np.asarray(B.to_host(packed)).view(np.uint8)[0])
        assert first == ((xs[0] & 0xF) | ((xs[1] & 0xF) << 4))  # low nibble first (nx_c_map.c:1046-1049)
        assert logical(B.cast(packed, s)).tolist() == xs


def zero_division_and_nan_rules(B):
    g = GOLD["int_zero_division"]
    a, z, want = (np.array(v, np.int32) for v in g["idiv"])
    assert logical(B.binary("idiv", T(B, a, dt.int32), T(B, z, dt.int32))).tolist() == want.tolist()
    a, z, want = (np.array(v, np.int32) for v in g["mod"])
    assert logical(B.binary("mod", T(B, a, dt.int32), T(B, z, dt.int32))).tolist() == want.tolist()
    x, want = (np.array(v, np.int32) for v in g["recip"])
    assert logical(B.unary("recip", T(B, x, dt.int32))).tolist() == want.tolist()
    n = GOLD["nan_rules"]
    r = T(B, np.array([fl(v) for v in n["reduce_input"]]), dt.float64)
    assert np.isnan(logical(B.reduce("max", [0], r)))
    assert np.isnan(logical(B.reduce("min", [0], r)))
    a = T(B, np.array([fl(v) for v in n["arg_input"]]), dt.float64)
    assert int(logical(B.argmax(a, 0))) == n["argmax"]
    assert int(logical(B.argmin(a, 0))) == n["argmin"]


def int_extra_and_pow(B, int_dtypes):
    g = GOLD["int_extra"]
    t = T(B, np.array(g["prod_input"], np.int32), dt.int32)
    assert logical(B.reduce("prod", [1], t)).tolist() == g["prod_axis1"]
    t = T(B, np.array(g["arg_input"], np.int32), dt.int32)
    assert logical(B.argmax(t, 1)).tolist() == g["argmax_axis1"]
    assert logical(B.argmin(t, 1)).tolist() == g["argmin_axis1"]
    t = T(B, np.array(g["uint32_argmax_input"], np.uint32), dt.uint32)
    assert int(logical(B.argmax(t, 0))) == g["uint32_argmax"]
    c = GOLD["cumprod_int32"]
    got = logical(B.associative_scan(c["axis"], "prod", T(B, np.array(c["x"], np.int32), dt.int32)))
    assert got.tolist() == c["out"]
    p = GOLD["int_pow"]
    for d in int_dtypes:
        case = p["signed" if d.np_storage.kind == "i" else "unsigned"]
        bases, exps = (np.array(case[k]).astype(d.np_storage) for k in ("bases", "exps"))
        got = logical(B.binary("pow", T(B, bases, d), T(B, exps, d)))
        assert got.tolist() == np.array(case["expected"]).astype(d.np_storage).tolist(), d.name


def sums_of_ones(B, encode_one):
    """A storage-width accumulator sticks (f16 at 2048, bf16 at 256, f32 at 2^24): the sums must not."""
    for dname, n in GOLD["sum_of_ones"]["cases"]:
        d = dt.BY_NAME[dname]
        t = B.full(d, (n,), encode_one(d))
        got = to_f64(B, B.reduce("sum", [0], t))
        assert float(got) == float(n), (dname, n, got)
    g = GOLD["regression"]["f32_sum_of_ones"]
    t = B.full(dt.float32, (g["n"],), encode_one(dt.float32))
    assert_close(to_f64(B, B.reduce("sum", [0], t)), float(g["n"]), g["rel"], 0.0, "2^25 ones")


def threefry(B):
    for c in GOLD["threefry_kat"]["cases"]:
        key, ctr = (T(B, np.array(c[k], np.int32), dt.int32) for k in ("key", "counter"))
        assert logical(B.threefry(key, ctr)).tolist() == c["out"]


# ── complex (backend_contract.ml:2319-2387) ─────────────────────────────────
def complex_group(B):
    g = GOLD["complex"]
    pool = cplx(g["pool"])
    for dname, tol in g["dtypes"]:
        d = dt.BY_NAME[dname]
        st = d.np_storage
        a, b = T(B, pool[0:12].astype(st).reshape(3, 4), d), T(B, pool[4:16].astype(st).reshape(3, 4), d)
        sa, sb = logical(a).astype(np.complex128), logical(b).astype(np.complex128)  # the stored values
        for name, op, ref in (("add", "add", sa + sb), ("sub", "sub", sa - sb), ("mul", "mul", sa * sb), ("div", "fdiv", sa / sb)):
            assert_close(logical(B.binary(op, a, b)), ref, tol, tol, f"{dname} {name}")
        assert_close(logical(B.unary("neg", a)), -sa, tol, tol, f"{dname} neg")
        bt_base = T(B, pool[4:16].astype(st).reshape(4, 3), d)
        bt = B.permute(bt_base, [1, 0])
        assert_close(logical(B.binary("mul", a, bt)), sa * logical(bt_base).astype(np.complex128).T, tol, tol, f"{dname} mul-transposed")
        m = g["matmul"]
        ma = T(B, pool[m["a_from"]:m["a_from"] + m["m"] * m["k"]].astype(st).reshape(m["m"], m["k"]), d)
        mb = T(B, pool[m["b_from"]:m["b_from"] + m["k"] * m["n"]].astype(st).reshape(m["k"], m["n"]), d)
        sma, smb = logical(ma).astype(np.complex128), logical(mb).astype(np.complex128)
        want = np.zeros((m["m"], m["n"]), np.complex128)
        for i in range(m["m"]):
            for j in range(m["n"]):
                for p in range(m["k"]):
                    want[i, j] += sma[i, p] * smb[p, j]
        assert_close(logical(B.matmul(ma, mb)), want, tol, tol, f"{dname} matmul")


# ── bool (backend_contract.ml:2388-2436) ────────────────────────────────────
def bool_group(B):
    g = GOLD["bool"]
    a, b = (T(B, np.array(g[k], np.uint8), dt.bool_) for k in ("a", "b"))
    for name, op in (("and", "and"), ("or", "or"), ("xor", "xor"), ("max", "max"), ("min", "min")):
        assert logical(B.binary(op, a, b)).astype(int).tolist() == g[name], name
    assert logical(B.compare("cmpeq", a, b)).astype(int).tolist() == g["cmpeq"]
    w = g["where"]
    got = B.where(T(B, np.array(w["cond"], np.uint8), dt.bool_), T(B, np.array(w["x"], np.int32), dt.int32),
                  T(B, np.array(w["y"], np.int32), dt.int32))
    assert logical(got).tolist() == w["out"]
    r = g["reduce_min"]
    got = B.reduce("min", [r["axis"]], T(B, np.array(r["x"], np.uint8), dt.bool_))
    assert logical(got).astype(int).tolist() == r["out"]


# ── regression (backend_contract.ml:2437-2700) ──────────────────────────────
def regression_group(B):
    g = GOLD["regression"]
    s = g["nan_sort"]
    x = T(B, np.array([fl(v) for v in s["x"]]), dt.float64)
    for key, desc in (("ascending", False), ("descending", True)):
        assert_close(logical(B.sort(x, 0, desc)), np.array([fl(v) for v in s[key]]), 0.0, 0.0, f"nan sort {key}")
    for key in ("complex_nan_sort", "complex_lexicographic_sort"):
        c = g[key]
        got = logical(B.sort(T(B, cplx(c["x"]).astype(np.complex64), dt.complex64), 0, False))
        assert_close(got, cplx(c["ascending"]), 0.0, 0.0, key)
    c = g["complex_sort_ties_nan"]
    got = logical(B.sort(T(B, cplx(c["x"]).astype(np.complex64), dt.complex64), 0, False)).astype(np.complex128)
    prefix = cplx(c["finite_prefix"])
    assert_close(got[:len(prefix)], prefix, 0.0, 0.0, "complex sort: the finite prefix is lexicographic")
    assert all(np.isnan(z.real) or np.isnan(z.imag) for z in got[len(prefix):]), "complex sort: the suffix is all NaN"
    r = g["complex_rejected"]
    a, b = (T(B, cplx(r[k]).astype(np.complex64), dt.complex64) for k in ("a", "b"))
    with pytest.raises(Exception):
        B.binary("mod", a, b)
    with pytest.raises(Exception):
        B.compare("cmplt", a, b)
    with pytest.raises(Exception):
        B.unary("round", T(B, cplx(r["round_input"]).astype(np.complex64), dt.complex64))
    e = g["empty_axis"]
    for op in ("max", "min"):
        with pytest.raises(ValueError):  # Invalid_argument
            B.reduce(op, [e["axis"]], B.buffer(dt.float64, tuple(e["shape"])))
    for fn in (B.argmax, B.argmin):
        with pytest.raises(ValueError):
            fn(B.buffer(dt.float64, tuple(e["shape"])), e["axis"])
    c = g["complex_abs"]
    z = cplx(c["x"])
    got = logical(B.unary("abs", T(B, z.astype(np.complex64), dt.complex64)))
    assert_close(got, np.hypot(z.real, z.imag) + 0j, c["tol"], c["tol"], "complex abs = |z| + 0i")
    c = g["complex_sign"]
    z = cplx(c["x"])
    m = np.hypot(z.real, z.imag)
    want = np.where(m == 0, 0, z / np.where(m == 0, 1, m))
    got = logical(B.unary("sign", T(B, z.astype(np.complex64), dt.complex64)))
    assert_close(got, want, c["tol"], c["tol"], "complex sign = z / |z|, sign 0 = 0")


# ── high rank (backend_contract.ml:3012-3042) ───────────────────────────────
def highrank_group(B):
    g = GOLD["highrank"]
    nd = g["rank"]
    shape = tuple(2 if i < 2 else 1 for i in range(nd))
    mk = lambda: B.reshape(B.from_host(np.array(g["data"]), dt.float64), shape)  # noqa: E731
    t = mk()
    assert tuple(t.shape) == shape
    assert logical(B.binary("add", t, t)).reshape(-1).tolist() == g["add_self"]
    got = B.reduce("sum", [0], mk())
    assert tuple(got.shape) == shape[1:]
    assert logical(got).reshape(-1).tolist() == g["sum_axis0"]
    axes = [1, 0] + list(range(2, nd))
    p = B.permute(mk(), axes)
    assert tuple(p.shape) == shape
    assert logical(p).reshape(-1).tolist() == g["swap_leading_axes"]
    assert logical(B.contiguous(p)).reshape(-1).tolist() == g["swap_leading_axes"]


# ── fp8 elementwise (backend_contract.ml:3050-3122 over the layouts of :555-592) ──
def fp8_group(B):
    g = GOLD["fp8"]
    pool = np.array(g["pool"], dtype=np.float32)
    for dname, rel, abs_ in g["dtypes"]:
        d = dt.BY_NAME[dname]
        mk = lambda vals, shape: B.reshape(from_f32(B, np.asarray(vals, np.float32).reshape(-1), d), shape)  # noqa: E731
        stored = lambda t: to_f64(B, t)  # noqa: E731
        sub_a, sub_b = (lambda n: pool[0:n]), (lambda n: pool[4:4 + n])
        ca, cb = mk(sub_a(12), (3, 4)), mk(sub_b(12), (3, 4))
        tb43 = mk(sub_b(12), (4, 3))
        ba14 = mk(sub_a(4), (1, 4))
        b36 = mk(pool[0:18], (3, 6))
        r5a, r5b = mk(sub_a(12), (1, 3, 1, 2, 2)), mk(sub_b(12), (1, 3, 1, 2, 2))
        p3a, p3b = mk(sub_a(12), (2, 3, 2)), mk(sub_b(12), (2, 3, 2))
        cases = [
            ("contig,contig", ca, cb),
            ("contig,transpose", ca, B.permute(tb43, [1, 0])),
            ("broadcast,contig", B.expand(ba14, (3, 4)), cb),
            ("flip,slice", B.flip(ca, [False, True]), B.shrink(b36, [(0, 3), (1, 5)])),
            ("scalar,scalar", mk(sub_a(1), ()), mk(sub_b(1), ())),
            ("empty,empty", B.buffer(d, (0, 4)), B.buffer(d, (0, 4))),
            ("rank5,rank5", r5a, r5b),
            ("permute3,permute3", B.permute(p3a, [2, 0, 1]), B.permute(p3b, [2, 0, 1])),
        ]
        for lname, ta, tb in cases:
            la, lb = stored(ta), stored(tb)  # the logical values each operand really holds
            assert_close(stored(B.binary("add", ta, tb)), la + lb, rel, abs_, f"{dname} add {lname}")
            assert_close(stored(B.binary("mul", ta, tb)), la * lb, rel, abs_, f"{dname} mul {lname}")
        for lname, t in (("contig", ca), ("transpose", B.permute(mk(sub_a(12), (4, 3)), [1, 0]))):
            assert_close(stored(B.unary("neg", t)), -stored(t), rel, abs_, f"{dname} neg {lname}")
