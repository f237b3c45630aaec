"""Pins the CPU oracle before anything is compared against it.

Sources of truth used here, none of which is the oracle's own formula:
the reference tests' known-answer vectors (tests/golden/reference_vectors.json,
each group cites its file:line), the reference's two bit-pattern fixtures,
numpy's independent float16 / IEEE arithmetic, torch's bfloat16 and float8
casts, int64 closed forms with explicit wrap, and brute force.
"""

import json
import math
import struct
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle.nx_oracle import OracleBackend, lib, logical
from raven_amd import dtype as dt

GOLD = json.loads((Path(__file__).parent / "golden" / "reference_vectors.json").read_text())
B = OracleBackend()


def fl(x):
    return {"inf": math.inf, "-inf": -math.inf, "nan": math.nan}.get(x, x) if isinstance(x, str) else x


def T(arr, d):
    a = np.asarray(arr)
    t = B.from_host(a.astype(d.np_storage) if d not in (dt.bfloat16,) else a, d)
    return B.reshape(t, a.shape)


def from_f32(values, d):
    """Host f32 values -> tensor of dtype d through the oracle's own cast."""
    t = T(np.asarray(values, dtype=np.float32), dt.float32)
    return t if d is dt.float32 else B.cast(t, d)


def to_f64(t):
    if t.dtype in (dt.bfloat16, dt.float8_e4m3, dt.float8_e5m2, dt.float16):
        t = B.cast(t, dt.float32)
    return logical(t).astype(np.float64)


# ── converters ──────────────────────────────────────────────────────────────

def test_f16_decode_exhaustive_vs_numpy():
    L = lib()
    bits = np.arange(65536, dtype=np.uint16)
    ref = bits.view(np.float16).astype(np.float32)
    got = np.array([L.nxo_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    finite = ~np.isnan(ref)
    assert np.array_equal(got[finite].view(np.uint32), ref[finite].view(np.uint32))
    # NaN: payload shifted up 13 bits and forced quiet (nx_buffer_stubs.h:155-157)
    nb = bits[~finite].astype(np.uint32)
    want = ((nb & 0x8000) << 16) | 0x7F800000 | ((nb & 0x3FF) << 13) | 0x400000
    assert np.array_equal(got[~finite].view(np.uint32), want)


def _edge_f32_bits(rng, n):
    bits = rng.integers(0, 2**32, size=n, dtype=np.uint64).astype(np.uint32)
    # dense sweep of the half rounding band at several exponents, both signs
    band = []
    for e in range(0x30, 0x4A):
        lo = np.arange(0, 0x2000, dtype=np.uint32)
        for mhi in (0, 0x100000, 0x3FE000, 0x7FE000):
            band.append((np.uint32(e) << 23) | np.uint32(mhi & 0x7FE000) | lo)
    band = np.concatenate(band)
    edges = np.array([0, 0x80000000, 0x33000000, 0x33000001, 0x33800000, 0x38000000,
                      0x387FFFFF, 0x38800000, 0x477FE000, 0x477FEFFF, 0x477FF000, 0x47800000,
                      0x7F7FFFFF, 0xFF7FFFFF, 0x7F800000, 0xFF800000, 0x7F800001, 0x7FABCDEF,
                      0x7FC00000, 0x7FFFFFFF, 0xFF800001, 0xFFABCDEF, 0xFFC00000, 0xFFFFFFFF,
                      0x00000001, 0x007FFFFF, 0x00800000], dtype=np.uint32)
    return np.concatenate([bits, band, band | np.uint32(0x80000000), edges])


def test_f32_to_f16_vs_numpy_bitexact():
    rng = np.random.default_rng(1)
    bits = _edge_f32_bits(rng, 300_000)
    x = bits.view(np.float32)
    got = logical(B.cast(T(x, dt.float32), dt.float16)).view(np.uint16)
    with np.errstate(all="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got, want)


def test_f32_to_bf16_vs_torch_and_nan_rule():
    rng = np.random.default_rng(2)
    bits = _edge_f32_bits(rng, 300_000)
    x = bits.view(np.float32)
    got = logical(B.cast(T(x, dt.float32), dt.bfloat16))
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    nan = np.isnan(x)
    assert np.array_equal(got[~nan], want[~nan])
    # NaN keeps sign + top payload and is quieted (nx_buffer_stubs.h:78-82)
    assert np.array_equal(got[nan], ((bits[nan] >> 16) | 0x40).astype(np.uint16))
    # decode is a pure shift
    back = logical(B.cast(T(got, dt.bfloat16), dt.float32)).view(np.uint32)
    assert np.array_equal(back, got.astype(np.uint32) << 16)


@pytest.mark.parametrize("d,tdt", [(dt.float8_e4m3, torch.float8_e4m3fn),
                                   (dt.float8_e5m2, torch.float8_e5m2)])
def test_fp8_vs_torch(d, tdt):
    allb = np.arange(256, dtype=np.uint8)
    dec = logical(B.cast(T(allb, d), dt.float32))
    want = torch.from_numpy(allb.copy()).view(tdt).to(torch.float32).numpy()
    assert np.array_equal(np.isnan(dec), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(dec[ok].view(np.uint32), want[ok].view(np.uint32))
    rng = np.random.default_rng(3)
    x = np.concatenate([
        rng.standard_normal(200_000).astype(np.float32) * 8,
        rng.uniform(-500, 500, 100_000).astype(np.float32),
        (rng.standard_normal(100_000) * 2.0 ** rng.integers(-20, 18, 100_000)).astype(np.float32),
        dec[ok], np.array([0.0, -0.0, 448.0, 449.0, 464.0, 465.0, 480.0, 57344.0, 61440.0,
                           65536.0, 1e30, -1e30, np.inf, -np.inf], dtype=np.float32)])
    # midpoints between neighbouring representable values exercise ties-to-even
    vals = np.sort(dec[ok & (allb < 128)])
    mids = ((vals[:-1].astype(np.float64) + vals[1:].astype(np.float64)) / 2).astype(np.float32)
    x = np.concatenate([x, mids, -mids])
    enc = logical(B.cast(T(x, dt.float32), d))
    want = torch.from_numpy(x.copy()).to(tdt).view(torch.uint8).numpy()
    fin = np.isfinite(x)
    assert np.array_equal(enc[fin], want[fin])
    # inf: e4m3fn has none -> NaN with the sign kept; e5m2 keeps inf
    # (nx_buffer_stubs.h:190-191, 245-246)
    pinf, ninf = enc[x == np.inf][0], enc[x == -np.inf][0]
    assert (pinf, ninf) == ((0x7F, 0xFF) if d is dt.float8_e4m3 else (0x7C, 0xFC))
    assert logical(B.cast(T(np.array([np.nan], np.float32), dt.float32), d))[0] == 0x7F


def test_reference_bit_fixtures():
    """The reference's .safetensors fixtures decode to 0, min subnormal, 1, inf, NaN."""
    for name, d in (("f16", dt.float16), ("bf16", dt.bfloat16)):
        raw = (Path(__file__).parent / "golden" / f"{name}_bit_exact.safetensors").read_bytes()
        hlen = struct.unpack("<Q", raw[:8])[0]
        meta = json.loads(raw[8:8 + hlen])[f"{name}_tensor"]
        lo, hi = meta["data_offsets"]
        bits = np.frombuffer(raw[8 + hlen + lo:8 + hlen + hi], dtype=np.uint16)
        assert bits.tolist() == GOLD["safetensor_bits"][name]
        v = logical(B.cast(T(bits.view(d.np_storage), d), dt.float32))
        tiny = 2.0 ** -24 if d is dt.float16 else float(np.uint32(0x00010000).view(np.float32))
        assert v[0] == 0.0 and v[1] == np.float32(tiny) and v[2] == 1.0 and v[3] == np.inf
        assert np.isnan(v[4])
        # and the way back reproduces the stored bits
        assert np.array_equal(logical(B.cast(T(v, dt.float32), d)).view(np.uint16), bits)


def test_reference_quantize_vectors():
    for key, d in (("bf16_quantize", dt.bfloat16), ("f16_quantize", dt.float16)):
        for x, want in GOLD[key]["cases"]:
            got = to_f64(from_f32([x], d))[0]
            assert got == want, (key, x, got, want)
    for (m, e), (wm, we) in GOLD["f16_subnormal_exp2"]["cases"]:
        got = to_f64(from_f32([math.ldexp(m, e)], dt.float16))[0]
        assert got == math.ldexp(wm, we)
    for x, want in GOLD["f16_overflow"]["cases"]:
        assert to_f64(from_f32([x], dt.float16))[0] == fl(want)
    vals = GOLD["half_exact_roundtrip"]["values"]
    for d in (dt.float16, dt.bfloat16):
        assert to_f64(from_f32(vals, d)).tolist() == vals


def test_reference_half_binary_vectors():
    byname = {"bfloat16": dt.bfloat16, "float16": dt.float16}
    for dn, op, a, b, want in GOLD["half_binary_rounding"]["cases"]:
        d = byname[dn]
        got = to_f64(B.binary(op, from_f32([a], d), from_f32([b], d)))[0]
        assert got == want
    g = GOLD["half_binary_exact"]
    for d in (dt.float16, dt.bfloat16):
        for op in ("add", "sub", "mul", "fdiv"):
            got = to_f64(B.binary(op, from_f32(g["a"], d), from_f32(g["b"], d)))
            assert got.tolist() == g[op]


def test_reference_cast_vectors():
    byname = dt.BY_NAME
    for sname, dname, xs, want in GOLD["cast"]["cases"]:
        s, d = byname[sname], byname[dname]
        x = T(np.array([fl(v) for v in xs], dtype=s.np_storage), s)
        got = logical(B.cast(x, d))
        assert got.tolist() == want, (sname, dname)
    for sname, pname, xs in GOLD["cast"]["int4_roundtrip"]:
        s, p = byname[sname], byname[pname]
        x = T(np.array(xs, dtype=s.np_storage), s)
        packed = B.cast(x, p)
        # low nibble first (nx_c_map.c:1046-1049)
        assert packed.storage[0] == ((xs[0] & 0xF) | ((xs[1] & 0xF) << 4))
        assert logical(B.cast(packed, s)).tolist() == xs


def test_reference_int_zero_division_and_nan_rules():
    g = GOLD["int_zero_division"]
    a, z, want = (np.array(v, np.int32) for v in g["idiv"])
    assert logical(B.binary("idiv", T(a, dt.int32), T(z, dt.int32))).tolist() == want.tolist()
    a, z, want = (np.array(v, np.int32) for v in g["mod"])
    assert logical(B.binary("mod", T(a, dt.int32), T(z, dt.int32))).tolist() == want.tolist()
    x, want = (np.array(v, np.int32) for v in g["recip"])
    assert logical(B.unary("recip", T(x, dt.int32))).tolist() == want.tolist()
    n = GOLD["nan_rules"]
    r = T(np.array([fl(v) for v in n["reduce_input"]]), dt.float64)
    assert np.isnan(logical(B.reduce("max", [0], r)))
    assert np.isnan(logical(B.reduce("min", [0], r)))
    a = T(np.array([fl(v) for v in n["arg_input"]]), dt.float64)
    assert int(logical(B.argmax(a, 0))) == n["argmax"]
    assert int(logical(B.argmin(a, 0))) == n["argmin"]
    for op in ("max", "min"):
        with pytest.raises(ValueError):
            B.reduce(op, [0], B.buffer(dt.float64, (0, 3)))
    with pytest.raises(ValueError):
        B.argmax(B.buffer(dt.float64, (0, 3)), 0)


INT_DTYPES = [dt.int8, dt.uint8, dt.int16, dt.uint16, dt.int32, dt.uint32, dt.int64, dt.uint64]


def wrap(v, d):
    """Python ints -> values of integer dtype d with two's-complement wrap."""
    bits = d.itemsize * 8
    out = []
    for x in v:
        x &= (1 << bits) - 1
        if d.cls == "sint" and x >= 1 << (bits - 1):
            x -= 1 << bits
        out.append(x)
    return out


def int_pool(d, rng, n=257):
    bits = d.itemsize * 8
    lo, hi = (-(1 << (bits - 1)), (1 << (bits - 1)) - 1) if d.cls == "sint" else (0, (1 << bits) - 1)
    special = [lo, hi, 0, 1, 2, 3, 5, 7, hi - 1, lo + 1] + ([-1, -2, -7] if d.cls == "sint" else [hi // 2 + 1])
    rnd = [int(rng.integers(lo, hi, endpoint=True, dtype=np.int64 if d.cls == "sint" else np.uint64))
           for _ in range(n - len(special))]
    small = [int(rng.integers(max(lo, -20), min(hi, 20), endpoint=True)) for _ in range(64)]
    return special + rnd + small


def tdiv(a, b):
    q = abs(a) // abs(b)
    return q if (a < 0) == (b < 0) else -q


def ipow(b, e):
    if e < 0:
        return 1 if b == 1 else ((-1 if e & 1 else 1) if b == -1 else 0)
    return b ** e if e < 200 else pow(b, e, 1 << 64)


@pytest.mark.parametrize("d", INT_DTYPES, ids=lambda d: d.name)
def test_int_ops_closed_form(d):
    rng = np.random.default_rng(d.tag)
    a = int_pool(d, rng)
    b = list(reversed(int_pool(d, np.random.default_rng(d.tag + 100))))
    n = min(len(a), len(b))
    a, b = a[:n], b[:n]
    ta, tb = T(np.array(a, dtype=d.np_storage), d), T(np.array(b, dtype=d.np_storage), d)
    cases = {
        "add": [x + y for x, y in zip(a, b)],
        "sub": [x - y for x, y in zip(a, b)],
        "mul": [x * y for x, y in zip(a, b)],
        "idiv": [0 if y == 0 else tdiv(x, y) for x, y in zip(a, b)],
        "mod": [0 if y == 0 else x - tdiv(x, y) * y for x, y in zip(a, b)],
        "max": [max(x, y) for x, y in zip(a, b)],
        "min": [min(x, y) for x, y in zip(a, b)],
        "xor": [x ^ y for x, y in zip(a, b)],
        "or": [x | y for x, y in zip(a, b)],
        "and": [x & y for x, y in zip(a, b)],
    }
    for op, want in cases.items():
        got = logical(B.binary(op, ta, tb)).tolist()
        assert got == wrap(want, d), op
    un = {
        "neg": [-x for x in a],
        "abs": [abs(x) for x in a],
        "sign": [(x > 0) - (x < 0) for x in a],
        "recip": [0 if x == 0 else tdiv(1, x) for x in a],
        "trunc": a, "ceil": a, "floor": a, "round": a,
    }
    for op, want in un.items():
        assert logical(B.unary(op, ta)).tolist() == wrap(want, d), op
    for op, f in (("cmpeq", lambda x, y: x == y), ("cmpne", lambda x, y: x != y),
                  ("cmplt", lambda x, y: x < y), ("cmple", lambda x, y: x <= y)):
        assert logical(B.compare(op, ta, tb)).tolist() == [int(f(x, y)) for x, y in zip(a, b)]
    # pow: reference vectors plus wrap at bits-1 / bits
    g = GOLD["int_pow"]["signed" if d.cls == "sint" else "unsigned"]
    bits = d.itemsize * 8
    bases, exps = g["bases"] + [2, 2, 3], g["exps"] + [bits - 1, bits, 41 if bits > 8 else 5]
    got = logical(B.binary("pow", T(np.array(bases, dtype=d.np_storage), d),
                           T(np.array(exps, dtype=d.np_storage), d))).tolist()
    assert got[:len(g["expected"])] == g["expected"]
    assert got == wrap([ipow(x, y) for x, y in zip(bases, exps)], d)
    # sums/prods wrap; argmax is the first extreme in the dtype's own order
    m = np.array(a[:240], dtype=d.np_storage).reshape(12, 20)
    for axes in ([0], [1], [0, 1]):
        s = logical(B.reduce("sum", axes, T(m, d)))
        want = wrap(np.asarray(np.sum(m.astype(object), axis=tuple(axes))).reshape(-1).tolist(), d)
        assert s.reshape(-1).tolist() == want
        p = logical(B.reduce("prod", axes, T(m, d)))
        wantp = wrap(np.asarray(np.prod(m.astype(object), axis=tuple(axes))).reshape(-1).tolist(), d)
        assert p.reshape(-1).tolist() == wantp
    assert logical(B.reduce("max", [1], T(m, d))).tolist() == m.max(axis=1).tolist()
    assert logical(B.reduce("min", [0], T(m, d))).tolist() == m.min(axis=0).tolist()
    assert logical(B.argmax(T(m, d), 1)).tolist() == m.argmax(axis=1).tolist()
    assert logical(B.argmin(T(m, d), 0)).tolist() == m.argmin(axis=0).tolist()


def test_reference_int_extra_vectors():
    g = GOLD["int_extra"]
    t = T(np.array(g["prod_input"], np.int32), dt.int32)
    assert logical(B.reduce("prod", [1], t)).tolist() == g["prod_axis1"]
    t = T(np.array(g["arg_input"], np.int32), dt.int32)
    assert logical(B.argmax(t, 1)).tolist() == g["argmax_axis1"]
    assert logical(B.argmin(t, 1)).tolist() == g["argmin_axis1"]
    t = T(np.array(g["uint32_argmax_input"], np.uint32), dt.uint32)
    assert int(logical(B.argmax(t, 0))) == g["uint32_argmax"]


# ── IEEE-exact float ops: numpy is a bit-exact second implementation ──────

@pytest.mark.parametrize("d", [dt.float32, dt.float64], ids=lambda d: d.name)
def test_float_exact_ops_vs_numpy(d):
    rng = np.random.default_rng(7)
    npd = d.np_storage
    a = np.concatenate([rng.standard_normal(5000) * 10.0 ** rng.integers(-30, 30, 5000),
                        [0.0, -0.0, np.inf, -np.inf, np.nan, 1.5, 2.5, -2.5, 0.5, -0.5]]).astype(npd)
    b = np.concatenate([rng.standard_normal(5000) * 10.0 ** rng.integers(-30, 30, 5000),
                        [1.0, 0.0, 2.0, np.nan, 3.0, -0.0, np.inf, 7.0, -np.inf, 0.0]]).astype(npd)
    ta, tb = T(a, d), T(b, d)
    bits = np.uint32 if d is dt.float32 else np.uint64

    def same(got, want):
        gn, wn = np.isnan(got), np.isnan(want)
        assert np.array_equal(gn, wn)
        assert np.array_equal(got[~gn].view(bits), want[~wn].view(bits))

    with np.errstate(all="ignore"):
        same(logical(B.binary("add", ta, tb)), a + b)
        same(logical(B.binary("sub", ta, tb)), a - b)
        same(logical(B.binary("mul", ta, tb)), a * b)
        same(logical(B.binary("fdiv", ta, tb)), a / b)
        same(logical(B.binary("idiv", ta, tb)), np.trunc(a / b))
        same(logical(B.binary("mod", ta, tb)), np.fmod(a, b))
        same(logical(B.binary("max", ta, tb)), np.maximum(a, b))  # NaN-propagating
        same(logical(B.binary("min", ta, tb)), np.minimum(a, b))
        same(logical(B.unary("neg", ta)), -a)
        same(logical(B.unary("abs", ta)), np.abs(a))
        same(logical(B.unary("sqrt", ta)), np.sqrt(a))
        same(logical(B.unary("recip", ta)), npd.type(1) / a)
        same(logical(B.unary("floor", ta)), np.floor(a))
        same(logical(B.unary("ceil", ta)), np.ceil(a))
        same(logical(B.unary("trunc", ta)), np.trunc(a))
        # round: half away from zero (backend_intf.ml:316-318), not numpy's half-even
        tr = np.trunc(a)
        r = np.where(np.abs(a - tr) >= npd.type(0.5), tr + np.copysign(npd.type(1), a), tr)
        r = np.where(np.isfinite(a), r, a).astype(npd)
        same(logical(B.unary("round", ta)), np.copysign(r, a))
        # sign: (x > 0) - (x < 0) as a float, so sign(-0.0) is +0.0; NaN stays NaN
        sg = np.where(np.isnan(a), a, (a > 0).astype(npd) - (a < 0).astype(npd)).astype(npd)
        same(logical(B.unary("sign", ta)), sg)
        assert np.array_equal(logical(B.compare("cmplt", ta, tb)), (a < b).astype(np.uint8))
        assert np.array_equal(logical(B.compare("cmple", ta, tb)), (a <= b).astype(np.uint8))
        assert np.array_equal(logical(B.compare("cmpeq", ta, tb)), (a == b).astype(np.uint8))
        assert np.array_equal(logical(B.compare("cmpne", ta, tb)), (a != b).astype(np.uint8))


def test_transcendentals_within_contract_tolerance():
    # f32 rel 1e-4 / abs 1e-5 is the reference contract (backend_contract.ml:159-168)
    rng = np.random.default_rng(9)
    x = rng.uniform(-4, 4, 4000).astype(np.float32)
    pos = np.abs(x) + np.float32(0.01)
    unit = (x / 4.001).astype(np.float32)
    table = {"exp": (x, np.exp), "log": (pos, np.log), "sin": (x, np.sin), "cos": (x, np.cos),
             "tan": (unit, np.tan), "asin": (unit, np.arcsin), "acos": (unit, np.arccos),
             "atan": (x, np.arctan), "sinh": (x, np.sinh), "cosh": (x, np.cosh),
             "tanh": (x, np.tanh), "erf": (x, np.vectorize(math.erf))}
    for op, (arg, f) in table.items():
        got = logical(B.unary(op, T(arg, dt.float32))).astype(np.float64)
        want = f(arg.astype(np.float64))
        assert np.allclose(got, want, rtol=1e-4, atol=1e-5), op
    y = rng.uniform(0.1, 3, 4000).astype(np.float32)
    got = logical(B.binary("pow", T(pos, dt.float32), T(y, dt.float32))).astype(np.float64)
    assert np.allclose(got, pos.astype(np.float64) ** y, rtol=1e-4, atol=1e-5)
    got = logical(B.binary("atan2", T(x, dt.float32), T(y, dt.float32))).astype(np.float64)
    assert np.allclose(got, np.arctan2(x.astype(np.float64), y), rtol=1e-4, atol=1e-5)


def test_where_and_cast_matrix_closed_forms():
    rng = np.random.default_rng(11)
    c = rng.integers(0, 2, 1000).astype(np.uint8)
    a, b = rng.integers(-1000, 1000, 1000).astype(np.int32), rng.integers(-1000, 1000, 1000).astype(np.int32)
    got = logical(B.where(T(c, dt.bool_), T(a, dt.int32), T(b, dt.int32)))
    assert np.array_equal(got, np.where(c != 0, a, b))
    # int -> int wraps; float -> int saturates with NaN -> 0; -> bool is != 0
    src = np.array([-129, -128, -1, 0, 1, 127, 128, 255, 256, 65535, 65536, 2**31 - 1, -2**31,
                    2**31, 2**40 + 3, -2**40 - 3], dtype=np.int64)
    for d in INT_DTYPES:
        assert logical(B.cast(T(src, dt.int64), d)).tolist() == wrap(src.tolist(), d)
    f = np.array([np.nan, np.inf, -np.inf, 0.0, -0.0, 0.9, -0.9, 1e3, -1e3, 1e10, -1e10, 1e20,
                  -1e20, 3e38, 127.5, -128.5, 255.9, 65535.5, 4294967295.0, 4294967296.0])
    for d in INT_DTYPES:
        bits = d.itemsize * 8
        lo, hi = (-(1 << (bits - 1)), (1 << (bits - 1)) - 1) if d.cls == "sint" else (0, (1 << bits) - 1)
        want = [0 if math.isnan(v) else (lo if v <= lo else (hi if v >= hi + 1 else int(v))) for v in f]
        assert logical(B.cast(T(f, dt.float64), d)).tolist() == want, d.name
    assert logical(B.cast(T(f, dt.float64), dt.bool_)).tolist() == [int(v != 0) for v in f]
    z = np.array([1 + 2j, 0j, -3.5 + 0j, 0 + 1j], dtype=np.complex64)
    assert logical(B.cast(T(z, dt.complex64), dt.float32)).tolist() == [1.0, 0.0, -3.5, 0.0]
    assert logical(B.cast(T(z, dt.complex64), dt.bool_)).tolist() == [1, 0, 1, 1]
    assert logical(B.cast(T(np.array([1.5, -2.0]), dt.float64), dt.complex128)).tolist() == [1.5 + 0j, -2 + 0j]
    # f64 -> f16 double-rounds through f32 (nx_c_map.c:206-209)
    v = np.array([1.0 + 2.0 ** -11 + 2.0 ** -30, 65519.99999], dtype=np.float64)
    with np.errstate(all="ignore"):
        want = v.astype(np.float32).astype(np.float16)
    assert np.array_equal(logical(B.cast(T(v, dt.float64), dt.float16)).view(np.uint16), want.view(np.uint16))


# ── sums, argmax, matmul, gather ─────────────────────────────────────────

def test_float_sum_invariants():
    for name, n in GOLD["sum_of_ones"]["cases"]:
        d = dt.BY_NAME[name]
        one = from_f32([1.0], d)
        ones = B.full(d, (n,), one.storage)  # contiguous, as the reference test builds it
        assert to_f64(B.reshape(B.reduce("sum", [0], ones), (1,)))[0] == float(n)
    rng = np.random.default_rng(13)
    x = rng.standard_normal((300, 257)).astype(np.float32)
    for axes in ([0], [1], [0, 1]):
        got = logical(B.reduce("sum", axes, T(x, dt.float32))).astype(np.float64)
        want = x.astype(np.float64).sum(axis=tuple(axes))
        k = np.prod([x.shape[a] for a in axes])
        assert np.all(np.abs(got - want) <= k * 1e-5 * np.maximum(1.0, np.abs(want)))
    # permuted view: the streaming and per-output paths agree within tolerance
    xt = B.permute(T(x, dt.float32), (1, 0))
    got = logical(B.reduce("sum", [1], xt)).astype(np.float64)
    assert np.allclose(got, x.astype(np.float64).sum(axis=0), rtol=1e-5, atol=1e-4)
    # empty reduced extent stores the identity
    assert logical(B.reduce("sum", [0], B.buffer(dt.float32, (0, 3)))).tolist() == [0, 0, 0]
    assert logical(B.reduce("prod", [0], B.buffer(dt.float32, (0, 3)))).tolist() == [1, 1, 1]


def brute_arg(x, axis, is_max):
    """First extreme; the first NaN wins (backend_contract.ml:999-1032)."""
    xm = np.moveaxis(x, axis, -1)
    out = np.zeros(xm.shape[:-1], dtype=np.int32)
    for idx in np.ndindex(*xm.shape[:-1]):
        row = xm[idx]
        best, nan_seen = 0, bool(np.isnan(row[0]))
        for k in range(1, len(row)):
            v = row[k]
            if np.isnan(v):
                if not nan_seen:
                    best, nan_seen = k, True
            elif not nan_seen and ((v > row[best]) if is_max else (v < row[best])):
                best = k
        out[idx] = best
    return out


def test_arg_and_minmax_brute_force():
    rng = np.random.default_rng(17)
    x = rng.integers(-5, 5, (9, 14, 6)).astype(np.float32)  # many ties
    x[rng.random(x.shape) < 0.03] = np.nan
    for axis in (0, 1, 2):
        assert np.array_equal(logical(B.argmax(T(x, dt.float32), axis)), brute_arg(x, axis, True))
        assert np.array_equal(logical(B.argmin(T(x, dt.float32), axis)), brute_arg(x, axis, False))
        with np.errstate(all="ignore"):
            got = logical(B.reduce("max", [axis], T(x, dt.float32)))
            want = np.max(x, axis=axis)  # numpy max propagates NaN
            assert np.array_equal(np.isnan(got), np.isnan(want))
            assert np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
    kd = B.argmax(T(x, dt.float32), 1, keepdims=True)
    assert kd.shape == (9, 1, 6)


def test_matmul_vs_f64_and_cancellation():
    rng = np.random.default_rng(19)
    for (m, k, n) in [(5, 7, 3), (33, 70, 41), (64, 300, 50)]:
        a = rng.standard_normal((m, k)).astype(np.float32)
        b = rng.standard_normal((k, n)).astype(np.float32)
        want = a.astype(np.float64) @ b.astype(np.float64)
        for ta, tb in [(T(a, dt.float32), T(b, dt.float32)),
                       (B.permute(T(a.T.copy(), dt.float32), (1, 0)),
                        B.permute(T(b.T.copy(), dt.float32), (1, 0)))]:
            got = logical(B.matmul(ta, tb)).astype(np.float64)
            assert np.allclose(got, want, rtol=1e-3, atol=1e-3)  # matmul_test.ml:831-850
    # batch broadcast: [2,1,m,k] x [3,k,n] -> [2,3,m,n]
    a = rng.standard_normal((2, 1, 4, 6)).astype(np.float32)
    b = rng.standard_normal((3, 6, 5)).astype(np.float32)
    got = logical(B.matmul(T(a, dt.float32), T(b, dt.float32)))
    assert got.shape == (2, 3, 4, 5)
    assert np.allclose(got, a.astype(np.float64) @ b.astype(np.float64), rtol=1e-4, atol=1e-4)
    # integer matmul is exact modulo 2^w
    ai = rng.integers(-2**31, 2**31 - 1, (6, 9)).astype(np.int32)
    bi = rng.integers(-2**31, 2**31 - 1, (9, 4)).astype(np.int32)
    want = (ai.astype(object) @ bi.astype(object)).reshape(-1).tolist()
    assert logical(B.matmul(T(ai, dt.int32), T(bi, dt.int32))).reshape(-1).tolist() == wrap(want, dt.int32)
    # cancellation witness: accumulate in f32, round to storage once
    g = GOLD["matmul_cancel"]
    for d, (m, k, n) in [(dt.float16, (16, 4096, 24)), (dt.bfloat16, (16, 4096, 24)),
                         (dt.float16, (4, 64, 4))]:
        av = np.full((m, k), g["a"], np.float32)
        av[:, k // 2:] *= -1
        A, Bm = from_f32(av, d), from_f32(np.full((k, n), g["b"], np.float32), d)
        got = to_f64(B.matmul(A, Bm))
        assert np.max(np.abs(got)) <= 0.1
    # k == 0 gives zeros
    z = logical(B.matmul(B.buffer(dt.float32, (3, 0)), B.buffer(dt.float32, (0, 2))))
    assert z.tolist() == [[0, 0], [0, 0], [0, 0]]


def test_gather_vectors_and_rules():
    data = T(np.arange(12, dtype=np.float64).reshape(3, 4), dt.float64)
    g = GOLD["gather"]
    for axis, key in ((1, "axis1"), (0, "axis0")):
        idx = T(np.array(g[key]["indices"], np.int32), dt.int32)
        assert logical(B.gather(data, idx, axis)).tolist() == g[key]["expected"]
    # negative index wraps once; out of range raises Failure (nx_c_move.c:342-366)
    idx = T(np.array([[-1, -4, 3, 0]], np.int32), dt.int32)
    assert logical(B.gather(data, B.expand(idx, (1, 4)), 1)).tolist() == [[3.0, 0.0, 3.0, 0.0]]
    for bad in (4, -5):
        with pytest.raises(RuntimeError):
            B.gather(data, T(np.array([[bad]], np.int32), dt.int32), 1)
    # embedding-style row gather with a column-broadcast index
    table = np.arange(50, dtype=np.float32).reshape(10, 5)
    ids = np.array([7, 0, 9, 7], np.int32)
    idx = B.expand(B.reshape(T(ids, dt.int32), (4, 1)), (4, 5))
    assert np.array_equal(logical(B.gather(T(table, dt.float32), idx, 0)), table[ids])


def test_layouts_copy_and_errors():
    rng = np.random.default_rng(23)
    x = rng.standard_normal((4, 5, 6)).astype(np.float32)
    t = T(x, dt.float32)
    views = {
        "permute": (B.permute(t, (2, 0, 1)), np.transpose(x, (2, 0, 1))),
        "flip": (B.flip(t, (True, False, True)), x[::-1, :, ::-1]),
        "shrink": (B.shrink(t, [(1, 3), (0, 5), (2, 6)]), x[1:3, :, 2:6]),
        "expand": (B.expand(B.shrink(t, [(0, 1), (0, 5), (0, 6)]), (3, 5, 6)),
                   np.broadcast_to(x[:1], (3, 5, 6))),
    }
    for name, (v, want) in views.items():
        assert np.array_equal(logical(B.copy(v)), want), name
        assert np.array_equal(logical(B.unary("neg", v)), -want), name
    dst = B.buffer(dt.float32, (6, 4, 5))
    B.assign(B.permute(dst, (1, 2, 0)), t)  # write through a permuted destination
    assert np.array_equal(dst.storage.reshape(6, 4, 5), np.transpose(x, (2, 0, 1)))
    with pytest.raises(ValueError):  # zero-stride output
        B.assign(B.expand(B.buffer(dt.float32, (1,)), (4,)), T(np.ones(4, np.float32), dt.float32))
    with pytest.raises(RuntimeError):  # unsupported pairs are rejected, never identity
        B.binary("mod", T(np.ones(2, np.complex64), dt.complex64), T(np.ones(2, np.complex64), dt.complex64))
    with pytest.raises(RuntimeError):
        B.unary("round", T(np.ones(2, np.complex64), dt.complex64))
    with pytest.raises(RuntimeError):
        B.compare("cmplt", T(np.ones(2, np.complex64), dt.complex64), T(np.ones(2, np.complex64), dt.complex64))


# ── pad, cat, scan, threefry, scatter ────────────────────────────────────────

def _mk(B, a, d):
    a = np.ascontiguousarray(a)
    return B.reshape(B.from_host(a, d), a.shape)


def _threefry_py(k0, k1, c0, c1):
    """Threefry-2x32-20 from its published definition, in Python integers."""
    m = 0xFFFFFFFF
    rots = (13, 15, 26, 6, 17, 29, 16, 24)
    ks = (k0, k1, 0x1BD11BDA ^ k0 ^ k1)
    x0, x1 = (c0 + k0) & m, (c1 + k1) & m
    for r in range(20):
        x0 = (x0 + x1) & m
        x1 = ((x1 << rots[r % 8]) | (x1 >> (32 - rots[r % 8]))) & m
        x1 ^= x0
        if (r + 1) % 4 == 0:
            s = (r + 1) // 4
            x0 = (x0 + ks[s % 3]) & m
            x1 = (x1 + ks[(s + 1) % 3] + s) & m
    return x0, x1


def test_threefry_known_answers_and_independent_port():
    B = OracleBackend()
    for case in GOLD["threefry_kat"]["cases"]:
        k = _mk(B, np.array(case["key"], np.int32), dt.int32)
        c = _mk(B, np.array(case["counter"], np.int32), dt.int32)
        assert logical(B.threefry(k, c)).tolist() == case["out"]
    rng = np.random.default_rng(5)
    key = rng.integers(-2**31, 2**31, (3, 7, 2)).astype(np.int32)
    ctr = rng.integers(-2**31, 2**31, (3, 7, 2)).astype(np.int32)
    want = np.empty_like(key)
    for i in np.ndindex(3, 7):
        a, b = _threefry_py(*(int(v) & 0xFFFFFFFF for v in (*key[i], *ctr[i])))
        want[i] = np.array([a, b], np.uint32).view(np.int32)
    assert np.array_equal(logical(B.threefry(_mk(B, key, dt.int32), _mk(B, ctr, dt.int32))), want)
    # strided operands: the word pair is read along the last axis' own stride
    kt = B.permute(_mk(B, np.ascontiguousarray(key.transpose(2, 0, 1)), dt.int32), (1, 2, 0))
    assert np.array_equal(logical(B.threefry(kt, _mk(B, ctr, dt.int32))), want)
    with pytest.raises(ValueError):
        B.threefry(_mk(B, key[..., :1], dt.int32), _mk(B, ctr[..., :1], dt.int32))


def test_pad_cat_reference_vectors_and_numpy():
    B = OracleBackend()
    g = GOLD["pad_cat"]
    pc = g["pad_constant"]
    got = B.pad(_mk(B, np.array(pc["x"]), dt.float64), pc["padding"], np.array([pc["fill"]]))
    assert logical(got).tolist() == pc["out"]
    c0 = g["cat_axis0"]
    assert logical(B.cat([_mk(B, np.array(c0["a"]), dt.float64), _mk(B, np.array(c0["b"]), dt.float64)], 0)).tolist() == c0["out"]
    c1 = g["cat_axis1_strided"]
    a = B.permute(_mk(B, np.array(c1["a_storage"]), dt.float64), c1["a_permute"])
    assert logical(B.cat([a, _mk(B, np.array(c1["b"]), dt.float64)], 1)).tolist() == c1["out"]
    rng = np.random.default_rng(9)
    x = rng.integers(-100, 100, (3, 4, 5)).astype(np.int16)
    t = B.flip(B.permute(_mk(B, x, dt.int16), (2, 0, 1)), (False, True, False))
    xl = x.transpose(2, 0, 1)[:, ::-1, :]
    padding = [(2, 0), (0, 3), (1, 1)]
    assert np.array_equal(logical(B.pad(t, padding, np.array([7], np.int16))), np.pad(xl, padding, constant_values=7))
    assert np.array_equal(logical(B.pad(t, [(0, 0)] * 3, np.array([7], np.int16))), xl)
    parts = [xl, xl[:, :1, :], np.zeros((5, 0, 4), np.int16), xl[:, 1:, :]]
    tens = [t, B.shrink(t, [(0, 5), (0, 1), (0, 4)]), _mk(B, parts[2], dt.int16), B.shrink(t, [(0, 5), (1, 3), (0, 4)])]
    assert np.array_equal(logical(B.cat(tens, 1)), np.concatenate(parts, 1))
    assert np.array_equal(logical(B.cat(tens, -2)), np.concatenate(parts, 1))


def test_scan_vs_numpy_and_reference_vector():
    B = OracleBackend()
    g = GOLD["cumprod_int32"]
    assert logical(B.associative_scan(g["axis"], "prod", _mk(B, np.array(g["x"], np.int32), dt.int32))).tolist() == g["out"]
    rng = np.random.default_rng(21)
    # integers: exact with wrap-around in the storage width
    x = rng.integers(-120, 120, (4, 9, 6)).astype(np.int8)
    t = B.permute(_mk(B, x, dt.int8), (1, 0, 2))
    xl = x.transpose(1, 0, 2)
    for axis in (0, 1, 2):
        assert np.array_equal(logical(B.associative_scan(axis, "sum", t)), np.cumsum(xl.astype(np.int64), axis).astype(np.int8))
        # |x| <= 120 and at most 9 factors: the int64 running product never overflows, so the
        # reference's modular product is the exact product truncated to 8 bits
        assert np.array_equal(logical(B.associative_scan(axis, "prod", t)),
                              np.cumprod(xl.astype(np.int64), axis).astype(np.int8))
        assert np.array_equal(logical(B.associative_scan(axis, "max", t)), np.maximum.accumulate(xl, axis))
        assert np.array_equal(logical(B.associative_scan(axis, "min", t)), np.minimum.accumulate(xl, axis))
    # floats: f64 is the sequential IEEE sum exactly; NaN sticks from its position on
    y = rng.standard_normal((5, 33))
    y[2, 7] = np.nan
    ty = _mk(B, y, dt.float64)
    assert np.array_equal(logical(B.associative_scan(1, "sum", ty)), np.cumsum(y, 1), equal_nan=True)
    got = logical(B.associative_scan(1, "max", ty))
    assert np.all(np.isnan(got[2, 7:])) and not np.any(np.isnan(got[2, :7]))
    assert np.array_equal(np.delete(got, 2, 0), np.maximum.accumulate(np.delete(y, 2, 0), 1))
    # narrow floats carry the running value in f32 and store rounded copies
    h = (rng.standard_normal(200) * 4).astype(np.float16)
    run, want = np.float32(0), []
    for v in h:
        run = np.float32(run + np.float32(v))
        want.append(np.float16(run))
    assert np.array_equal(logical(B.associative_scan(0, "sum", _mk(B, h, dt.float16))), np.array(want, np.float16))
    with pytest.raises(RuntimeError):
        B.associative_scan(0, "sum", _mk(B, np.array([1, 0], np.uint8), dt.bool_))


def test_scatter_reference_vectors_and_brute_force():
    B = OracleBackend()
    for c in GOLD["scatter"]["cases"]:
        got = B.scatter(c["mode"], False, _mk(B, np.array(c["template"]), dt.float64),
                        _mk(B, np.array(c["indices"], np.int32), dt.int32),
                        _mk(B, np.array(c["updates"]), dt.float64), c["axis"])
        assert logical(got).tolist() == c["out"], c["name"]
    rng = np.random.default_rng(33)
    tmpl = rng.integers(-50, 50, (4, 6, 5)).astype(np.int32)
    for axis in (0, 1, 2):
        ishape = list(tmpl.shape)
        ishape[axis] = 9
        idx = rng.integers(-tmpl.shape[axis], tmpl.shape[axis], ishape).astype(np.int32)  # negatives wrap once
        upd = rng.integers(-50, 50, ishape).astype(np.int32)
        for mode in ("set", "add"):
            want = tmpl.copy()
            for c in np.ndindex(*ishape):  # row-major serial walk
                o = list(c)
                o[axis] = int(idx[c]) % tmpl.shape[axis]
                want[tuple(o)] = upd[c] if mode == "set" else want[tuple(o)] + upd[c]
            got = B.scatter(mode, False, _mk(B, tmpl, dt.int32), _mk(B, idx, dt.int32), _mk(B, upd, dt.int32), axis)
            assert np.array_equal(logical(got), want), (axis, mode)
    bad = np.array([[9]], np.int32)
    with pytest.raises(RuntimeError, match="out of bounds"):
        B.scatter("set", False, _mk(B, np.zeros((1, 4)), dt.float64), _mk(B, bad, dt.int32),
                  _mk(B, np.ones((1, 1)), dt.float64), 1)


def _nanlist(v):
    return np.array([[float(c) for c in e] if isinstance(e, list) else float(e) for e in v])


def _sort_case_arrays(c):
    d = getattr(dt, c["dtype"])
    x, want = _nanlist(c["x"]), _nanlist(c["out"])
    if d.is_complex:
        x, want = (x[:, 0] + 1j * x[:, 1]).astype(np.complex64), (want[:, 0] + 1j * want[:, 1]).astype(np.complex64)
    return d, x, want


def test_sort_reference_vectors_and_numpy():
    B = OracleBackend()
    for c in GOLD["sort"]["cases"]:
        d, x, want = _sort_case_arrays(c)
        got = logical(B.sort(_mk(B, x, d), 0, c["descending"]))
        assert np.array_equal(got, want, equal_nan=True), c["name"]
    t = GOLD["sort"]["complex_ties_nan"]
    x = _nanlist(t["x"])
    got = logical(B.sort(_mk(B, (x[:, 0] + 1j * x[:, 1]).astype(np.complex64), dt.complex64), 0, False))
    pre = _nanlist(t["finite_prefix"])
    assert np.array_equal(got[:len(pre)], (pre[:, 0] + 1j * pre[:, 1]).astype(np.complex64))
    assert np.all(np.isnan(got[len(pre):].real) | np.isnan(got[len(pre):].imag))
    a = GOLD["sort"]["argsort_int32"]
    idx = logical(B.argsort(_mk(B, np.array(a["x"], np.int32), dt.int32), 0, False))
    assert [a["x"][i] for i in idx] == a["gathered"]
    # against numpy on every axis: values, stable indices, both directions,
    # NaNs last both ways, unsigned high bits, bool
    rng = np.random.default_rng(60)
    for d, arr in ((dt.int32, rng.integers(-5, 5, (4, 7, 3)).astype(np.int32)),
                   (dt.uint32, rng.integers(0, 2**32, (4, 7, 3), dtype=np.uint64).astype(np.uint32)),
                   (dt.uint8, rng.integers(0, 4, (4, 7, 3)).astype(np.uint8)),
                   (dt.bool_, rng.integers(0, 2, (4, 7, 3)).astype(np.uint8))):
        for ax in range(3):
            neg = arr.astype(np.int64) * -1
            assert np.array_equal(logical(B.sort(_mk(B, arr, d), ax, False)), np.sort(arr, axis=ax))
            assert np.array_equal(logical(B.sort(_mk(B, arr, d), ax, True)), np.flip(np.sort(arr, axis=ax), ax))
            assert np.array_equal(logical(B.argsort(_mk(B, arr, d), ax, False)), np.argsort(arr, axis=ax, kind="stable"))
            assert np.array_equal(logical(B.argsort(_mk(B, arr, d), ax, True)), np.argsort(neg, axis=ax, kind="stable"))
    f = rng.standard_normal((6, 40)).astype(np.float32)
    f[rng.random(f.shape) < 0.2] = np.nan
    f[0, :5] = [0.0, -0.0, 0.0, np.inf, -np.inf]
    got = logical(B.sort(_mk(B, f, dt.float32), 1, False))
    assert np.array_equal(got, np.sort(f, axis=1), equal_nan=True)  # numpy also puts NaN last
    got = logical(B.sort(_mk(B, f, dt.float32), 1, True))
    for r in range(6):
        fin = f[r][~np.isnan(f[r])]
        assert np.array_equal(got[r][:fin.size], np.sort(fin)[::-1]) and np.all(np.isnan(got[r][fin.size:]))
    ia = logical(B.argsort(_mk(B, f, dt.float32), 1, True))
    for r in range(6):
        key = np.where(np.isnan(f[r]), np.inf, -f[r].astype(np.float64))  # NaN last, descending otherwise
        assert np.array_equal(ia[r], np.argsort(key, kind="stable"))
    with pytest.raises(ValueError):
        B.sort(_mk(B, f, dt.float32), 2, False)


def test_window_reference_vectors_and_brute_force():
    B = OracleBackend()
    W = GOLD["window"]
    for c in W["cases"]:
        got = B.unfold(_mk(B, np.array(c["x"]), dt.float64), c["kernel"], c["stride"], c["dilation"],
                       [tuple(p) for p in c["padding"]])
        assert logical(got).tolist() == c["out"], c["name"]
    c = W["fold_inverts_unfold"]
    x = np.array(c["x"])
    u = B.unfold(_mk(B, x, dt.float64), c["kernel"], c["stride"], [1], [(0, 0)])
    assert np.array_equal(logical(B.fold(u, [x.shape[1]], c["kernel"], c["stride"], [1], [(0, 0)])), x)
    # fold(unfold(x))[i] = coverage[i] * x[i] (backend_contract.ml:1861-1890)
    for leading, length, k, s in W["fold_overlap"]:
        x = ((np.arange(leading * length) % 13) + 1).astype(np.float64).reshape(leading, length)
        u = B.unfold(_mk(B, x, dt.float64), [k], [s], [1], [(0, 0)])
        f = logical(B.fold(u, [length], [k], [s], [1], [(0, 0)]))
        nwin = (length - k) // s + 1
        cover = np.array([sum(1 for w in range(nwin) if w * s <= j < w * s + k) for j in range(length)])
        assert np.array_equal(f, x * cover)
    # two window dims with stride, dilation and asymmetric padding, against a direct numpy im2col
    rng = np.random.default_rng(61)
    x = rng.standard_normal((2, 3, 7, 9))
    ks, st, dl, pd = [3, 2], [2, 1], [1, 2], [(1, 0), (2, 1)]
    u = logical(B.unfold(_mk(B, x, dt.float64), ks, st, dl, pd))
    xp = np.pad(x, ((0, 0), (0, 0), pd[0], pd[1]))
    oh = (xp.shape[2] - (dl[0] * (ks[0] - 1) + 1)) // st[0] + 1
    ow = (xp.shape[3] - (dl[1] * (ks[1] - 1) + 1)) // st[1] + 1
    want = np.zeros((2, 3, ks[0] * ks[1], oh * ow))
    for a in range(ks[0]):
        for b in range(ks[1]):
            for i in range(oh):
                for j in range(ow):
                    want[:, :, a * ks[1] + b, i * ow + j] = xp[:, :, i * st[0] + a * dl[0], j * st[1] + b * dl[1]]
    assert u.shape == want.shape and np.array_equal(u, want)
    # fold is the adjoint of unfold: <unfold(x), y> = <x, fold(y)>, and on integers exactly col2im
    y = rng.integers(-9, 9, want.shape).astype(np.int32)
    f = logical(B.fold(_mk(B, y, dt.int32), [7, 9], ks, st, dl, pd))
    acc = np.zeros(xp.shape, np.int64)
    for a in range(ks[0]):
        for b in range(ks[1]):
            for i in range(oh):
                for j in range(ow):
                    acc[:, :, i * st[0] + a * dl[0], j * st[1] + b * dl[1]] += y[:, :, a * ks[1] + b, i * ow + j]
    assert np.array_equal(f, acc[:, :, pd[0][0]:pd[0][0] + 7, pd[1][0]:pd[1][0] + 9].astype(np.int32))


def _dft(a, inverse=False):
    """The O(n^2) transform straight from the definition, as backend_contract.ml:2831-2844 states it."""
    n = len(a)
    k = np.arange(n)
    ang = (1.0 if inverse else -1.0) * 2.0 * np.pi * ((k[:, None] * k[None, :]) % n) / n
    return (np.cos(ang) + 1j * np.sin(ang)) @ np.asarray(a, np.complex128)


def test_fft_reference_cases_and_the_definition():
    B = OracleBackend()
    F = GOLD["fft"]
    cdata = lambda n: np.array([((i % 5) - 2) + 1j * ((i % 3) - 1) for i in range(n)], np.complex128)
    tol = F["tolerance"]["complex128"]
    near = lambda got, want, t=tol: np.all(np.abs(np.asarray(got) - np.asarray(want)) <= t * (1 + np.abs(want)))
    for n in F["dft_lengths"]:  # powers of two, radix 7, mixed radix, odd prime products, a Bluestein prime
        x = cdata(n)
        assert near(logical(B.fft(_mk(B, x, dt.complex128), [0])), _dft(x)), n
        assert near(logical(B.ifft(_mk(B, x, dt.complex128), [0])), _dft(x, inverse=True)), n
        assert near(logical(B.ifft(B.fft(_mk(B, x, dt.complex128), [0]), [0])), n * x), n
    n = F["complex64_length"]
    got = logical(B.fft(_mk(B, cdata(n).astype(np.complex64), dt.complex64), [0]))
    assert got.dtype == np.complex64 and near(got, _dft(cdata(n)), F["tolerance"]["complex64"])
    # a strided axis: the signal interleaved with filler, then sliced out (backend_contract.ml:2877-2887)
    n = F["strided"]["n"]
    inter = np.empty((n, 2), np.complex128)
    inter[:, 0] = complex(*F["strided"]["filler"])
    inter[:, 1] = cdata(n)
    view = B.shrink(_mk(B, inter, dt.complex128), [(0, n), (1, 2)])
    assert near(logical(B.fft(view, [0]))[:, 0], _dft(cdata(n)))
    rt = F["roundtrip_2d"]
    x = cdata(12).reshape(rt["shape"])
    assert near(logical(B.ifft(B.fft(_mk(B, x, dt.complex128), [0, 1]), [0, 1])), rt["scale"] * x)
    # two axes are the two 1-D definitions composed, first listed axis first
    got = logical(B.fft(_mk(B, x, dt.complex128), [0, 1]))
    want = np.array([_dft(r) for r in np.array([_dft(c) for c in x.T]).T])
    assert near(got, want)
    for key in ("rfft_even", "rfft_odd"):
        x = np.array(F[key]["x"])
        n = F[key]["n"]
        spec = B.rfft(_mk(B, x, dt.float64), dt.complex128, [0])
        assert logical(spec).shape == (n // 2 + 1,) and near(logical(spec), _dft(x)[:n // 2 + 1])
        assert near(logical(B.irfft(spec, dt.float64, [0], [n])), n * x), key
    c = F["irfft_truncates"]
    ones = _mk(B, np.ones(c["bins"], np.complex128), dt.complex128)
    assert near(logical(B.irfft(ones, dt.float64, [0], [c["s"]])), np.array(c["out"], float))
    c = F["irfft_pads"]
    ones = _mk(B, np.ones(c["bins"], np.complex128), dt.complex128)
    want = np.array([a + b * math.sqrt(2.0) for a, b in c["out_sqrt2_form"]])
    assert near(logical(B.irfft(ones, dt.float64, [0], [c["s"]])), want)
    # irfft = real part of the +sign definition on the conjugate-symmetric extension; bins' imaginary
    # parts at 0 and at the Nyquist index contribute nothing
    rng = np.random.default_rng(71)
    for bins, s in ((5, 8), (5, 9), (4, 9), (7, 6)):
        g = rng.standard_normal(bins) + 1j * rng.standard_normal(bins)
        half = min(bins, s // 2 + 1)
        full = np.zeros(s, np.complex128)
        full[:half] = g[:half]
        for k in range(1, half):
            if s - k != k:
                full[s - k] = np.conj(g[k])
        assert near(logical(B.irfft(_mk(B, g, dt.complex128), dt.float64, [0], [s])), _dft(full, inverse=True).real)
    k = F["known"]
    assert near(logical(B.fft(_mk(B, np.ones(4, np.complex128), dt.complex128), [0])), np.array(k["ones4"], complex))
    assert near(logical(B.fft(_mk(B, np.array([1, 0, 0, 0], np.complex128), dt.complex128), [0])), np.array(k["delta4"], complex))
    x = cdata(F["parseval"]["n"])
    e = lambda a: float(np.sum(np.abs(a) ** 2))
    assert abs(e(logical(B.fft(_mk(B, x, dt.complex128), [0]))) - len(x) * e(x)) <= F["parseval"]["rel"] * len(x) * e(x)


def test_linalg_reference_cases():
    """The reference's own linalg cases, checked the way it checks them: residuals
    relative to the matrix norm (backend_contract.ml:2075-2311), exact values where it has them."""
    B = OracleBackend()
    L = GOLD["linalg"]
    tol = L["tolerance"]
    f = lambda a: _mk(B, np.array(a, np.float64), dt.float64)
    rr = lambda ref, x: np.max(np.abs(np.asarray(ref) - np.asarray(x))) / max(1e-30, np.sqrt(np.sum(np.abs(ref) ** 2)))
    Hm = lambda a: np.swapaxes(a, -1, -2).conj()
    m4x3, sq4 = np.array(L["m4x3"], float), np.array(L["sq4"], float)
    spd4 = sq4 @ sq4.T + 4 * np.eye(4)
    low = logical(B.cholesky(f(spd4), False))
    assert np.all(np.triu(low, 1) == 0) and rr(spd4, low @ low.T) <= tol
    up = logical(B.cholesky(f(spd4), True))
    assert np.all(np.tril(up, -1) == 0) and rr(spd4, up.T @ up) <= tol
    for reduced, qs, rs in ((True, (4, 3), (3, 3)), (False, (4, 4), (4, 3))):
        q, r = (logical(t) for t in B.qr(f(m4x3), reduced))
        assert q.shape == qs and r.shape == rs and rr(m4x3, q @ r) <= tol
        assert rr(np.eye(qs[1]), q.T @ q) <= tol and np.all(np.abs(np.tril(r, -1)) <= tol)
    for full, us, vs in ((False, (4, 3), (3, 3)), (True, (4, 4), (3, 3))):
        u, s, vt = (logical(t) for t in B.svd(f(m4x3), full))
        assert u.shape == us and s.shape == (3,) and vt.shape == vs and s.dtype == np.float64
        assert np.all(s >= -tol) and np.all(np.diff(s) <= tol)
        sigma = np.zeros((us[1], 3))
        sigma[:3, :3] = np.diag(s)
        assert rr(m4x3, u @ sigma @ vt) <= tol
    w, v = (logical(t) for t in B.eigh(f(spd4)))
    assert rr(spd4 @ v, v @ np.diag(w)) <= tol and rr(np.eye(4), v.T @ v) <= tol
    assert rr(w, logical(B.eigvalsh(f(spd4)))) <= tol
    tri = np.array(L["tri3"], float)
    x = logical(B.triangular_solve(f(tri), f(L["tri3_rhs"]), False, False, False))
    assert rr(np.array(L["tri3_rhs"], float), tri @ x) <= tol
    c = L["tri3_vector"]
    x = logical(B.triangular_solve(f(tri), f(c["b"]), False, False, False))
    assert x.shape == (3,) and np.max(np.abs(x - c["x"])) <= c["tol"]
    c = L["tri_batched"]
    x = logical(B.triangular_solve(f(c["a"]), f(c["b"]), False, False, False))
    assert x.shape == (2, 2) and np.max(np.abs(x - np.array(c["x"]))) <= c["tol"]
    a = np.array(L["eig3"], float)
    w, v = (logical(t) for t in B.eig(f(a)))
    assert w.dtype == np.complex128 and rr(a @ v, v @ np.diag(w)) <= tol
    assert rr(w, logical(B.eigvals(f(a)))) <= tol
    ab = np.array(L["eigh_batched"], float)
    w, v = (logical(t) for t in B.eigh(f(ab)))
    assert w.shape == (2, 3)
    for i in range(2):
        assert rr(ab[i] @ v[i], v[i] @ np.diag(w[i])) <= tol
    ca = np.array([[complex(*e) for e in row] for row in L["chol_complex"]])
    l = logical(B.cholesky(_mk(B, ca, dt.complex128), False))
    assert rr(ca, l @ Hm(l)) <= tol
    # beyond the reference's cases: every substitution variant against numpy's general solver,
    # the failures, and complex Householder factors
    rng = np.random.default_rng(81)
    A = rng.standard_normal((5, 5)) + 1j * rng.standard_normal((5, 5)) + 6 * np.eye(5)
    Bm = rng.standard_normal((5, 3)) + 1j * rng.standard_normal((5, 3))
    for upper in (False, True):
        for transpose in (False, True):
            for unit in (False, True):
                M = np.triu(A) if upper else np.tril(A)
                if unit:
                    M = M - np.diag(np.diag(M)) + np.eye(5)
                want = np.linalg.solve(Hm(M) if transpose else M, Bm)
                got = logical(B.triangular_solve(_mk(B, A, dt.complex128), _mk(B, Bm, dt.complex128), upper, transpose, unit))
                assert np.max(np.abs(got - want)) <= 1e-12, (upper, transpose, unit)
    with pytest.raises(RuntimeError, match="not positive definite"):
        B.cholesky(f(np.diag([1.0, -1.0])), False)
    with pytest.raises(RuntimeError, match="singular"):
        B.triangular_solve(f(np.diag([1.0, 0.0])), f([1.0, 1.0]), False, False, False)
    for m, n in ((6, 4), (4, 6), (5, 5)):
        a = rng.standard_normal((m, n)) + 1j * rng.standard_normal((m, n))
        q, r = (logical(t) for t in B.qr(_mk(B, a, dt.complex128), True))
        assert rr(a, q @ r) <= 1e-13 and rr(np.eye(q.shape[1]), Hm(q) @ q) <= 1e-13
        k = min(m, n)
        assert np.max(np.abs(np.diagonal(r)[:k - 1].imag)) <= 1e-15  # reflected columns have a real diagonal
