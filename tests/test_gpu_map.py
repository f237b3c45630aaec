"""GPU parity of the map family (unary, binary, compare, where, cast, copy,
full) against the CPU oracle, through the C ABI, over the reference's layout
matrix. Integer, bool, compare, where, cast, copy: bit-exact. Float arithmetic
that IEEE fixes (add sub mul div sqrt rounding max min neg abs sign): bit-exact.
Transcendentals: the reference contract's tolerance per dtype
(packages/nx/test/backend_contract.ml:147-189), written in helpers.TOL."""

import numpy as np
import pytest

from helpers import (COMPLEX_DTYPES, FLOAT_DTYPES, INT_DTYPES, TOL, close, decode, encode, layouts,
                     logical, pair, same_bits, same_bits_nan_any)
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu

SHAPE = (5, 33, 70)
EXACT_UNARY = ["neg", "recip", "abs", "sign", "sqrt", "trunc", "ceil", "floor", "round"]
TRANS_UNARY = ["exp", "log", "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "tanh", "erf"]


def float_pool(rng, shape, d, lo=-4.0, hi=4.0, specials=True):
    x = rng.uniform(lo, hi, size=shape)
    if specials:
        flat = x.reshape(-1)
        sp = [0.0, -0.0, np.inf, -np.inf, np.nan, 1.0, -1.0, 0.5, -0.5, 1.5, 2.5, -2.5, 1e-3, 3.999]
        k = min(len(sp), flat.size)
        flat[:k] = sp[:k]
    return x


def int_pool(rng, shape, d):
    info = np.iinfo(d.np_storage)
    x = rng.integers(info.min, info.max, size=shape, endpoint=True, dtype=d.np_storage)
    flat = x.reshape(-1)
    sp = [info.min, info.max, 0, 1, 2, 3, info.max - 1] + ([-1, -2, info.min + 1] if info.min < 0 else [])
    k = min(len(sp), flat.size)
    flat[:k] = [int(v) for v in sp[:k]]
    m = max(0, min(200, flat.size - k))
    flat[k:k + m] = rng.integers(max(info.min, -9), min(info.max, 9), m, endpoint=True)
    return x


@pytest.mark.parametrize("d", FLOAT_DTYPES, ids=lambda d: d.name)
def test_unary_float(hip, oracle, d):
    rng = np.random.default_rng(100 + d.tag)
    for lname, src_shape, build in layouts(SHAPE):
        x = encode(float_pool(rng, src_shape, d), d, oracle)
        h, o = pair(x, d, hip, oracle, build)
        for op in EXACT_UNARY:
            same_bits_nan_any(logical(hip.unary(op, h)), logical(oracle.unary(op, o)), d, oracle, f"{op}/{lname}")
        for op in TRANS_UNARY:
            close(logical(hip.unary(op, h)), logical(oracle.unary(op, o)), d, oracle,
                  TOL[d.name][1], TOL[d.name][1], f"{op}/{lname}")


def test_unary_f32_ulp_report(hip, oracle):
    """States the measured f32 distance to glibc for the config-1 op (sin) and exp/tanh."""
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, 1 << 20).astype(np.float32)
    h, o = pair(x, dt.float32, hip, oracle)
    for op, lim in (("sin", 4), ("exp", 4), ("tanh", 4), ("cos", 4), ("log", 4), ("erf", 8)):
        arg_h, arg_o = (h, o)
        if op == "log":
            ax = np.abs(x) + np.float32(1e-3)
            arg_h, arg_o = pair(ax, dt.float32, hip, oracle)
        g = logical(hip.unary(op, arg_h)).view(np.int32).astype(np.int64)
        w = logical(oracle.unary(op, arg_o)).view(np.int32).astype(np.int64)
        ulp = np.abs(g - w).max()
        assert ulp <= lim, (op, int(ulp))


@pytest.mark.parametrize("d", INT_DTYPES, ids=lambda d: d.name)
def test_unary_int(hip, oracle, d):
    rng = np.random.default_rng(200 + d.tag)
    for lname, src_shape, build in layouts(SHAPE):
        h, o = pair(int_pool(rng, src_shape, d), d, hip, oracle, build)
        for op in ["neg", "recip", "abs", "sign", "trunc", "ceil", "floor", "round"]:
            same_bits(logical(hip.unary(op, h)), logical(oracle.unary(op, o)), f"{op}/{lname}")


def layout_pairs():
    ls = layouts(SHAPE)
    idx = [(0, 0), (0, 1), (1, 0), (1, 1), (2, 4), (3, 5), (4, 0), (5, 2), (1, 2), (0, 4)]
    return [(ls[i], ls[j]) for i, j in idx]


@pytest.mark.parametrize("d", FLOAT_DTYPES, ids=lambda d: d.name)
def test_binary_float(hip, oracle, d):
    rng = np.random.default_rng(300 + d.tag)
    for (na, sa, ba), (nb, sb, bb) in layout_pairs():
        xa = encode(float_pool(rng, sa, d), d, oracle)
        xb = encode(float_pool(rng, sb, d, lo=0.25, hi=3.0), d, oracle)
        ha, oa = pair(xa, d, hip, oracle, ba)
        hb, ob = pair(xb, d, hip, oracle, bb)
        for op in ["add", "sub", "mul", "fdiv", "idiv", "max", "min", "mod"]:
            same_bits_nan_any(logical(hip.binary(op, ha, hb)), logical(oracle.binary(op, oa, ob)), d, oracle, f"{op}/{na}/{nb}")
        # pow / atan2: libm, contract tolerance; positive bases keep pow real
        pa = encode(np.abs(decode(xa, d, oracle)) + 0.25, d, oracle)
        hpa, opa = pair(pa, d, hip, oracle, ba)
        for op, (x_h, x_o) in (("pow", (hpa, opa)), ("atan2", (ha, oa))):
            close(logical(hip.binary(op, x_h, hb)), logical(oracle.binary(op, x_o, ob)), d, oracle,
                  TOL[d.name][1], TOL[d.name][1], f"{op}/{na}/{nb}")


@pytest.mark.parametrize("d", INT_DTYPES + [dt.bool_], ids=lambda d: d.name)
def test_binary_int(hip, oracle, d):
    rng = np.random.default_rng(400 + d.tag)
    ops = (["max", "min", "xor", "or", "and"] if d is dt.bool_ else
           ["add", "sub", "mul", "idiv", "mod", "max", "min", "xor", "or", "and", "pow"])
    for (na, sa, ba), (nb, sb, bb) in layout_pairs():
        if d is dt.bool_:
            xa = rng.integers(0, 2, sa).astype(np.uint8)
            xb = rng.integers(0, 2, sb).astype(np.uint8)
        else:
            xa, xb = int_pool(rng, sa, d), int_pool(rng, sb, d)
        ha, oa = pair(xa, d, hip, oracle, ba)
        hb, ob = pair(xb, d, hip, oracle, bb)
        for op in ops:
            if op == "pow":  # small exponents as well as wild ones
                e = (xb.astype(np.int64) % 9 - (2 if np.iinfo(d.np_storage).min < 0 else 0)).astype(d.np_storage)
                he, oe = pair(e, d, hip, oracle, bb)
                same_bits(logical(hip.binary(op, ha, he)), logical(oracle.binary(op, oa, oe)), f"{op}(small exp)/{na}/{nb}")
            same_bits(logical(hip.binary(op, ha, hb)), logical(oracle.binary(op, oa, ob)), f"{op}/{na}/{nb}")


@pytest.mark.parametrize("d", COMPLEX_DTYPES, ids=lambda d: d.name)
def test_complex_ops(hip, oracle, d):
    rng = np.random.default_rng(450 + d.tag)
    rel = TOL[d.name][1]
    for (na, sa, ba), (nb, sb, bb) in layout_pairs()[:4]:
        xa = (rng.uniform(-2, 2, sa) + 1j * rng.uniform(-2, 2, sa)).astype(d.np_storage)
        xb = (rng.uniform(0.5, 2, sb) + 1j * rng.uniform(-2, 2, sb)).astype(d.np_storage)
        ha, oa = pair(xa, d, hip, oracle, ba)
        hb, ob = pair(xb, d, hip, oracle, bb)
        for op in ["add", "sub"]:
            same_bits(logical(hip.binary(op, ha, hb)), logical(oracle.binary(op, oa, ob)))
        for op in ["mul", "fdiv", "pow"]:
            close(logical(hip.binary(op, ha, hb)), logical(oracle.binary(op, oa, ob)), d, oracle, rel * 10, rel * 10, op)
        same_bits(logical(hip.unary("neg", ha)), logical(oracle.unary("neg", oa)))
        for op in ["recip", "abs", "sign", "sqrt", "exp", "log", "sin", "cos", "tan", "sinh", "cosh", "tanh",
                   "asin", "acos", "atan"]:
            close(logical(hip.unary(op, ha)), logical(oracle.unary(op, oa)), d, oracle, rel * 10, rel * 10, op)
        for op in ["cmpeq", "cmpne"]:
            same_bits(logical(hip.compare(op, ha, ha)), logical(oracle.compare(op, oa, oa)))
    x = np.ones(4, d.np_storage)
    (h,) = pair(x, d, hip, oracle)[:1]
    # no ordered comparison, remainder or rounding on complex: rejected, never identity
    for call in (lambda: hip.binary("mod", h, h), lambda: hip.compare("cmplt", h, h),
                 lambda: hip.unary("round", h), lambda: hip.binary("max", h, h), lambda: hip.unary("erf", h)):
        with pytest.raises(RuntimeError):
            call()


@pytest.mark.parametrize("d", FLOAT_DTYPES + INT_DTYPES + [dt.bool_], ids=lambda d: d.name)
def test_compare_where(hip, oracle, d):
    rng = np.random.default_rng(500 + d.tag)
    for (na, sa, ba), (nb, sb, bb) in layout_pairs():
        if d.is_float:
            xa = encode(np.round(float_pool(rng, sa, d)), d, oracle)  # many equal pairs
            xb = encode(np.round(float_pool(rng, sb, d)), d, oracle)
        elif d is dt.bool_:
            xa, xb = rng.integers(0, 2, sa).astype(np.uint8), rng.integers(0, 2, sb).astype(np.uint8)
        else:
            xa = rng.integers(-3 if d.cls == "sint" else 0, 4, sa).astype(d.np_storage)
            xb = rng.integers(-3 if d.cls == "sint" else 0, 4, sb).astype(d.np_storage)
            xa.reshape(-1)[:2] = [np.iinfo(d.np_storage).max, np.iinfo(d.np_storage).min]
        ha, oa = pair(xa, d, hip, oracle, ba)
        hb, ob = pair(xb, d, hip, oracle, bb)
        for op in ["cmpeq", "cmpne", "cmplt", "cmple"]:
            hm, om = hip.compare(op, ha, hb), oracle.compare(op, oa, ob)
            same_bits(logical(hm), logical(om), f"{op}/{na}/{nb}")
        same_bits(logical(hip.where(hm, ha, hb)), logical(oracle.where(om, oa, ob)))
        # a strided condition as well
        cm = rng.integers(0, 2, sb).astype(np.uint8)
        hc, oc = pair(cm, dt.bool_, hip, oracle, bb)
        same_bits(logical(hip.where(hc, ha, hb)), logical(oracle.where(oc, oa, ob)))


CAST_DTYPES = FLOAT_DTYPES + INT_DTYPES + COMPLEX_DTYPES + [dt.bool_]


def cast_source(rng, d, n, oracle):
    if d.is_float:
        v = np.concatenate([
            rng.uniform(-300, 300, n), rng.standard_normal(n) * 10.0 ** rng.integers(-12, 12, n),
            [np.nan, np.inf, -np.inf, 0.0, -0.0, 0.5, -0.5, 0.9, -0.9, 1.5, 2.5, 127.5, -128.5, 255.5, 256.0,
             32767.5, -32768.5, 65535.5, 65536.0, 2147483647.0, 2147483648.0, -2147483649.0, 4294967295.0,
             4294967296.0, 9.3e18, -9.3e18, 1.9e19, 3e38, -3e38, 1e-45, 6e-8, 65504.0, 65520.0, 448.0, 464.0]])
        x = encode(v, d, oracle)
        if d is dt.float32:  # NaN payloads and subnormals by bit pattern
            bits = np.array([0x7F800001, 0x7FABCDEF, 0xFFC00001, 0x00000001, 0x807FFFFF, 0x33000000,
                             0x33000001, 0x387FC000, 0x477FEFFF, 0x477FF000], dtype=np.uint32)
            x = np.concatenate([x, bits.view(np.float32)])
        return x
    if d.is_complex:
        re = cast_source(rng, dt.float64, n // 2, oracle)
        im = rng.uniform(-5, 5, re.size)
        im[::7] = 0.0
        return (re + 1j * im).astype(d.np_storage)
    if d is dt.bool_:
        return rng.integers(0, 2, n).astype(np.uint8)
    info = np.iinfo(d.np_storage)
    x = rng.integers(info.min, info.max, n, endpoint=True, dtype=d.np_storage)
    x[:6] = [info.min, info.max, 0, 1, info.max - 1, info.min + 1]
    x[6:106] = rng.integers(max(info.min, -300), min(info.max, 300), 100, endpoint=True)
    return x


@pytest.mark.parametrize("src", CAST_DTYPES, ids=lambda d: d.name)
def test_cast_matrix_bit_exact(hip, oracle, src):
    rng = np.random.default_rng(600 + src.tag)
    x = cast_source(rng, src, 3000, oracle)
    h, o = pair(x, src, hip, oracle)
    m = (x.size // 6) * 6
    views = [("contig", lambda B, t: t),
             ("strided", lambda B, t: B.permute(B.reshape(B.shrink(t, [(0, m)]), (m // 6, 6)), (1, 0)))]
    for dst in CAST_DTYPES:
        for vname, build in views:
            hv, ov = build(hip, h), build(oracle, o)
            got, want = logical(hip.cast(hv, dst)), logical(oracle.cast(ov, dst))
            try:
                same_bits(got, want)
            except AssertionError as e:
                raise AssertionError(f"cast {src.name}->{dst.name} ({vname}): {e}") from None


def test_cast_f32_half_exhaustive_band(hip, oracle):
    """f32 -> f16 / bf16 over every rounding decision the reference's own gate
    sweeps (nx_c_map.c:1291-1351): all f16 grid points, the rounding band at
    every exponent from below the smallest subnormal to past overflow, both
    signs, NaN payloads."""
    grid = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float32)
    band = []
    lo = np.arange(0, 0x2000, dtype=np.uint32)
    for e in range(0x60, 0x93):
        for mhi in range(0, 0x800000, 0x100000):
            band.append((np.uint32(e) << 23) | np.uint32(mhi & 0x7FE000) | lo)
    band = np.concatenate(band)
    x = np.concatenate([grid, band.view(np.float32), (band | np.uint32(0x80000000)).view(np.float32)])
    h, o = pair(x, dt.float32, hip, oracle)
    for d in (dt.float16, dt.bfloat16, dt.float8_e4m3, dt.float8_e5m2):
        same_bits(logical(hip.cast(h, d)), logical(oracle.cast(o, d)))


def test_cast_int4(hip, oracle):
    rng = np.random.default_rng(7)
    for src, p in ((dt.int8, dt.int4), (dt.uint8, dt.uint4), (dt.int32, dt.int4), (dt.float32, dt.uint4),
                   (dt.float64, dt.int4)):
        n = 1001
        if src.is_float:
            x = np.concatenate([rng.uniform(-20, 20, n - 6), [np.nan, np.inf, -np.inf, 7.9, -8.9, 15.5]]).astype(src.np_storage)
        else:
            info = np.iinfo(src.np_storage)
            x = rng.integers(max(info.min, -40), min(info.max, 40), n, endpoint=True).astype(src.np_storage)
        h, o = pair(x, src, hip, oracle)
        hp, op_ = hip.cast(h, p), oracle.cast(o, p)

        def nibbles(storage):  # n is odd: the last byte's high nibble is padding, not data
            b = np.array(storage[:(n + 1) // 2], dtype=np.uint8)
            b[-1] &= 0x0F
            return b

        same_bits(nibbles(hip.to_host(hp)), nibbles(op_.storage))
        for back in (dt.int8, dt.int32, dt.float32, dt.int64):
            same_bits(logical(hip.cast(hp, back)), logical(oracle.cast(op_, back)))
        # packed -> packed and whole-buffer copy keep the nibbles
        same_bits(nibbles(hip.to_host(hip.copy(hp))), nibbles(op_.storage))
    with pytest.raises(RuntimeError):  # compute ops reject packed dtypes
        hip.unary("neg", hp)


@pytest.mark.parametrize("d", [dt.uint8, dt.bfloat16, dt.float32, dt.int64, dt.complex128], ids=lambda d: d.name)
def test_copy_assign_contiguous_full(hip, oracle, d):
    rng = np.random.default_rng(700 + d.tag)
    for lname, src_shape, build in layouts(SHAPE):
        x = rng.integers(0, 255, size=src_shape + (d.itemsize,), dtype=np.uint8).view(d.np_storage).reshape(src_shape)
        h, o = pair(x, d, hip, oracle, build)
        same_bits(logical(hip.copy(h)), logical(oracle.copy(o)))
        c = hip.contiguous(h)
        assert c.view.is_c_contiguous() and c.view.offset == 0
        assert (c is h) == (h.view.is_c_contiguous() and h.view.offset == 0)
        # assign through a permuted / flipped / offset destination is visible through the base
        hb, ob = hip.buffer(d, (SHAPE[2], SHAPE[0] + 1, SHAPE[1])), oracle.buffer(d, (SHAPE[2], SHAPE[0] + 1, SHAPE[1]))
        zero = np.zeros(1, d.np_storage)
        hip.assign(hb, hip.expand(hip.reshape(hip.from_host(zero, d), ()), hb.shape))
        for B, base, src in ((hip, hb, h), (oracle, ob, o)):
            dst = B.flip(B.permute(B.shrink(base, [(0, SHAPE[2]), (1, SHAPE[0] + 1), (0, SHAPE[1])]), (1, 2, 0)),
                         (True, False, False))
            B.assign(dst, src)
        same_bits(logical(hb), logical(ob))
    one = encode(np.array([1.5]), d, oracle) if d.is_float else np.array([3], d.np_storage)
    for shape in [(), (1,), (7,), (4099,), (3, 0, 2), (17, 33)]:
        same_bits(logical(hip.full(d, shape, one)), logical(oracle.full(d, shape, one)))
    # full through a strided destination view (fill entry point with any layout)
    import ctypes as C
    base = hip.full(d, (6, 10), np.zeros(1, d.np_storage))
    v = hip.permute(hip.shrink(base, [(1, 5), (2, 9)]), (1, 0))
    desc = v._desc()
    hip._check(hip._lib.nxh_fill(hip._h, C.byref(desc), one.ctypes.data))
    want = np.zeros((6, 10), d.np_storage)
    want[1:5, 2:9] = one[0]
    same_bits(logical(base), want)


def test_contiguous_sizes_and_tails(hip, oracle):
    """Vector body + ragged tail + scalar broadcast operands of the contiguous kernel."""
    rng = np.random.default_rng(8)
    for n in (1, 2, 3, 5, 15, 16, 17, 255, 1024, 4099, 1 << 20, (1 << 20) + 3):
        a = rng.standard_normal(n).astype(np.float32)
        b = rng.standard_normal(n).astype(np.float32)
        ha, oa = pair(a, dt.float32, hip, oracle)
        hb, ob = pair(b, dt.float32, hip, oracle)
        same_bits(logical(hip.binary("add", ha, hb)), logical(oracle.binary("add", oa, ob)))
        s = np.array([0.5], np.float32)
        hs, os_ = pair(s, dt.float32, hip, oracle, lambda B, t: B.expand(B.reshape(t, ()), (n,)))
        same_bits(logical(hip.binary("mul", ha, hs)), logical(oracle.binary("mul", oa, os_)))
        same_bits(logical(hip.binary("sub", hs, ha)), logical(oracle.binary("sub", os_, oa)))
        same_bits(logical(hip.cast(ha, dt.float16)), logical(oracle.cast(oa, dt.float16)))
        # a view that starts one element in: misaligned for 16-byte access
        if n > 4:
            hv, ov = (B.shrink(t, [(1, n)]) for B, t in ((hip, ha), (oracle, oa)))
            same_bits(logical(hip.unary("neg", hv)), logical(oracle.unary("neg", ov)))


def test_kernel_paths_are_the_intended_ones(hip):
    """The planner picks the vector, tiled and generic kernels where designed."""
    a = hip.reshape(hip.from_host(np.zeros(64 * 96 * 80, np.float32), dt.float32), (64, 96, 80))
    hip.binary("add", a, a)
    assert hip.last_path() == "map_contig"
    hip.binary("add", hip.permute(a, (0, 2, 1)), hip.reshape(a, (64, 80, 96)))
    assert hip.last_path() == "map_tiled"
    b = hip.expand(hip.reshape(hip.from_host(np.zeros(96, np.float32), dt.float32), (1, 96, 1)), (64, 96, 80))
    hip.binary("add", a, b)
    assert hip.last_path() == "map_generic_vec"
    hip.unary("neg", hip.flip(a, (False, False, True)))
    assert hip.last_path() == "map_generic"


def test_high_rank_and_empty(hip, oracle):
    rng = np.random.default_rng(9)
    x = rng.standard_normal(2 ** 10).astype(np.float32)
    shape = (2,) * 10
    perm = (9, 0, 8, 1, 7, 2, 6, 3, 5, 4)  # nothing coalesces: rank 10 > one launch's 8 dims
    h, o = pair(x, dt.float32, hip, oracle, lambda B, t: B.permute(B.reshape(t, shape), perm))
    same_bits(logical(hip.unary("neg", h)), logical(oracle.unary("neg", o)))
    r32 = (1,) * 15 + (3,) + (1,) * 15 + (5,)
    h, o = pair(x[:15], dt.float32, hip, oracle, lambda B, t: B.reshape(t, r32))
    assert logical(hip.binary("add", h, h)).shape == r32
    same_bits(logical(hip.binary("add", h, h)), logical(oracle.binary("add", o, o)))
    e = hip.buffer(dt.float32, (3, 0, 2))
    assert logical(hip.unary("exp", e)).shape == (3, 0, 2)
    assert logical(hip.cast(e, dt.int32)).shape == (3, 0, 2)


def test_error_kinds(hip):
    x = hip.from_host(np.ones(4, np.float32), dt.float32)
    with pytest.raises(ValueError, match="output has a broadcast"):
        hip.assign(hip.expand(hip.reshape(hip.buffer(dt.float32, (1,)), (1,)), (4,)), x)
    with pytest.raises(RuntimeError, match="dtype not supported"):
        hip.binary("xor", x, x)
    with pytest.raises(RuntimeError, match="dtype not supported"):
        hip.binary("fdiv", hip.cast(x, dt.int32), hip.cast(x, dt.int32))
    with pytest.raises(RuntimeError, match="dtype not supported"):
        hip.unary("sin", hip.cast(x, dt.int32))
    with pytest.raises(RuntimeError, match="dtype not supported"):
        hip.binary("add", hip.cast(x, dt.bool_), hip.cast(x, dt.bool_))


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_tanh_of_16bit_dtypes_over_every_input(hip, oracle, d):
    """tanh of a bfloat16 / float16 tensor uses a short form of its own (hardware exponential and
    reciprocal) instead of the library's tanhf. All 65536 inputs: NaNs, zeros and their signs and
    the saturation at +-1 are exactly the oracle's; every other result is the oracle's correctly
    rounded one or its neighbour, the neighbour in fewer than 1 % of the inputs."""
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    storage = bits.view(d.np_storage)
    (hx, ox) = pair(storage, d, hip, oracle)
    got = logical(hip.unary("tanh", hx)).view(np.uint16)
    want = logical(oracle.unary("tanh", ox)).view(np.uint16)
    gv, wv = decode(got.view(d.np_storage), d, oracle), decode(want.view(d.np_storage), d, oracle)
    assert np.array_equal(np.isnan(gv), np.isnan(wv))
    finite = ~np.isnan(wv)
    assert np.array_equal(np.signbit(gv[finite]), np.signbit(wv[finite]))
    assert np.array_equal(gv[finite] == 0, wv[finite] == 0)
    assert np.array_equal(np.abs(gv[finite]) == 1, np.abs(wv[finite]) == 1) or np.mean((np.abs(gv[finite]) == 1) != (np.abs(wv[finite]) == 1)) < 1e-3
    step = np.abs(got[finite].astype(np.int32) - want[finite].astype(np.int32))  # same sign: adjacent patterns are adjacent values
    assert step.max() <= 1, int(step.max())
    assert np.mean(step != 0) < 0.01, float(np.mean(step != 0))
