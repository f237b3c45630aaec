"""GPU parity of reductions and argmax/argmin against the CPU oracle.

Integer sums/products/extremes and every arg result are bit-exact. Float
max/min are bit-exact (NaN anywhere -> NaN). Float sums and products are
reassociated on the GPU, so they are compared with the reference contract's
rule |err| <= k * a_rel * scale (packages/nx/test/backend_contract.ml:908-913)
against the oracle, and against exact invariants (sums of ones,
backend_contract.ml:2611-2644)."""

import numpy as np
import pytest

from helpers import FLOAT_DTYPES, INT_DTYPES, TOL, close, decode, encode, logical, pair, same_bits
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu

# (source shape, view builder, logical rank)
def fold_layouts():
    return [
        ("contig", (6, 40, 70), lambda B, t: t),
        ("transposed", (6, 70, 40), lambda B, t: B.permute(t, (0, 2, 1))),
        ("sliced", (8, 41, 73), lambda B, t: B.shrink(t, [(1, 7), (0, 40), (3, 73)])),
        ("flipped", (6, 40, 70), lambda B, t: B.flip(t, (True, False, True))),
        ("broadcast", (6, 1, 70), lambda B, t: B.expand(t, (6, 40, 70))),
    ]

AXES = [[0], [1], [2], [0, 1], [1, 2], [0, 2], [0, 1, 2], []]


def check_float_reduce(hip, oracle, d, h, o, what):
    arith = TOL[d.name][0]
    for axes in AXES:
        k = int(np.prod([h.shape[a] for a in axes])) if axes else 1
        g, w = logical(hip.reduce("sum", axes, h)), logical(oracle.reduce("sum", axes, o))
        vals = np.abs(decode(logical(oracle.copy(o)), d, oracle))
        scale = float(np.nanmax(np.where(np.isfinite(vals), vals, 0))) * k
        close(g, w, d, oracle, arith, arith * max(scale, 1.0), f"sum {axes} {what}")
        for op in ("max", "min"):
            g, w = logical(hip.reduce(op, axes, h)), logical(oracle.reduce(op, axes, o))
            gv, wv = decode(g, d, oracle), decode(w, d, oracle)
            assert np.array_equal(np.isnan(gv), np.isnan(wv)), (op, axes, what)
            assert np.array_equal(gv[~np.isnan(gv)], wv[~np.isnan(wv)]), (op, axes, what)


@pytest.mark.parametrize("d", FLOAT_DTYPES, ids=lambda d: d.name)
def test_reduce_float(hip, oracle, d):
    rng = np.random.default_rng(800 + d.tag)
    for lname, shape, build in fold_layouts():
        x = rng.uniform(-2, 2, shape)
        x.reshape(-1)[rng.integers(0, x.size, 5)] = np.nan
        h, o = pair(encode(x, d, oracle), d, hip, oracle, build)
        check_float_reduce(hip, oracle, d, h, o, lname)
    # products stay near 1 so they neither overflow nor vanish
    x = encode(rng.uniform(0.9, 1.1, (6, 40, 70)), d, oracle)
    h, o = pair(x, d, hip, oracle)
    for axes in ([0], [2], [1, 2]):
        k = int(np.prod([h.shape[a] for a in axes]))
        close(logical(hip.reduce("prod", axes, h)), logical(oracle.reduce("prod", axes, o)), d, oracle,
              TOL[d.name][0] * k, TOL[d.name][0], f"prod {axes}")


@pytest.mark.parametrize("d", INT_DTYPES + [dt.bool_], ids=lambda d: d.name)
def test_reduce_int_exact(hip, oracle, d):
    rng = np.random.default_rng(900 + d.tag)
    for lname, shape, build in fold_layouts():
        if d is dt.bool_:
            x = (rng.random(shape) < 0.97).astype(np.uint8)
        else:
            info = np.iinfo(d.np_storage)
            x = rng.integers(info.min, info.max, shape, endpoint=True, dtype=d.np_storage)
        h, o = pair(x, d, hip, oracle, build)
        for axes in AXES:
            for op in (["max", "min"] if d is dt.bool_ else ["sum", "prod", "max", "min"]):
                same_bits(logical(hip.reduce(op, axes, h)), logical(oracle.reduce(op, axes, o)))
    if d is dt.bool_:
        with pytest.raises(RuntimeError):
            hip.reduce("sum", [0], h)


@pytest.mark.parametrize("d", [dt.complex64, dt.complex128], ids=lambda d: d.name)
def test_reduce_complex(hip, oracle, d):
    rng = np.random.default_rng(950)
    x = (rng.uniform(-1, 1, (6, 40, 70)) + 1j * rng.uniform(-1, 1, (6, 40, 70))).astype(d.np_storage)
    h, o = pair(x, d, hip, oracle)
    for axes in ([0], [2], [0, 1, 2]):
        k = int(np.prod([h.shape[a] for a in axes]))
        close(logical(hip.reduce("sum", axes, h)), logical(oracle.reduce("sum", axes, o)), d, oracle,
              TOL[d.name][0], TOL[d.name][0] * k, "csum")
    with pytest.raises(RuntimeError):
        hip.reduce("max", [0], h)


@pytest.mark.parametrize("d", FLOAT_DTYPES + INT_DTYPES + [dt.bool_], ids=lambda d: d.name)
def test_argreduce_exact(hip, oracle, d):
    rng = np.random.default_rng(1000 + d.tag)
    for lname, shape, build in fold_layouts():
        if d.is_float:
            x = np.round(rng.uniform(-3, 3, shape))  # many ties
            x.reshape(-1)[rng.integers(0, x.size, 40)] = np.nan
            x = encode(x, d, oracle)
        elif d is dt.bool_:
            x = rng.integers(0, 2, shape).astype(np.uint8)
        else:
            info = np.iinfo(d.np_storage)
            x = rng.integers(max(info.min, -4), min(info.max, 4), shape, endpoint=True).astype(d.np_storage)
            x.reshape(-1)[:2] = [info.max, info.min]
        h, o = pair(x, d, hip, oracle, build)
        for axis in (0, 1, 2):
            for keep in (False, True):
                for f in ("argmax", "argmin"):
                    g = getattr(hip, f)(h, axis, keep)
                    w = getattr(oracle, f)(o, axis, keep)
                    assert g.shape == w.shape
                    same_bits(logical(g), logical(w))


def test_long_rows_columns_and_full_reductions(hip, oracle):
    """Shapes that take the split (two-pass) row and column paths."""
    rng = np.random.default_rng(11)
    x = rng.standard_normal((3, 200_000)).astype(np.float32)
    x[1, 150_000] = np.nan
    h, o = pair(x, dt.float32, hip, oracle)
    close(logical(hip.reduce("sum", [1], h)), logical(oracle.reduce("sum", [1], o)), dt.float32, oracle, 1e-5, 2.0)
    assert hip.last_path() == "fold_row_split"
    g, w = logical(hip.reduce("max", [1], h)), logical(oracle.reduce("max", [1], o))
    assert np.array_equal(np.isnan(g), np.isnan(w)) and np.array_equal(g[~np.isnan(g)], w[~np.isnan(w)])
    same_bits(logical(hip.argmax(h, 1)), logical(oracle.argmax(o, 1)))
    assert hip.last_path() == "arg_row_split"
    same_bits(logical(hip.argmin(h, 1)), logical(oracle.argmin(o, 1)))
    y = rng.integers(-1000, 1000, (5000, 300)).astype(np.int32)
    h, o = pair(y, dt.int32, hip, oracle)
    same_bits(logical(hip.reduce("sum", [0], h)), logical(oracle.reduce("sum", [0], o)))
    assert hip.last_path() == "fold_col_split"
    same_bits(logical(hip.argmax(h, 0)), logical(oracle.argmax(o, 0)))
    assert hip.last_path() == "arg_col_split"
    same_bits(logical(hip.reduce("sum", [0, 1], h)), logical(oracle.reduce("sum", [0, 1], o)))
    # column form on floats: NaNs (first one wins), whole columns of -inf / +inf / NaN, a NaN in the
    # last row, ties with the worst value: the three-instruction inner loop and the full rule behind it
    f = np.round(rng.uniform(-5, 5, (5000, 300))).astype(np.float32)
    f[4000, 3] = np.nan
    f[17, 3] = np.nan
    f[:, 7] = -np.inf
    f[:, 8] = np.inf
    f[:, 9] = np.nan
    f[4999, 10] = np.nan
    f[0, 11] = -np.inf
    f[2500:, 12] = -np.inf
    f[1234, 13] = np.inf
    for d in (dt.float32, dt.float64, dt.bfloat16):
        h, o = pair(encode(f, d, oracle), d, hip, oracle)
        for fn in ("argmax", "argmin"):
            same_bits(logical(getattr(hip, fn)(h, 0)), logical(getattr(oracle, fn)(o, 0)), f"{fn} {d.name}")
            assert hip.last_path() == "arg_col_split"
    u = rng.integers(0, 3, (5000, 300)).astype(np.uint8)
    u[:, 5] = 0
    u[:, 6] = 255
    h, o = pair(u, dt.uint8, hip, oracle)
    for fn in ("argmax", "argmin"):
        same_bits(logical(getattr(hip, fn)(h, 0)), logical(getattr(oracle, fn)(o, 0)), fn)
    z = np.round(rng.uniform(-5, 5, (4097, 513))).astype(np.float32)  # ties across chunk boundaries
    h, o = pair(z, dt.float32, hip, oracle)
    for axis in (0, 1):
        same_bits(logical(hip.argmax(h, axis)), logical(oracle.argmax(o, axis)))
        same_bits(logical(hip.argmin(h, axis)), logical(oracle.argmin(o, axis)))


def test_sum_invariants_and_identities(hip, oracle):
    # backend_contract.ml:2611-2644: a too-narrow accumulator would stall
    for d, n in ((dt.float32, 1 << 25), (dt.float16, 4096), (dt.bfloat16, 512), (dt.bfloat16, 1024)):
        ones = hip.full(d, (n,), encode(np.array([1.0]), d, oracle))
        got = decode(logical(hip.reshape(hip.reduce("sum", [0], ones), (1,))), d, oracle)[0]
        assert got == float(n), (d.name, n, got)
    # int sums wrap
    x = np.full((3, 1000), 2**31 - 1, np.int32)
    h, o = pair(x, dt.int32, hip, oracle)
    same_bits(logical(hip.reduce("sum", [1], h)), logical(oracle.reduce("sum", [1], o)))
    # empty reduced extent: identities for sum/prod, Invalid_argument for max/min/arg
    for d in (dt.float32, dt.int16, dt.bfloat16, dt.complex64):
        e = hip.buffer(d, (0, 5)), oracle.buffer(d, (0, 5))
        for op in ("sum", "prod"):
            same_bits(logical(hip.reduce(op, [0], e[0])), logical(oracle.reduce(op, [0], e[1])))
    for op in ("max", "min"):
        with pytest.raises(ValueError):
            hip.reduce(op, [0], hip.buffer(dt.float64, (0, 3)))
    with pytest.raises(ValueError):
        hip.argmax(hip.buffer(dt.float64, (0, 3)), 0)
    # an empty RESULT is a no-op, not an error
    assert logical(hip.reduce("max", [1], hip.buffer(dt.float32, (0, 3)))).shape == (0,)
    # reference NaN vectors (backend_contract.ml:2486-2512)
    t, _ = pair(np.array([1.0, np.nan, 3.0, 2.0]), dt.float64, hip, oracle)
    assert np.isnan(logical(hip.reduce("max", [0], t))) and np.isnan(logical(hip.reduce("min", [0], t)))
    t, _ = pair(np.array([np.nan, 1.0, 2.0]), dt.float64, hip, oracle)
    assert int(logical(hip.argmax(t, 0))) == 0 and int(logical(hip.argmin(t, 0))) == 0
    t, _ = pair(np.array([5, 0x80000000, 3], np.uint32), dt.uint32, hip, oracle)
    assert int(logical(hip.argmax(t, 0))) == 1  # backend_contract.ml:2810-2816


def test_views_of_high_rank_with_nothing_to_merge(hip, oracle):
    """Sixteen dims of size 2, every other one flipped, so that no two neighbours compose
    (the reference reduces any view up to rank 32: nx_c.h:45, nx_c_engine.c:1052-1170). Reduced
    over every other axis (eight kept, eight reduced), over the odd ones only (twelve kept),
    and over all but one; argmax along one axis; a scan along one."""
    nd = 16
    rng = np.random.default_rng(1600)
    x = rng.integers(-1000, 1000, (2,) * nd).astype(np.int32)
    flips = tuple(i % 2 == 0 for i in range(nd))
    h, o = pair(x, dt.int32, hip, oracle, lambda B, t: B.flip(t, flips))
    want_np = x[tuple(slice(None, None, -1) if f else slice(None) for f in flips)]
    for axes in ([a for a in range(nd) if a % 2 == 0], [1, 5, 9, 13], list(range(1, nd)), list(range(nd - 1))):
        got = logical(hip.reduce("sum", axes, h))
        same_bits(got, logical(oracle.reduce("sum", axes, o)), f"sum over {axes}")
        same_bits(got, want_np.sum(axis=tuple(axes), dtype=np.int32), f"sum over {axes} against numpy")
        same_bits(logical(hip.reduce("max", axes, h)), logical(oracle.reduce("max", axes, o)), f"max over {axes}")
    for axis in (0, 7, nd - 1):
        same_bits(logical(hip.argmax(h, axis)), logical(oracle.argmax(o, axis)), f"argmax along {axis}")
    for axis in (0, 5, nd - 1):
        same_bits(logical(hip.associative_scan(axis, "sum", h)), logical(oracle.associative_scan(axis, "sum", o)),
                  f"cumsum along {axis}")
    xf = rng.standard_normal((2,) * nd).astype(np.float32)
    hf, of = pair(xf, dt.float32, hip, oracle, lambda B, t: B.flip(t, flips))
    got = logical(hip.reduce("sum", [a for a in range(nd) if a % 2], hf))
    want = logical(oracle.reduce("sum", [a for a in range(nd) if a % 2], of))
    assert np.allclose(got, want, rtol=1e-5, atol=1e-4)
    # rank 32 itself: thirty-two dims of size 2 would be 16 GiB of int32; sizes 2 and 1 interleaved
    shape = tuple(2 if i % 2 == 0 else 1 for i in range(32))
    y = rng.integers(-50, 50, shape).astype(np.int32)
    flips32 = tuple(i % 4 == 0 for i in range(32))
    h32, o32 = pair(y, dt.int32, hip, oracle, lambda B, t: B.flip(t, flips32))
    axes = [a for a in range(32) if a % 4 == 2]
    same_bits(logical(hip.reduce("sum", axes, h32)), logical(oracle.reduce("sum", axes, o32)), "rank 32")


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.int32, dt.int8, dt.float64], ids=lambda d: d.name)
def test_two_reduced_dims_that_do_not_merge(hip, oracle, d):
    """Sums, maxima and minima over two axes with a kept axis between them (the batch and the
    positions of [N, C, H, W] with the channels kept; axes 0 and 2 of a rank-3 tensor): the
    unit-stride or the longer reduced dim is walked, every index of the other is a partial result
    that the second pass folds. Both forms (a reduced dim with unit stride; a kept dim with unit
    stride), ragged extents, a window of a wider tensor, against the oracle."""
    rng = np.random.default_rng(1300 + d.tag)
    cases = [
        ("NCHW, channels kept", (9, 20, 13, 11), None, [0, 2, 3], "fold_row_outer"),
        ("axes 0 and 2", (33, 50, 130), None, [0, 2], "fold_row_outer"),
        ("axes 0 and 2, short rows", (70, 6, 9), None, [0, 2], "fold_row_outer"),
        ("window of a wider tensor", (12, 22, 70), lambda B, t: B.shrink(t, [(1, 11), (2, 20), (3, 67)]), [0, 2], "fold_row_outer"),
        ("unit stride kept: axes 0 and 2 of rank 4", (7, 30, 12, 64), None, [0, 2], "fold_col_outer"),
        ("unit stride kept, the earlier dim longer", (40, 3, 9, 48), None, [0, 2], "fold_col_outer"),
        ("channels last, batch and one position axis", (10, 9, 8, 32), None, [0, 2], "fold_col_outer"),
    ]
    for what, shape, build, axes, path in cases:
        if d.is_float:
            x = encode(rng.uniform(-2, 2, shape), d, oracle)
        else:
            info = np.iinfo(d.np_storage)
            x = rng.integers(max(info.min, -100), min(info.max, 100), shape, endpoint=True).astype(d.np_storage)
        h, o = pair(x, d, hip, oracle, build)
        k = int(np.prod([h.shape[a] for a in axes]))
        for op in ("sum", "max", "min"):
            g, w = logical(hip.reduce(op, axes, h)), logical(oracle.reduce(op, axes, o))
            assert hip.last_path() == path, (what, op, hip.last_path())
            if d.is_float and op == "sum":
                close(g, w, d, oracle, TOL[d.name][0], TOL[d.name][0] * 2.0 * k, f"{what} {op}")
            else:
                same_bits(g, w, f"{what} {op}")
    # sums of ones count the reduced elements exactly
    ones = hip.contiguous(hip.full(dt.float32, (64, 48, 512), 1.0))
    same_bits(logical(hip.reduce("sum", [0, 2], ones)), np.full((48,), 64.0 * 512.0, np.float32), "sum of ones")
    assert hip.last_path() == "fold_row_outer"


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.float64, dt.int32, dt.int8, dt.uint8, dt.complex64],
                         ids=lambda d: d.name)
def test_tall_narrow_matrices_reduced_down_their_rows(hip, oracle, d):
    """[rows, L] with fewer than 16 columns, reduced over the rows (class counts, the bias gradient of a
    small layer): read as one flat run, a lane always on the same column. One block and many,
    ragged last blocks, every L from 2 to 15 among the cases."""
    rng = np.random.default_rng(1400 + d.tag)
    for rows, L in ((512, 2), (700, 15), (5000, 10), (100001, 3), (40000, 7), (3000, 13)):
        if d.is_complex:
            x = (rng.uniform(-1, 1, (rows, L)) + 1j * rng.uniform(-1, 1, (rows, L))).astype(np.complex64)
        elif d.is_float:
            x = encode(rng.uniform(-2, 2, (rows, L)), d, oracle)
        else:
            info = np.iinfo(d.np_storage)
            x = rng.integers(max(info.min, -100), min(info.max, 100), (rows, L), endpoint=True).astype(d.np_storage)
        h, o = pair(x, d, hip, oracle)
        for op in ("sum", "max", "min"):
            if d.is_complex and op != "sum":
                continue
            g, w = logical(hip.reduce(op, [0], h)), logical(oracle.reduce(op, [0], o))
            assert hip.last_path() == "fold_narrow", (rows, L, op, hip.last_path())
            if d.is_complex:
                assert np.allclose(g, w, rtol=1e-4, atol=1e-4 * rows), (rows, L)
            elif d.is_float and op == "sum":
                close(g, w, d, oracle, TOL[d.name][0], TOL[d.name][0] * 2.0 * rows, f"[{rows},{L}] {op}")
            else:
                same_bits(g, w, f"[{rows},{L}] {op}")
    ones = hip.contiguous(hip.full(dt.float32, (1 << 20, 10), 1.0))
    same_bits(logical(hip.reduce("sum", [0], ones)), np.full((10,), float(1 << 20), np.float32), "sum of ones")


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.int32, dt.uint8], ids=lambda d: d.name)
def test_argreduce_of_many_short_rows(hip, oracle, d):
    """argmax / argmin along rows of fewer than 32 elements, 65 536 rows or more: a lane per row.
    Ties (the first index wins) and NaNs (the first NaN wins) included, bit for bit."""
    rng = np.random.default_rng(1500 + d.tag)
    for rows, n in ((70000, 10), (65536 + 7, 31), (100000, 2)):
        if d.is_float:
            v = rng.integers(-5, 6, (rows, n)).astype(np.float64)  # many ties
            v[rng.random(v.shape) < 0.01] = np.nan
            x = encode(v, d, oracle)
        else:
            info = np.iinfo(d.np_storage)
            x = rng.integers(max(info.min, -5), min(info.max, 5), (rows, n), endpoint=True).astype(d.np_storage)
        h, o = pair(x, d, hip, oracle)
        same_bits(logical(hip.argmax(h, 1)), logical(oracle.argmax(o, 1)), f"argmax [{rows},{n}]")
        assert hip.last_path() == "arg_row_lane", hip.last_path()
        same_bits(logical(hip.argmin(h, 1)), logical(oracle.argmin(o, 1)), f"argmin [{rows},{n}]")
        # the same rows as columns of the transposed matrix (strided axis)
        ht, ot = pair(np.ascontiguousarray(x.T), d, hip, oracle)
        same_bits(logical(hip.argmax(ht, 0)), logical(oracle.argmax(ot, 0)), f"argmax axis 0 [{n},{rows}]")


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.int32, dt.int8, dt.uint8, dt.bool_], ids=lambda d: d.name)
def test_many_short_rows_reduced_along_the_row(hip, oracle, d):
    """[rows, R] with R from 2 to 32 and thousands of rows (the classes of a batch of logits): a block
    brings 256 rows into LDS and a lane folds its own. Every R at the bank-conflict corners (2, 16,
    31, 32), a ragged last block, NaNs in float rows."""
    rng = np.random.default_rng(1600 + d.tag)
    for rows, R in ((4096, 2), (5000, 10), (70001, 3), (4100, 16), (9000, 31), (8192, 32)):
        if d.is_float:
            v = rng.uniform(-2, 2, (rows, R))
            v.reshape(-1)[rng.integers(0, v.size, 7)] = np.nan
            x = encode(v, d, oracle)
        elif d is dt.bool_:
            x = rng.integers(0, 2, (rows, R)).astype(np.uint8)
        else:
            info = np.iinfo(d.np_storage)
            x = rng.integers(max(info.min, -100), min(info.max, 100), (rows, R), endpoint=True).astype(d.np_storage)
        h, o = pair(x, d, hip, oracle)
        for op in (("max", "min") if d is dt.bool_ else ("sum", "max", "min", "prod")):
            g, w = logical(hip.reduce(op, [1], h)), logical(oracle.reduce(op, [1], o))
            assert hip.last_path() == "fold_short_rows", (rows, R, op, hip.last_path())
            if d.is_float and op in ("sum", "prod"):
                gv, wv = decode(g, d, oracle), decode(w, d, oracle)
                assert np.array_equal(np.isnan(gv), np.isnan(wv)), (rows, R, op)
                ok = ~np.isnan(wv)
                lim = TOL[d.name][0] * R * (np.abs(wv[ok]) + 2.0 ** R if op == "prod" else np.abs(wv[ok]) + 2.0 * R)
                assert np.all(np.abs(gv[ok] - wv[ok]) <= lim), (rows, R, op)
            else:
                same_bits(g, w, f"[{rows},{R}] {op}")
