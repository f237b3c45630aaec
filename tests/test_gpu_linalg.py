"""cholesky / triangular_solve / qr / eigh / svd / eig on the GPU. Unique results
(L, the solve, Q and R under LAPACK's sign convention, eigenvalues, singular
values) are compared with the CPU oracle; vectors that are only determined up
to a unit phase are checked through the invariants the reference's own tests
use (backend_contract.ml:2075-2311: reconstruction and orthogonality residuals
relative to the matrix norm, 1e-9 in double)."""

import numpy as np
import pytest

from helpers import decode, logical
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu

DTYPES = {"float64": dt.float64, "float32": dt.float32, "complex128": dt.complex128, "complex64": dt.complex64}
TOL = {"float64": 1e-10, "complex128": 1e-10, "float32": 2e-5, "complex64": 2e-5}


def matrix(rng, shape, d):
    a = rng.standard_normal(shape)
    if d.is_complex:
        a = a + 1j * rng.standard_normal(shape)
    return a.astype(d.np_storage)


def both(hip, oracle, a, d, build=None):
    a = np.ascontiguousarray(a)
    out = []
    for B in (hip, oracle):
        t = B.reshape(B.from_host(a, d), a.shape)
        out.append(build(B, t) if build else t)
    return out


def arr(t):
    return logical(t).astype(np.complex128 if np.iscomplexobj(logical(t)) else np.float64)


def rel(a, b):
    return np.max(np.abs(a - b)) / max(1e-30, np.max(np.abs(b)))


def H(a):
    return np.swapaxes(a, -1, -2).conj()


def spd(rng, batch, n, d):
    g = matrix(rng, batch + (n, n), d).astype(np.complex128 if d.is_complex else np.float64)
    return (g @ H(g) + n * np.eye(n)).astype(d.np_storage)


@pytest.mark.parametrize("name", list(DTYPES))
def test_cholesky(hip, oracle, name):
    d, tol = DTYPES[name], TOL[name]
    rng = np.random.default_rng(1)
    for batch, n in (((), 1), ((), 4), ((3,), 17), ((2, 2), 64), ((), 200)):
        a = spd(rng, batch, n, d)
        a[..., 0, n - 1] = 77  # the upper triangle is not read (nx_c_tri.c:11-16)
        h, o = both(hip, oracle, a, d)
        for upper in (False, True):
            got, want = arr(hip.cholesky(h, upper)), arr(oracle.cholesky(o, upper))
            assert rel(got, want) <= tol, (n, upper)
            assert np.all((np.triu(got, 1) if not upper else np.tril(got, -1)) == 0)
    # a permuted (transposed) view of a Hermitian matrix is its conjugate
    a = spd(rng, (), 9, d)
    h, o = both(hip, oracle, a, d, lambda B, t: B.permute(t, (1, 0)))
    assert rel(arr(hip.cholesky(h)), arr(oracle.cholesky(o))) <= tol
    bad = np.eye(5).astype(d.np_storage)
    bad[3, 3] = -1
    with pytest.raises(RuntimeError, match="not positive definite"):
        hip.cholesky(hip.reshape(hip.from_host(bad, d), (5, 5)))
    bad[3, 3] = np.nan
    with pytest.raises(RuntimeError, match="not positive definite"):
        hip.cholesky(hip.reshape(hip.from_host(bad, d), (5, 5)))
    good = hip.reshape(hip.from_host(np.eye(5).astype(d.np_storage), d), (5, 5))
    assert np.array_equal(arr(hip.cholesky(good)), np.eye(5))  # the failure did not stick


@pytest.mark.parametrize("name", list(DTYPES))
def test_triangular_solve(hip, oracle, name):
    d, tol = DTYPES[name], TOL[name] * 50
    rng = np.random.default_rng(2)
    for batch, n, nrhs in (((), 3, 2), ((2,), 33, 5), ((), 150, 1), ((), 70, 300)):
        a = matrix(rng, batch + (n, n), d)
        a[..., np.arange(n), np.arange(n)] += (4 + n / 8)  # well conditioned
        b = matrix(rng, batch + (n, nrhs), d)
        ha, oa = both(hip, oracle, a, d)
        hb, ob = both(hip, oracle, b, d)
        for upper in (False, True):
            for transpose in (False, True):
                for unit in (False, True):
                    got = arr(hip.triangular_solve(ha, hb, upper, transpose, unit))
                    want = arr(oracle.triangular_solve(oa, ob, upper, transpose, unit))
                    assert rel(got, want) <= tol, (n, upper, transpose, unit)
    # vector right-hand sides (backend_contract.ml:2186-2209)
    a = np.array([[2, 0, 0], [1, 3, 0], [-1, 2, 4]], d.np_storage)
    ha = hip.reshape(hip.from_host(a, d), (3, 3))
    x = hip.triangular_solve(ha, hip.from_host(np.array([2, 7, 15], d.np_storage), d), False, False, False)
    assert logical(x).shape == (3,) and np.allclose(arr(x), [1, 2, 3], atol=1e-6)
    a[1, 1] = 0
    with pytest.raises(RuntimeError, match="singular"):
        hip.triangular_solve(hip.reshape(hip.from_host(a, d), (3, 3)), hip.from_host(np.ones(3, d.np_storage), d),
                             False, False, False)
    hip.triangular_solve(hip.reshape(hip.from_host(a, d), (3, 3)), hip.from_host(np.ones(3, d.np_storage), d),
                         False, False, True)  # the diagonal is not read with unit_diag


@pytest.mark.parametrize("name", list(DTYPES))
def test_qr(hip, oracle, name):
    d, tol = DTYPES[name], TOL[name] * 20
    rng = np.random.default_rng(3)
    for batch, m, n in (((), 4, 3), ((), 3, 4), ((2,), 20, 20), ((3,), 65, 17), ((), 10, 130), ((), 1, 1)):
        a = matrix(rng, batch + (m, n), d)
        h, o = both(hip, oracle, a, d)
        for reduced in (True, False):
            (q, r), (oq, orr) = hip.qr(h, reduced), oracle.qr(o, reduced)
            q, r = arr(q), arr(r)
            k = min(m, n)
            assert q.shape == batch + (m, k if reduced else m) and r.shape == batch + (k if reduced else m, n)
            wide = a.astype(q.dtype)
            assert rel(q @ r, wide) <= tol and rel(H(q) @ q, np.broadcast_to(np.eye(q.shape[-1]), q.shape[:-2] + (q.shape[-1],) * 2)) <= tol
            assert np.all(np.tril(r, -1) == 0)
            # the same Householder convention: factors agree, not only their product
            assert rel(r, arr(orr)) <= tol and rel(q[..., :k], arr(oq)[..., :k]) <= tol, (m, n, reduced)


@pytest.mark.parametrize("name", list(DTYPES))
def test_eigh_and_eigvalsh(hip, oracle, name):
    d, tol = DTYPES[name], TOL[name] * 20
    rng = np.random.default_rng(4)
    for batch, n in (((), 1), ((), 2), ((), 3), ((2,), 4), ((3,), 17), ((), 64), ((), 129), ((3,), 70)):
        g = matrix(rng, batch + (n, n), d)
        a = (g + H(g)).astype(d.np_storage)
        a[..., 0, n - 1] = 55 if n > 1 else a[..., 0, 0]  # the upper triangle is not read (nx_c_eigh.c:14)
        h, o = both(hip, oracle, a, d)
        w, v = hip.eigh(h)
        assert hip.last_path() == ("eigh_jacobi_wide" if n > 64 else "eigh_jacobi")
        ow, _ = oracle.eigh(o)
        w, v, ow = logical(w), arr(v), logical(ow)
        assert w.dtype == np.float64 and w.shape == batch + (n,)
        scale = max(1.0, np.max(np.abs(ow)))
        assert np.max(np.abs(w - ow)) <= tol * scale and np.all(np.diff(w, axis=-1) >= 0)
        assert np.max(np.abs(logical(hip.eigvalsh(h)) - ow)) <= tol * scale
        low = np.tril(a.astype(v.dtype))
        full = low + H(np.tril(a.astype(v.dtype), -1))
        assert np.max(np.abs(full @ v - v * w[..., None, :])) <= tol * scale * n
        assert rel(H(v) @ v, np.broadcast_to(np.eye(n), batch + (n, n))) <= tol * n
    nan = np.full((3, 3), np.nan).astype(d.np_storage)
    for call in (hip.eigh, hip.svd, hip.eig):
        with pytest.raises(RuntimeError, match="did not converge"):
            call(hip.reshape(hip.from_host(nan, d), (3, 3)))


@pytest.mark.parametrize("name", list(DTYPES))
def test_svd(hip, oracle, name):
    d, tol = DTYPES[name], TOL[name] * 20
    rng = np.random.default_rng(5)
    cases = [((), 4, 3), ((), 3, 4), ((2,), 16, 16), ((3,), 40, 7), ((), 9, 70), ((), 1, 1), ((), 100, 100),
             ((2,), 90, 75), ((2,), 67, 130)]
    for batch, m, n in cases:
        a = matrix(rng, batch + (m, n), d)
        if m == 16:
            a[..., :, 3] = a[..., :, 5]  # rank deficient
        h, o = both(hip, oracle, a, d)
        for full in (False, True):
            u, s, vt = hip.svd(h, full)
            _, os_, _ = oracle.svd(o, full)
            u, s, vt, os_ = arr(u), logical(s), arr(vt), logical(os_)
            k = min(m, n)
            assert s.dtype == np.float64 and s.shape == batch + (k,)
            assert u.shape == batch + (m, m if full else k) and vt.shape == batch + (n if full else k, n)
            scale = max(1.0, os_.max())
            assert np.max(np.abs(s - os_)) <= tol * scale and np.all(np.diff(s, axis=-1) <= 0) and np.all(s >= 0)
            recon = (u[..., :, :k] * s[..., None, :]) @ vt[..., :k, :]
            assert np.max(np.abs(recon - a.astype(recon.dtype))) <= tol * scale * 4
            for f in (u, H(vt)):
                assert rel(H(f) @ f, np.broadcast_to(np.eye(f.shape[-1]), f.shape[:-2] + (f.shape[-1],) * 2)) <= tol * 4


@pytest.mark.parametrize("name", list(DTYPES))
def test_eig_and_eigvals(hip, oracle, name):
    d, tol = DTYPES[name], TOL[name] * 100
    rng = np.random.default_rng(6)
    fixed = np.array([[2, -1, 0], [1, 3, -1], [0, 1, 2]], d.np_storage)  # backend_contract.ml:2236-2256
    mats = [fixed] + [matrix(rng, batch + (n, n), d) for batch, n in (((), 1), ((), 2), ((3,), 5), ((2,), 20), ((), 77))]
    mats.append(np.triu(matrix(rng, (6, 6), d)))            # already triangular
    mats.append(np.diag(np.arange(1, 6)).astype(d.np_storage))  # diagonal, nothing to iterate
    for a in mats:
        n = a.shape[-1]
        h, o = both(hip, oracle, a, d)
        w, v = hip.eig(h)
        w, v, ow = logical(w), logical(v), logical(oracle.eigvals(o))
        assert w.dtype == np.complex128 and v.dtype == np.complex128 and v.shape == a.shape
        scale = max(1.0, np.max(np.abs(ow)))
        wide = a.astype(np.complex128)
        assert np.max(np.abs(wide @ v - v * w[..., None, :])) <= tol * scale * n
        assert np.max(np.abs(np.linalg.norm(v, axis=-2) - 1)) <= 1e-12
        wv = logical(hip.eigvals(h))
        for got in (w, wv):  # the same multiset as LAPACK's, whatever the order
            for idx in np.ndindex(*a.shape[:-2]):
                dist = np.abs(got[idx][:, None] - ow[idx][None, :])
                assert dist.min(axis=1).max() <= tol * scale * 10 and dist.min(axis=0).max() <= tol * scale * 10


def test_half_precision_storage_and_rejections(hip, oracle):
    rng = np.random.default_rng(7)
    for d in (dt.bfloat16, dt.float16):
        g = rng.standard_normal((6, 6))
        a = g @ g.T + 6 * np.eye(6)
        from helpers import encode
        st = encode(a, d, oracle)
        h, o = both(hip, oracle, st, d)
        got, want = decode(logical(hip.cholesky(h)), d, oracle), decode(logical(oracle.cholesky(o)), d, oracle)
        assert np.max(np.abs(got - want)) <= 0.02 * np.max(np.abs(want))
        assert logical(hip.eigh(h)[0]).dtype == np.float64
    ints = hip.reshape(hip.from_host(np.eye(3, dtype=np.int32), dt.int32), (3, 3))
    for call in (hip.cholesky, hip.eigh, hip.svd, hip.eig, hip.qr):
        with pytest.raises(RuntimeError, match="float or complex"):
            call(ints)
    rect = hip.reshape(hip.from_host(np.zeros(6, np.float32), dt.float32), (2, 3))
    for call in (hip.cholesky, hip.eigh, hip.eig):
        with pytest.raises(ValueError, match="square"):
            call(rect)
    empty = hip.reshape(hip.from_host(np.zeros(0, np.float32), dt.float32), (0, 3, 3))
    assert logical(hip.cholesky(empty)).shape == (0, 3, 3)


def test_failures_of_the_device_wide_forms(hip):
    """From 65 rows on the factorisations run as many launches: the numeric
    failures must come out of those too, and must not stick to the next call."""
    d, n = dt.float64, 100
    rng = np.random.default_rng(8)
    g = rng.standard_normal((n, n))
    a = g @ g.T + n * np.eye(n)
    mk = lambda x: hip.reshape(hip.from_host(np.ascontiguousarray(x), d), x.shape)
    bad = a.copy()
    bad[60, 60] = -1e6
    with pytest.raises(RuntimeError, match="not positive definite"):
        hip.cholesky(mk(bad))
    assert hip.last_path() == "cholesky_columns_wide"
    low = arr(hip.cholesky(mk(a)))
    assert rel(low @ low.T, a) <= 1e-12
    tri = np.tril(a)
    tri[77, 77] = 0.0
    with pytest.raises(RuntimeError, match="singular"):
        hip.triangular_solve(mk(tri), mk(np.ones((n, 3))), False, False, False)
    x = arr(hip.triangular_solve(mk(np.tril(a)), mk(np.ones((n, 3))), False, False, False))
    assert rel(np.tril(a) @ x, np.ones((n, 3))) <= 1e-10
    nan = a.copy()
    nan[5, 3] = np.nan
    for call in (hip.eigh, hip.svd):
        with pytest.raises(RuntimeError, match="did not converge"):
            call(mk(nan))
    w, _ = hip.eigh(mk(a))
    assert np.max(np.abs(logical(w) - np.linalg.eigvalsh(a))) <= 1e-9 * np.max(np.abs(a))
    # two matrices, one of which fails: the call fails as a whole
    pair = np.stack([a, bad])
    with pytest.raises(RuntimeError, match="not positive definite"):
        hip.cholesky(mk(pair))
