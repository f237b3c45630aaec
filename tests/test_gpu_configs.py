"""Parity at the benchmark's five configurations, full size, through the C ABI.

Configs 1-3 are compared with the CPU oracle directly (it finishes them in
seconds). Config 4's big GEMMs are compared with an f64 product on sampled
rows/columns and through size-independent properties (linearity in A, the
identity matrix, batch independence); their small-shape parity is in
test_gpu_matmul.py."""

import numpy as np
import pytest

from helpers import decode, encode, logical, pair, same_bits
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu


def test_config1_chain(hip, oracle):
    n = 4096
    a, b, c = (np.random.default_rng(s).uniform(-1, 1, (n, n)).astype(np.float32) for s in (1, 2, 3))

    def chain(B, ta, tb, tc):
        t1 = B.binary("mul", ta, tb)
        t2 = B.unary("sin", tc)
        t3 = B.binary("add", t1, t2)
        return t1, t2, t3, B.reduce("sum", [1], t3)

    (ha, oa), (hb, ob), (hc, oc) = (pair(x, dt.float32, hip, oracle) for x in (a, b, c))
    h1, h2, h3, hz = chain(hip, ha, hb, hc)
    o1, o2, o3, oz = chain(oracle, oa, ob, oc)
    same_bits(logical(h1), logical(o1), "mul")                      # IEEE-exact
    ulp = np.abs(logical(h2).view(np.int32).astype(np.int64) - logical(o2).view(np.int32)).max()
    assert ulp <= 2, f"sin differs from glibc by {ulp} ulp"          # stated f32 bound
    z, zr = logical(hz).astype(np.float64), logical(oz).astype(np.float64)
    exact = (a.astype(np.float64) * b + np.sin(c.astype(np.float64))).sum(axis=1)
    # contract: |err| <= k * a_rel (backend_contract.ml:908-913), k = 4096, a_rel = 1e-5
    assert np.max(np.abs(z - zr)) <= 4096 * 1e-5
    assert np.max(np.abs(z - exact)) <= 4096 * 1e-5
    print(f"config1: max |z - oracle| {np.max(np.abs(z - zr)):.3g}, max |z - f64| {np.max(np.abs(z - exact)):.3g}, "
          f"oracle vs f64 {np.max(np.abs(zr - exact)):.3g}")
    # the reduction alone, on identical t3, differs only by summation order
    h3o = pair(logical(o3), dt.float32, hip, oracle)[0]
    zz = logical(hip.reduce("sum", [1], h3o)).astype(np.float64)
    assert np.max(np.abs(zz - zr) / np.maximum(1.0, np.abs(zr))) <= 1e-4


def test_config2_strided_broadcast(hip, oracle):
    shp = (64, 512, 512)
    a = np.random.default_rng(4).standard_normal(shp).astype(np.float32)
    b = np.random.default_rng(5).standard_normal((1, 512, 1)).astype(np.float32)
    perm = lambda B, t: B.permute(t, (0, 2, 1))   # noqa: E731
    exp = lambda B, t: B.expand(t, shp)           # noqa: E731
    (ha, oa), (hb, ob) = pair(a, dt.float32, hip, oracle, perm), pair(b, dt.float32, hip, oracle, exp)
    assert ha.strides == (262144, 1, 512) and hb.strides == (0, 1, 0)
    res = []
    for B, ta, tb in ((hip, ha, hb), (oracle, oa, ob)):
        half = B.expand(B.full(dt.float32, (), np.array([0.5], np.float32)), shp)
        t = B.binary("add", ta, tb)
        u = B.binary("mul", t, half)
        res.append((t, u, B.cast(u, dt.float16)))
    for g, w, what in zip(res[0], res[1], ("add", "mul", "cast f16")):
        same_bits(logical(g), logical(w), what)
    ai = np.random.default_rng(6).integers(-1000, 1001, shp).astype(np.int32)
    bi = np.random.default_rng(7).integers(-1000, 1001, (1, 512, 1)).astype(np.int32)
    (ha, oa), (hb, ob) = pair(ai, dt.int32, hip, oracle, perm), pair(bi, dt.int32, hip, oracle, exp)
    res = []
    for B, ta, tb in ((hip, ha, hb), (oracle, oa, ob)):
        m = B.compare("cmplt", tb, ta)
        res.append((B.binary("add", ta, tb), B.binary("mul", ta, tb), m, B.where(m, ta, tb)))
    for g, w, what in zip(res[0], res[1], ("add", "mul", "cmplt", "where")):
        same_bits(logical(g), logical(w), what)
    # closed form, independent of the oracle
    at = np.transpose(ai, (0, 2, 1))
    assert np.array_equal(logical(res[0][3]), np.where(bi < at, at, np.broadcast_to(bi, shp)))


def test_config3_reductions(hip, oracle):
    n = 8192
    x = np.random.default_rng(8).standard_normal((n, n)).astype(np.float32)
    xi = np.random.default_rng(9).integers(-1000, 1001, (n, n)).astype(np.int32)
    (hx, ox), (hi, oi) = pair(x, dt.float32, hip, oracle), pair(xi, dt.int32, hip, oracle)
    for axis in (1, 0):
        s, sr = logical(hip.reduce("sum", [axis], hx)), logical(oracle.reduce("sum", [axis], ox))
        exact = x.astype(np.float64).sum(axis=axis)
        assert np.max(np.abs(s - exact)) <= n * 1e-5 * 4 and np.max(np.abs(sr - exact)) <= n * 1e-5 * 4
        same_bits(logical(hip.reduce("max", [axis], hx)), logical(oracle.reduce("max", [axis], ox)), f"max {axis}")
        same_bits(logical(hip.argmax(hx, axis)), logical(oracle.argmax(ox, axis)), f"argmax {axis}")
        same_bits(logical(hip.reduce("sum", [axis], hi)), logical(oracle.reduce("sum", [axis], oi)), f"isum {axis}")
        assert np.array_equal(logical(hip.argmax(hx, axis)), x.argmax(axis=axis).astype(np.int32))
        print(f"config3 axis {axis}: sum max |gpu - f64| {np.max(np.abs(s - exact)):.3g}, "
              f"oracle {np.max(np.abs(sr - exact)):.3g}")


def sample_check(got, a64, b64, rows, cols, tol, scale):
    want = a64[rows] @ b64[:, cols]
    err = np.abs(got[np.ix_(rows, cols)] - want)
    assert np.all(err <= tol * (np.abs(want) + scale)), float(err.max())


def test_config4_f32_2048(hip, oracle):
    a = (np.random.default_rng(10).standard_normal((2048, 2048)) * 0.02).astype(np.float32)
    b = (np.random.default_rng(11).standard_normal((2048, 2048)) * 0.02).astype(np.float32)
    ha, hb = pair(a, dt.float32, hip, oracle)[0], pair(b, dt.float32, hip, oracle)[0]
    got = logical(hip.matmul(ha, hb)).astype(np.float64)
    want = a.astype(np.float64) @ b.astype(np.float64)
    assert np.all(np.abs(got - want) <= 1e-3 * (np.abs(want) + 0.02 * 0.02 * np.sqrt(2048)))
    eye = pair(np.eye(2048, dtype=np.float32), dt.float32, hip, oracle)[0]
    same_bits(logical(hip.matmul(ha, eye)), a, "A @ I")
    same_bits(logical(hip.matmul(eye, hb)), b, "I @ B")
    # oracle on a slab of rows: same quantised inputs, k-ordered f32 sums
    oa, ob = pair(a[:64], dt.float32, hip, oracle)[1], pair(b, dt.float32, hip, oracle)[1]
    ref = logical(oracle.matmul(oa, ob)).astype(np.float64)
    assert np.max(np.abs(got[:64] - ref)) <= 1e-3 * (np.abs(ref).max() + 1e-3)


def cfg4_bf16_operands(hip, nb=16, n=4096):
    """A, B bf16 [16,4096,4096]: N(0, 0.02) float32 from seeds 12 / 13, sixteen distinct
    matrices each, narrowed to bf16 on the device (the cast is pinned bit for bit
    elsewhere). Returns the device tensors and the host float32 batches used for sampling."""
    out = []
    for seed in (12, 13):
        rng = np.random.default_rng(seed)
        full = hip.buffer(dt.bfloat16, (nb, n, n))
        keep = {}
        for i in range(nb):
            m = (rng.standard_normal((n, n)) * 0.02).astype(np.float32)
            t = hip.cast(hip.reshape(hip.from_host(m, dt.float32), (1, n, n)), dt.bfloat16)
            hip.assign(hip.shrink(full, [(i, i + 1), (0, n), (0, n)]), t)
            if i in (0, 1, 7, 15):
                keep[i] = m
        out.append((full, keep))
    return out


def test_config4_bf16_batched(hip, oracle):
    nb, n = 16, 4096
    (Afull, a32), (Bfull, b32) = cfg4_bf16_operands(hip, nb, n)
    Cf = hip.matmul(Afull, Bfull)
    assert hip.last_path() == "gemm_dl_256x256" and Cf.shape == (nb, n, n)
    rng = np.random.default_rng(99)
    rows, cols = rng.integers(0, n, 48), rng.integers(0, n, 48)
    enc = lambda m: decode(encode(m, dt.bfloat16, oracle), dt.bfloat16, oracle)  # noqa: E731  the quantised inputs
    for i in (0, 1, 7, 15):
        ci = decode(logical(hip.shrink(Cf, [(i, i + 1), (0, n), (0, n)])), dt.bfloat16, oracle)[0]
        sample_check(ci, enc(a32[i]), enc(b32[i]), rows, cols, 6e-2, 0.02 * 0.02 * np.sqrt(n))
    # a batch computed alone equals the same batch inside the batched call, bit for bit
    one = hip.matmul(hip.shrink(Afull, [(7, 8), (0, n), (0, n)]), hip.shrink(Bfull, [(7, 8), (0, n), (0, n)]))
    same_bits(logical(one), logical(hip.shrink(Cf, [(7, 8), (0, n), (0, n)])), "batch independence")
    # oracle on a thin slab of batch 0 (k-ordered f32 accumulate, one rounding)
    c0 = logical(hip.shrink(Cf, [(0, 1), (0, n), (0, n)]))
    oa = pair(encode(a32[0][:16], dt.bfloat16, oracle), dt.bfloat16, hip, oracle)[1]
    ob = pair(encode(b32[0][:, :256], dt.bfloat16, oracle), dt.bfloat16, hip, oracle)[1]
    ref = decode(logical(oracle.matmul(oa, ob)), dt.bfloat16, oracle)
    got = decode(c0[0][:16, :256], dt.bfloat16, oracle)
    assert np.max(np.abs(got - ref)) <= 6e-2 * (np.abs(ref).max())


def test_config4_skinny(hip, oracle):
    for d, tol in ((dt.bfloat16, 6e-2), (dt.float32, 1e-3)):
        a = encode(np.random.default_rng(14).standard_normal((8, 4096)) * 0.02, d, oracle)
        b = encode(np.random.default_rng(15).standard_normal((4096, 16384)) * 0.02, d, oracle)
        (ha, oa), (hb, ob) = pair(a, d, hip, oracle), pair(b, d, hip, oracle)
        got = decode(logical(hip.matmul(ha, hb)), d, oracle)
        assert hip.last_path().startswith("gemm_skinny")
        want = decode(a, d, oracle) @ decode(b, d, oracle)
        assert np.all(np.abs(got - want) <= tol * (np.abs(want) + 0.02 * 0.02 * 64))
        ref = decode(logical(oracle.matmul(oa, ob)), d, oracle)  # the oracle's k-ordered sum
        assert np.max(np.abs(got - ref)) <= tol * np.abs(ref).max()
