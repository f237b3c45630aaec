"""The register-blocked GEMM of the dtypes without a matrix instruction (integers, float8,
complex) against the CPU oracle (nx_c_matmul.c:128-605 behind :874-1108).

Integers are exact modulo 2^w in any order. float8 products are exact in float32 and both sides
add them in k order, so for k <= 2048 (where the reference does not cut K, nx_c_matmul.c:79-101)
the bits agree; above, the reference's tolerance applies. Complex products agree to the
reference's tolerance, and to the bit on small-integer data where every partial sum is
representable."""

import numpy as np
import pytest

from helpers import decode, encode, layouts, logical, pair, same_bits
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu

INTS = [dt.int8, dt.uint8, dt.int16, dt.uint16, dt.int32, dt.uint32, dt.int64, dt.uint64]
F8 = [dt.float8_e4m3, dt.float8_e5m2]
SHAPES = [(16, 8, 16), (19, 37, 23), (64, 16, 64), (65, 17, 129), (130, 70, 257), (200, 9, 31)]


def int_data(rng, d, shape):
    info = np.iinfo(d.np_storage)
    return rng.integers(info.min, info.max, shape, endpoint=True, dtype=d.np_storage)


def f8_data(rng, d, shape, oracle):
    return encode(rng.standard_normal(shape) * 0.5, d, oracle)


def both(hip, oracle, d, a, b, build_a=None, build_b=None):
    (ha, oa), (hb, ob) = pair(a, d, hip, oracle, build_a), pair(b, d, hip, oracle, build_b)
    got = logical(hip.matmul(ha, hb))
    path = hip.last_path()
    return got, logical(oracle.matmul(oa, ob)), path


@pytest.mark.parametrize("d", INTS, ids=lambda d: d.name)
def test_integers_every_operand_order(hip, oracle, d):
    rng = np.random.default_rng(4100 + d.tag)
    tr = lambda B, t: B.permute(t, (1, 0))
    for (m, k, n) in SHAPES:
        a, b = int_data(rng, d, (m, k)), int_data(rng, d, (k, n))
        for ta in (False, True):
            for tb in (False, True):
                got, want, path = both(hip, oracle, d, np.ascontiguousarray(a.T) if ta else a,
                                       np.ascontiguousarray(b.T) if tb else b, tr if ta else None, tr if tb else None)
                assert path == "gemm_block_64x64", (m, k, n, path)
                same_bits(got, want, f"{d.name} {m}x{k}x{n} ta={ta} tb={tb}")


@pytest.mark.parametrize("d", [dt.int8, dt.uint16, dt.int32, dt.uint32, dt.float8_e4m3], ids=lambda d: d.name)
def test_products_of_many_blocks(hip, oracle, d):
    rng = np.random.default_rng(4200 + d.tag)
    m, k, n = 2048, 72, 2040  # 32 x 32 blocks, ragged in n and in the last slab of k
    if d in F8:
        a, b = f8_data(rng, d, (m, k), oracle), f8_data(rng, d, (k, n), oracle)
    else:
        a, b = int_data(rng, d, (m, k)), int_data(rng, d, (k, n))
    got, want, path = both(hip, oracle, d, a, b)
    assert path == "gemm_block_64x64", path
    same_bits(got, want, d.name)
    # the same product with both operands transposed in memory
    tr = lambda B, t: B.permute(t, (1, 0))
    got, want, path = both(hip, oracle, d, np.ascontiguousarray(a.T), np.ascontiguousarray(b.T), tr, tr)
    assert path == "gemm_block_64x64", path
    same_bits(got, want, d.name + " transposed")


@pytest.mark.parametrize("d", [dt.int16, dt.int64, dt.float8_e5m2], ids=lambda d: d.name)
def test_views_of_the_layout_matrix(hip, oracle, d):
    """Batched operands in every layout of the reference's matrix (backend_contract.ml:423-468):
    permuted, offset, broadcast (stride 0) and flipped (negative strides)."""
    rng = np.random.default_rng(4300 + d.tag)
    la, lb = layouts((3, 40, 24)), layouts((3, 24, 50))
    for (na, sa, fa) in la:
        for (nb, sb, fb) in lb:
            if d in F8:
                a, b = f8_data(rng, d, sa, oracle), f8_data(rng, d, sb, oracle)
            else:
                a, b = int_data(rng, d, sa), int_data(rng, d, sb)
            got, want, path = both(hip, oracle, d, a, b, fa, fb)
            assert path == "gemm_block_64x64", (na, nb, path)
            same_bits(got, want, f"{d.name} {na} x {nb}")


@pytest.mark.parametrize("d", F8, ids=lambda d: d.name)
def test_float8_bits_up_to_the_uncut_k_and_tolerance_above(hip, oracle, d):
    rng = np.random.default_rng(4400 + d.tag)
    for (m, k, n) in SHAPES + [(48, 2048, 40)]:
        a, b = f8_data(rng, d, (m, k), oracle), f8_data(rng, d, (k, n), oracle)
        got, want, path = both(hip, oracle, d, a, b)
        assert path == "gemm_block_64x64", path
        same_bits(got, want, f"{d.name} {m}x{k}x{n}")
    m, k, n = 48, 2500, 56  # the reference sums 512-deep pieces separately here
    a, b = f8_data(rng, d, (m, k), oracle) , f8_data(rng, d, (k, n), oracle)
    got, want, _ = both(hip, oracle, d, a, b)
    g, w = decode(got, d, oracle), decode(want, d, oracle)
    tol = 0.3 if d is dt.float8_e4m3 else 0.4  # matmul_test.ml:831-974
    assert np.all(np.abs(g - w) <= tol * (np.abs(w) + np.sqrt(k) * 0.25))
    # values no sum can reach by rounding: a row of NaN, an overflowing row
    a = f8_data(rng, d, (32, 64), oracle)
    b = f8_data(rng, d, (64, 32), oracle)
    a[3, 5] = 0x7f  # NaN in both formats
    a[7, :] = encode(np.full((64,), 200.0), d, oracle)
    b[:, 9] = encode(np.full((64,), 200.0), d, oracle)
    got, want, _ = both(hip, oracle, d, a, b)
    gv, wv = decode(got, d, oracle), decode(want, d, oracle)
    assert np.array_equal(np.isnan(gv), np.isnan(wv)) and np.isnan(gv[3]).all()
    same_bits(np.where(np.isnan(gv), 0, got), np.where(np.isnan(wv), 0, want), d.name + " specials")


@pytest.mark.parametrize("d", [dt.complex64, dt.complex128], ids=lambda d: d.name)
def test_complex(hip, oracle, d):
    rng = np.random.default_rng(4500 + d.tag)
    tol = 1e-3 if d is dt.complex64 else 1e-9
    tr = lambda B, t: B.permute(t, (1, 0))
    for (m, k, n) in SHAPES + [(257, 300, 65)]:
        a = (rng.standard_normal((m, k)) + 1j * rng.standard_normal((m, k))).astype(d.np_storage)
        b = (rng.standard_normal((k, n)) + 1j * rng.standard_normal((k, n))).astype(d.np_storage)
        for ta, tb in ((False, False), (True, True)):
            got, _, path = both(hip, oracle, d, np.ascontiguousarray(a.T) if ta else a,
                                np.ascontiguousarray(b.T) if tb else b, tr if ta else None, tr if tb else None)
            assert path == "gemm_block_64x64", path
            want = a.astype(np.complex128) @ b.astype(np.complex128)
            assert np.all(np.abs(got.astype(np.complex128) - want) <= tol * (np.abs(want) + np.sqrt(k))), (m, k, n)
    # small integers: every partial sum is exact, so the bits are the oracle's
    a = (rng.integers(-4, 5, (70, 90)) + 1j * rng.integers(-4, 5, (70, 90))).astype(d.np_storage)
    b = (rng.integers(-4, 5, (90, 33)) + 1j * rng.integers(-4, 5, (90, 33))).astype(d.np_storage)
    got, want, _ = both(hip, oracle, d, a, b)
    same_bits(got, want, d.name + " small integers")


def test_thin_products_stay_with_one_lane_per_output(hip, oracle):
    rng = np.random.default_rng(4600)
    for (m, k, n) in [(1, 300, 200), (200, 300, 3), (40, 4, 40)]:
        a, b = int_data(rng, dt.int32, (m, k)), int_data(rng, dt.int32, (k, n))
        got, want, path = both(hip, oracle, dt.int32, a, b)
        assert path == "gemm_any", (m, k, n, path)
        same_bits(got, want)
