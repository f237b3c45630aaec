"""Shared helpers of the parity tests: build the same tensor (same host bytes,
same view) on the HIP backend and on the CPU oracle, and compare results."""

from __future__ import annotations

import numpy as np

from oracle import nx_oracle
from raven_amd import dtype as dt
from raven_amd import nx_backend

FLOAT_DTYPES = [dt.float16, dt.float32, dt.float64, dt.bfloat16, dt.float8_e4m3, dt.float8_e5m2]
INT_DTYPES = [dt.int8, dt.uint8, dt.int16, dt.uint16, dt.int32, dt.uint32, dt.int64, dt.uint64]
COMPLEX_DTYPES = [dt.complex64, dt.complex128]

# Tolerances of the reference contract for (arith, transcendental) results
# (packages/nx/test/backend_contract.ml:147-189), relative == absolute scale.
TOL = {
    "float64": (1e-11, 1e-9), "float32": (1e-5, 1e-4), "float16": (5e-3, 2e-2),
    "bfloat16": (3e-2, 6e-2), "float8_e4m3": (0.13, 0.26), "float8_e5m2": (0.26, 0.5),
    "complex64": (1e-5, 1e-4), "complex128": (1e-11, 1e-9),
}


def logical(t):
    if isinstance(t, nx_backend.Tensor):
        return nx_backend.logical(t)
    return nx_oracle.logical(t)


def encode(values: np.ndarray, d: dt.DType, oracle) -> np.ndarray:
    """Host storage bytes for float `values` in dtype d (oracle's pinned
    converters do the narrowing for bf16 / fp8)."""
    values = np.asarray(values)
    if d in (dt.bfloat16, dt.float8_e4m3, dt.float8_e5m2):
        t = oracle.reshape(oracle.from_host(values.astype(np.float32), dt.float32), values.shape)
        return nx_oracle.logical(oracle.cast(t, d))
    with np.errstate(all="ignore"):
        return values.astype(d.np_storage)


def decode(storage: np.ndarray, d: dt.DType, oracle) -> np.ndarray:
    """float64 (or complex128) values of a storage array of dtype d."""
    if d in (dt.bfloat16, dt.float8_e4m3, dt.float8_e5m2):
        t = oracle.reshape(oracle.from_host(storage, d), storage.shape)
        return nx_oracle.logical(oracle.cast(t, dt.float32)).astype(np.float64)
    if d.is_complex:
        return storage.astype(np.complex128)
    return storage.astype(np.float64)


def pair(storage: np.ndarray, d: dt.DType, hip, oracle, build=None):
    """The same tensor on both backends. `build(B, t)` applies view ops."""
    storage = np.ascontiguousarray(storage)
    out = []
    for B in (hip, oracle):
        t = B.reshape(B.from_host(storage, d), storage.shape)
        out.append(build(B, t) if build else t)
    return out


def layouts(shape3):
    """The reference's layout matrix (backend_contract.ml:423-468) as
    (name, source-array shape, view builder). Every builder maps a tensor of
    `src_shape` to a view of logical shape `shape3` (rank 3 here)."""
    a, b, c = shape3
    return [
        ("contiguous", (a, b, c), lambda B, t: t),
        ("transposed", (a, c, b), lambda B, t: B.permute(t, (0, 2, 1))),
        ("permuted", (c, a, b), lambda B, t: B.permute(t, (1, 2, 0))),
        ("offset_slice", (a + 2, b + 1, c + 3),
         lambda B, t: B.shrink(t, [(1, a + 1), (1, b + 1), (2, c + 2)])),
        ("broadcast", (1, b, 1), lambda B, t: B.expand(t, (a, b, c))),
        ("flipped", (a, b, c), lambda B, t: B.flip(t, (False, True, True))),
    ]


def same_bits(got: np.ndarray, want: np.ndarray, what=""):
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert got.dtype == want.dtype, (what, got.dtype, want.dtype)
    g = np.ascontiguousarray(got).view(np.uint8)
    w = np.ascontiguousarray(want).view(np.uint8)
    if not np.array_equal(g, w):
        bad = np.flatnonzero(np.ascontiguousarray(got).reshape(-1).view(f"V{got.dtype.itemsize}") !=
                             np.ascontiguousarray(want).reshape(-1).view(f"V{want.dtype.itemsize}"))
        i = int(bad[0])
        raise AssertionError(
            f"{what}: {bad.size} of {got.size} elements differ; first at {i}: "
            f"got {got.reshape(-1)[i]!r} want {want.reshape(-1)[i]!r}")


def same_bits_nan_any(got: np.ndarray, want: np.ndarray, d: dt.DType, oracle, what=""):
    """Bit-exact except that any NaN matches any NaN (payload/sign of a NaN
    produced by arithmetic is not part of the contract)."""
    gv, wv = decode(got, d, oracle), decode(want, d, oracle)
    gn, wn = np.isnan(gv), np.isnan(wv)
    assert np.array_equal(gn, wn), f"{what}: NaN positions differ"
    g = np.where(gn, np.zeros_like(got), got)
    w = np.where(wn, np.zeros_like(want), want)
    same_bits(g, w, what)


def close(got: np.ndarray, want: np.ndarray, d: dt.DType, oracle, rel: float, abs_: float, what=""):
    gv, wv = decode(got, d, oracle), decode(want, d, oracle)
    assert gv.shape == wv.shape, (gv.shape, wv.shape)
    gn, wn = np.isnan(gv), np.isnan(wv)
    assert np.array_equal(gn, wn), f"{what}: NaN positions differ"
    inf = np.isinf(wv)
    assert np.array_equal(gv[inf], wv[inf]), f"{what}: infinities differ"
    ok = ~(gn | inf)
    err = np.abs(gv[ok] - wv[ok])
    lim = abs_ + rel * np.abs(wv[ok])
    if np.any(err > lim):
        i = int(np.argmax(err - lim))
        raise AssertionError(f"{what}: max excess at {i}: got {gv[ok][i]!r} want {wv[ok][i]!r} "
                             f"(rel {rel}, abs {abs_})")
