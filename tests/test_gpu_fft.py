"""fft / ifft / rfft / irfft on the GPU against the CPU oracle (double-precision
passes, one rounding per pass). Tolerances: the reference contract's
(backend_contract.ml:2827-2828, 2870-2876: rel = abs = 1e-9 for complex128, 1e-4
for complex64), and a tighter bound relative to the largest bin that both
double-precision pipelines meet with room."""

import numpy as np
import pytest

from helpers import logical
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu

COMPLEX = {"complex64": dt.complex64, "complex128": dt.complex128}
REAL_OF = {"complex64": dt.float32, "complex128": dt.float64}


def both(hip, oracle, a, d, build=None):
    a = np.ascontiguousarray(a.astype(d.np_storage))
    out = []
    for B in (hip, oracle):
        t = B.reshape(B.from_host(a, d), a.shape)
        out.append(build(B, t) if build else t)
    return out


def close(got, want, d, what):
    got, want = logical(got), logical(want)
    assert got.shape == want.shape and got.dtype == want.dtype, (what, got.shape, want.shape, got.dtype)
    if want.size == 0:
        return
    single = d in (dt.complex64, dt.float32)
    contract = 1e-4 if single else 1e-9
    diff = np.abs(got.astype(np.complex128) - want.astype(np.complex128))
    assert np.all(diff <= contract * (1 + np.abs(want))), (what, diff.max())
    tight = (2e-6 if single else 1e-11) * max(1.0, np.abs(want).max())
    assert diff.max() <= tight, (what, diff.max(), tight)


def cdata(rng, shape):
    return rng.standard_normal(shape) + 1j * rng.standard_normal(shape)


LENGTHS = [1, 2, 3, 4, 5, 7, 8, 16, 17, 31, 60, 64, 100, 143, 256, 1000, 1024, 2047, 2048, 4095, 4096, 4097, 8192]


@pytest.mark.parametrize("name", list(COMPLEX))
@pytest.mark.parametrize("n", LENGTHS)
def test_fft_and_ifft_lengths(hip, oracle, name, n):
    d = COMPLEX[name]
    rng = np.random.default_rng(n)
    h, o = both(hip, oracle, cdata(rng, (3, n)), d)
    close(hip.fft(h, [1]), oracle.fft(o, [1]), d, f"fft {n}")
    close(hip.ifft(h, [1]), oracle.ifft(o, [1]), d, f"ifft {n}")


@pytest.mark.parametrize("n", [16384, 65536, 1 << 20, 5000, 10007, 44100, 100000])
def test_long_transforms_through_the_workspace(hip, oracle, n):
    rng = np.random.default_rng(n)
    h, o = both(hip, oracle, cdata(rng, (2, n)), dt.complex128)
    close(hip.fft(h, [1]), oracle.fft(o, [1]), dt.complex128, f"fft {n}")
    close(hip.ifft(h, [1]), oracle.ifft(o, [1]), dt.complex128, f"ifft {n}")
    hr, orr = both(hip, oracle, rng.standard_normal((2, n)), dt.float32)
    close(hip.rfft(hr, dt.complex64, [1]), oracle.rfft(orr, dt.complex64, [1]), dt.complex64, f"rfft {n}")


def test_many_short_lines_and_strided_axes(hip, oracle):
    rng = np.random.default_rng(5)
    for shape, axis in (((4096, 8), 1), ((8, 4096), 0), ((300, 17, 5), 1), ((64, 64, 64), 0), ((5000, 3), 1)):
        h, o = both(hip, oracle, cdata(rng, shape), dt.complex64)
        close(hip.fft(h, [axis]), oracle.fft(o, [axis]), dt.complex64, f"{shape} axis {axis}")


def test_views_permuted_sliced_flipped_broadcast(hip, oracle):
    rng = np.random.default_rng(6)
    views = {
        "permuted": ((12, 17, 5), lambda B, t: B.permute(t, (2, 0, 1))),
        "sliced": ((20, 19, 6), lambda B, t: B.shrink(t, [(2, 19), (1, 18), (1, 5)])),  # the contract's strided case
        "flipped": ((9, 16, 3), lambda B, t: B.flip(t, (True, True, False))),
        "broadcast": ((1, 16, 1), lambda B, t: B.expand(t, (4, 16, 3))),
    }
    for name, (shape, build) in views.items():
        for d in (dt.complex64, dt.complex128):
            h, o = both(hip, oracle, cdata(rng, shape), d, build)
            for axes in ([1], [0, 2], [2, 1, 0]):
                close(hip.fft(h, axes), oracle.fft(o, axes), d, f"{name} {axes}")
                close(hip.ifft(h, axes), oracle.ifft(o, axes), d, f"{name} inverse {axes}")


def test_multi_axis_round_trip_scales_by_the_transformed_size(hip, oracle):
    rng = np.random.default_rng(7)
    a = cdata(rng, (6, 20, 9))
    h, o = both(hip, oracle, a, dt.complex128)
    back = hip.ifft(hip.fft(h, [0, 1, 2]), [0, 1, 2])
    assert np.max(np.abs(logical(back) - a * a.size)) <= 1e-9 * a.size
    close(hip.fft(h, []), o, dt.complex128, "no axes: a copy")


@pytest.mark.parametrize("name", list(COMPLEX))
def test_rfft_and_irfft(hip, oracle, name):
    c, r = COMPLEX[name], REAL_OF[name]
    rng = np.random.default_rng(8)
    for shape, axes in (((8,), [0]), ((7,), [0]), ((5, 12), [1]), ((5, 12), [0, 1]), ((6, 10, 9), [2, 0]),
                        ((4, 1000), [1]), ((3, 4096), [1]), ((2, 6000), [1])):
        h, o = both(hip, oracle, rng.standard_normal(shape), r)
        hs, os_ = hip.rfft(h, c, axes), oracle.rfft(o, c, axes)
        close(hs, os_, c, f"rfft {shape} {axes}")
        n = shape[axes[-1]]
        sizes = [shape[a] for a in axes]
        close(hip.irfft(hs, r, axes, sizes), oracle.irfft(os_, r, axes, sizes), r, f"irfft {shape} {axes}")
        if n % 2 == 0:
            close(hip.irfft(hs, r, axes), oracle.irfft(os_, r, axes), r, f"irfft inferred size {shape} {axes}")
        for other in (n - 3, n + 5):  # the half-spectrum is truncated / zero-padded (nx_c_fft.c:1036-1041)
            if other > 0:
                sizes[-1] = other
                close(hip.irfft(hs, r, axes, sizes), oracle.irfft(os_, r, axes, sizes), r, f"irfft to {other}")


def test_mixed_precisions_and_known_values(hip, oracle):
    ones = hip.from_host(np.ones(4, np.complex128), dt.complex128)
    assert np.array_equal(logical(hip.fft(ones, [0])), np.array([4, 0, 0, 0], np.complex128))
    delta = hip.from_host(np.array([1, 0, 0, 0], np.complex128), dt.complex128)
    assert np.array_equal(logical(hip.fft(delta, [0])), np.ones(4, np.complex128))
    spec = hip.from_host(np.ones(3, np.complex128), dt.complex128)
    r2 = np.sqrt(2.0)
    want = np.array([5, 1 + r2, -1, 1 - r2, 1, 1 - r2, -1, 1 + r2])
    assert np.max(np.abs(logical(hip.irfft(spec, dt.float64, [0], [8])) - want)) <= 1e-12
    rng = np.random.default_rng(9)
    h, o = both(hip, oracle, rng.standard_normal((3, 50)), dt.float32)
    close(hip.rfft(h, dt.complex128, [1]), oracle.rfft(o, dt.complex128, [1]), dt.complex128, "f32 -> complex128")
    h, o = both(hip, oracle, cdata(rng, (3, 26)), dt.complex128)
    close(hip.irfft(h, dt.float32, [1]), oracle.irfft(o, dt.float32, [1]), dt.float32, "complex128 -> f32")


def test_empty_and_rejected_arguments(hip, oracle):
    e = hip.reshape(hip.from_host(np.zeros(0, np.complex64), dt.complex64), (0, 8))
    assert logical(hip.fft(e, [1])).shape == (0, 8)
    x = hip.reshape(hip.from_host(np.zeros(8, np.float32), dt.float32), (2, 4))
    with pytest.raises(RuntimeError):
        hip.fft(x, [0])  # real input
    c = hip.reshape(hip.from_host(np.zeros(8, np.complex64), dt.complex64), (2, 4))
    with pytest.raises(ValueError):
        hip.fft(c, [2])
    with pytest.raises(ValueError):
        hip.rfft(x, dt.complex64, [])
    with pytest.raises(RuntimeError):
        hip.rfft(c, dt.complex64, [1])
