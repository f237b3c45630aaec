"""The limits this backend has and the reference does not (sort axis 2^30, transform length
2^26 / 2^25, eigh / svd 4096 rows, eig 2048): each one refused with its
message one step beyond it, before anything is launched, and the cheap ones exercised
exactly at it. Results at the limit are checked through closed forms (a shifted impulse's
spectrum, the counts of a sorted byte array), not against the oracle, whose run times at
these sizes are minutes."""

import numpy as np
import pytest

from helpers import logical, same_bits
from raven_amd import dtype as dt
from raven_amd.nx_frontend import Nx

pytestmark = pytest.mark.gpu


def test_sort_axis_at_and_beyond_2_to_30(hip):
    n = 1 << 30
    rng = np.random.default_rng(30)
    host = rng.integers(0, 256, n + 1, dtype=np.uint8)
    x = hip.reshape(hip.from_host(host, dt.uint8), (n + 1,))
    with pytest.raises(RuntimeError, match="2\\^30"):
        hip.sort(x, 0, False)
    with pytest.raises(RuntimeError, match="INT32_MAX"):
        hip.argsort(x, 0, False)
    at = hip.shrink(x, [(1, n + 1)])  # exactly 2^30 elements, from an odd offset
    got = logical(hip.sort(at, 0, True))
    del x, at
    hip.trim()
    counts = np.bincount(host[1:], minlength=256)
    assert np.all(got[:-1] >= got[1:]), "descending order"
    assert np.array_equal(np.bincount(got, minlength=256), counts), "a permutation of the input"


def test_transform_length_at_and_beyond_the_limit(hip):
    n = 1 << 26
    for length, message in ((n + 2, "2\\^26"), ((1 << 25) + 1, "2\\^25")):
        z = hip.full(dt.complex64, (length,), 0.0)
        with pytest.raises(RuntimeError, match=message):
            hip.fft(z, [0])
        del z
    # exactly 2^26: impulses at p and q, x = d_p + 2 d_q, so X[k] = w^(k p) + 2 w^(k q), w = exp(-2 pi i / n)
    p, q = 12345, 40000001
    host = np.zeros(n, np.complex64)
    host[p], host[q] = 1.0, 2.0
    x = hip.reshape(hip.from_host(host, dt.complex64), (n,))
    got = logical(hip.fft(x, [0]))
    del x
    hip.trim()
    k = np.unique(np.concatenate([np.arange(0, 4096), np.random.default_rng(26).integers(0, n, 1 << 16), [n - 1]]))
    phase = lambda pos: np.exp(-2j * np.pi * ((k * pos) % n) / n)  # noqa: E731  (k * pos fits int64)
    want = phase(p) + 2 * phase(q)
    assert np.max(np.abs(got[k] - want)) <= 1e-5, float(np.max(np.abs(got[k] - want)))
    assert abs(float(np.sum(np.abs(got.astype(np.complex128)) ** 2)) / n - 5.0) <= 1e-3  # Parseval: |x|^2 = 5


def test_factorisations_refuse_what_they_cannot_hold(hip):
    big = hip.full(dt.float32, (4097, 4097), 0.0)
    for call in (hip.eigh, hip.eigvalsh, hip.svd):
        with pytest.raises(RuntimeError, match="limit is 4096"):
            call(big)
    del big
    mid = hip.full(dt.float32, (2049, 2049), 0.0)
    for call in (hip.eig, hip.eigvals):
        with pytest.raises(RuntimeError, match="limit is 2048"):
            call(mid)
    del mid
    hip.trim()


@pytest.mark.parametrize("row", [8192, 8193, 50257])
def test_fused_rows_at_and_beyond_what_a_block_holds(hip, row):
    """softmax over rows of 8192 elements is one fused kernel with the row in registers; a longer
    row is still one fused kernel, which walks it three times. Both agree with the eager sequence
    within the sum's reassociation."""
    rng = np.random.default_rng(row)
    nx = Nx(hip)
    x = hip.reshape(hip.from_host(rng.standard_normal((24, row)).astype(np.float32), dt.float32), (24, row))
    eager = logical(nx.softmax(x))
    hip.set_deferred(True)
    try:
        before = hip.deferred_stats()
        got = logical(nx.softmax(x))
        after = hip.deferred_stats()
    finally:
        hip.set_deferred(False)
    s = {k: after[k] - before[k] for k in after}
    assert s["softmax_rows"] == 1 and s["issued"] == 0, s
    assert np.allclose(got, eager, rtol=4e-6, atol=1e-9)
    assert np.allclose(got.sum(-1), 1.0, atol=1e-5)
