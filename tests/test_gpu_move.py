"""GPU parity of gather (bit-exact, any dtype) and its error rule, plus the
device buffer / transfer contract."""

import numpy as np
import pytest

from helpers import logical, pair, same_bits
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("d", [dt.uint8, dt.bfloat16, dt.float32, dt.float64, dt.complex128],
                         ids=lambda d: d.name)
def test_gather_matches_oracle(hip, oracle, d):
    rng = np.random.default_rng(1300 + d.tag)
    shape = (7, 11, 13)
    x = rng.integers(0, 255, shape + (d.itemsize,), dtype=np.uint8).view(d.np_storage).reshape(shape)
    for axis in (0, 1, 2):
        ishape = list(shape)
        ishape[axis] = 9
        idx = rng.integers(-shape[axis], shape[axis], ishape).astype(np.int32)  # negatives wrap once
        for dbuild in (None, lambda B, t: B.permute(t, (0, 1, 2))):
            (hd, od), (hi, oi) = pair(x, d, hip, oracle, dbuild), pair(idx, dt.int32, hip, oracle)
            same_bits(logical(hip.gather(hd, hi, axis)), logical(oracle.gather(od, oi, axis)))
    # strided data and a flipped index view
    xt = np.ascontiguousarray(np.transpose(x, (2, 0, 1)))
    (hd, od) = pair(xt, d, hip, oracle, lambda B, t: B.permute(t, (1, 2, 0)))
    idx = rng.integers(0, shape[1], (7, 5, 13)).astype(np.int32)
    (hi, oi) = pair(idx, dt.int32, hip, oracle, lambda B, t: B.flip(t, (False, True, False)))
    same_bits(logical(hip.gather(hd, hi, 1)), logical(oracle.gather(od, oi, 1)))


def test_gather_reference_vectors_and_embedding_path(hip, oracle):
    data = np.arange(12, dtype=np.float64).reshape(3, 4)  # backend_contract.ml:1690-1727
    hd, _ = pair(data, dt.float64, hip, oracle)
    hi, _ = pair(np.array([[3, 0], [1, 3], [0, 2]], np.int32), dt.int32, hip, oracle)
    assert logical(hip.gather(hd, hi, 1)).tolist() == [[3.0, 0.0], [5.0, 7.0], [8.0, 10.0]]
    hi, _ = pair(np.array([[2, 0, 1, 2], [0, 1, 2, 0]], np.int32), dt.int32, hip, oracle)
    assert logical(hip.gather(hd, hi, 0)).tolist() == [[8.0, 1.0, 6.0, 11.0], [0.0, 5.0, 10.0, 3.0]]
    # Embedding lookup: table [V, D], ids broadcast along D (kaun/lib/embedding.ml:31-36)
    rng = np.random.default_rng(16)
    for d, D in ((dt.bfloat16, 768), (dt.float32, 100), (dt.uint8, 7)):
        table = rng.integers(0, 2 ** 15, (5000, D)).astype(d.np_storage)
        ids = rng.integers(-5000, 5000, 3000).astype(np.int32)
        ht, ot = pair(table, d, hip, oracle)
        hi, oi = pair(ids, dt.int32, hip, oracle, lambda B, t: B.expand(B.reshape(t, (3000, 1)), (3000, D)))
        got = logical(hip.gather(ht, hi, 0))
        assert hip.last_path() == "gather_rows"
        same_bits(got, logical(oracle.gather(ot, oi, 0)))
        same_bits(got, table[ids])


def test_gather_out_of_bounds_is_a_failure_of_that_call(hip, oracle):
    hd, _ = pair(np.arange(12, dtype=np.float32).reshape(3, 4), dt.float32, hip, oracle)
    for bad in (4, -5, 2 ** 31 - 1):
        hi, _ = pair(np.array([[0, bad]], np.int32), dt.int32, hip, oracle)
        with pytest.raises(RuntimeError, match="index out of bounds"):
            hip.gather(hd, hi, 1)
    # the flag is cleared: the next call succeeds
    hi, _ = pair(np.array([[0, -1]], np.int32), dt.int32, hip, oracle)
    assert logical(hip.gather(hd, hi, 1)).tolist() == [[0.0, 3.0]]
    hi, _ = pair(np.full((300, 4), 3, np.int32), dt.int32, hip, oracle,
                 lambda B, t: B.expand(B.shrink(t, [(0, 300), (0, 1)]), (300, 4)))
    with pytest.raises(RuntimeError, match="index out of bounds"):
        hip.gather(hd, hi, 0)
    with pytest.raises(ValueError):
        hip.gather(hd, hi, 2)


def test_buffers_views_and_transfer(hip, oracle):
    x = np.arange(24, dtype=np.float32)
    t = hip.reshape(hip.from_host(x, dt.float32), (2, 3, 4))
    x[:] = -1  # from_host has already copied
    v = hip.shrink(hip.permute(t, (2, 0, 1)), [(1, 3), (0, 2), (1, 3)])
    # to_host returns the WHOLE backing storage; the view indexes into it
    storage = hip.to_host(v)
    assert storage.shape == (24,) and storage[v.offset] == 1 * 1 + 0 * 12 + 1 * 4
    assert np.array_equal(logical(v), np.arange(24, dtype=np.float32).reshape(2, 3, 4).transpose(2, 0, 1)[1:3, :, 1:3])
    # views share storage: assign through one is seen through the other
    hip.assign(hip.shrink(t, [(0, 1), (0, 3), (0, 4)]), hip.full(dt.float32, (1, 3, 4), 7.0))
    assert np.all(logical(t)[0] == 7.0) and np.all(logical(t)[1].reshape(-1) == np.arange(12, 24))
    # allocator: freed blocks are reused, never handed out twice while live
    before = hip.memory_stats()
    a = hip.buffer(dt.float32, (1000,))
    pa = a.buffer.ptr
    del a
    b = hip.buffer(dt.float32, (1000,))
    c = hip.buffer(dt.float32, (1000,))
    assert b.buffer.ptr == pa and c.buffer.ptr != pa
    assert hip.memory_stats()["driver_allocs"] <= before["driver_allocs"] + 2
    info = hip.device_info()
    assert "gfx950" in info["name"] and info["compute_units"] >= 200
