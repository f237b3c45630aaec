"""The effect layer's extended tier with no handler installed
(packages/nx/lib/effect/nx_effect.ml:320-376,559-573): deferred handles,
const_scalar, to_device, psum."""

import numpy as np
import pytest

from helpers import logical, same_bits
from raven_amd import dtype as dt
from raven_amd import nx_effect as E


def test_a_deferred_handle_answers_metadata_without_filling_and_fills_once(oracle):
    calls = []

    def fill():
        calls.append(1)
        return np.arange(12, dtype=np.float32)

    oracle.context = oracle  # the host backend's tensors carry no context of their own
    d = E.deferred(oracle, dt.float32, (3, 4), fill)
    d2 = E.deferred(oracle, dt.float32, (3, 4), fill)
    assert E.deferred_id(d) is not None and E.deferred_id(d) != E.deferred_id(d2)
    assert E.view(d).shape == (3, 4) and E.view(d).is_c_contiguous() and E.dtype(d) is dt.float32
    assert E.context(d) is oracle and not calls
    t = E.unwrap(d)
    assert calls == [1] and t.shape == (3, 4)
    assert E.unwrap(d) is t and calls == [1]  # memoised
    assert E.deferred_id(d) is None  # forced: a plain tensor from now on
    # writes through the memoised tensor are seen through the handle
    oracle.assign(t, oracle.full(dt.float32, (3, 4), np.float32(7).reshape(1)))
    assert np.all(E.unwrap(d).storage == 7)
    with pytest.raises(RuntimeError, match="psum must be used under vmap"):
        E.psum(t)


@pytest.mark.gpu
def test_const_scalar_to_device_and_deferred_on_the_gpu(hip):
    from raven_amd.nx_backend import Backend

    s = E.const_scalar(hip, 2.5, dt.bfloat16)
    assert s.shape == () and s.context is hip
    same_bits(logical(s), np.asarray(0x4020, dtype=np.uint16))
    assert E.to_device(hip, s) is s

    other = Backend()
    try:
        x = np.arange(24 * 40, dtype=np.int32).reshape(24, 40)
        t = hip.permute(hip.shrink(hip.reshape(hip.from_host(x, dt.int32), x.shape), ((2, 20), (1, 39))), (1, 0))
        u = E.to_device(other, t)  # a strided view of one context becomes a compact tensor of the other
        assert u.context is other and u.buffer is not t.buffer and u.view.is_c_contiguous()
        same_bits(logical(u), x[2:20, 1:39].T)
        del t
        v = other.binary("add", u, u)
        same_bits(logical(v), 2 * x[2:20, 1:39].T)

        calls = []

        def fill():
            calls.append(1)
            return hip.to_host(hip.contiguous(hip.reshape(hip.from_host(x, dt.int32), x.shape)))

        d = E.deferred(hip, dt.int32, x.shape, fill)
        assert E.view(d).shape == x.shape and not calls
        moved = E.to_device(other, d)  # forced in its own context, then copied
        assert moved.context is other and calls == [1]
        same_bits(logical(moved), x)
        assert E.unwrap(d).context is hip and calls == [1]  # the fill ran once, whoever asked
        same_bits(E.to_host(E.deferred(hip, dt.int32, x.shape, fill)).reshape(x.shape), x)
    finally:
        del u, v, moved
        other.close()
