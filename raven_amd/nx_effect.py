"""The extended tier of the effect layer, as it behaves with no handler installed
(packages/nx/lib/effect/nx_effect.ml:22-41,320-376,559-572; named as optional for
a backend by packages/nx/lib/core/backend_intf.ml:69-76): ``const_scalar``,
``to_device``, ``psum`` and the ``Deferred`` tensor handle, over a device
backend.

On this backend a plain tensor already lives in device memory and a scalar is
filled from a kernel argument, so ``const_scalar`` costs no host round trip and
``to_device`` has work to do only between two contexts. ``Deferred`` keeps the
reference's meaning: a tensor of the given context whose bytes are still
somewhere else (a compiled program's output buffer, a file); metadata is
answered from the record and the first data access runs the fill function once.
"""

from __future__ import annotations

import itertools
from typing import Callable, Sequence

import numpy as np

from . import dtype as dt
from .view import View

_ids = itertools.count(1)


class Deferred:
    """nx_effect.ml:33-41: context, dtype and a C-contiguous view over the shape,
    a fill function that runs at most once, and the tensor it produced."""

    __slots__ = ("d_id", "context", "dtype", "_view", "_fill", "forced")

    def __init__(self, context, dtype: dt.DType, shape: Sequence[int], fill: Callable[[], np.ndarray]):
        self.d_id = next(_ids)
        self.context = context
        self.dtype = dtype
        self._view = View.create(tuple(int(s) for s in shape))
        self._fill = fill
        self.forced = None

    @property
    def view(self) -> View:
        return self.forced.view if self.forced is not None else self._view

    @property
    def shape(self):
        return self.view.shape


def deferred(context, dtype: dt.DType, shape: Sequence[int], fill: Callable[[], np.ndarray]) -> Deferred:
    """nx_effect.ml:351-363. ``fill`` returns the flat storage array of the dtype."""
    return Deferred(context, dtype, shape, fill)


def deferred_id(t):
    """The handle's id until it is forced, then None: its creator's side state
    (a resident buffer, say) is gone by then (nx_effect.ml:365-369)."""
    return t.d_id if isinstance(t, Deferred) and t.forced is None else None


def force(d: Deferred):
    """nx_effect.ml:329-341: run the fill once, wrap the bytes as a tensor of the
    recorded shape, remember it. Later writes through the remembered tensor are
    seen through the handle."""
    if d.forced is None:
        host = d._fill()
        d._fill = None
        d.forced = d.context.reshape(d.context.from_host(host, d.dtype), d._view.shape)
    return d.forced


def unwrap(t):
    return force(t) if isinstance(t, Deferred) else t


def context(t):
    return t.context


def view(t) -> View:
    return t.view


def dtype(t) -> dt.DType:
    return t.dtype


def to_host(t) -> np.ndarray:
    """nx_effect.ml:391-396."""
    u = unwrap(t)
    return u.context.to_host(u)


def const_scalar(context, value, dtype: dt.DType):
    """A rank-0 tensor holding ``value`` (nx_effect.ml:559-561)."""
    return context.full(dtype, (), value)


def full(context, dtype: dt.DType, shape: Sequence[int], value):
    """nx_effect.ml:563-573 without a handler: a concrete, writable tensor."""
    return context.full(dtype, tuple(shape), value)


def to_device(context, t):
    """``t`` as a tensor of ``context``. The reference has one memory and returns
    its argument (nx_effect.ml:376). Here a tensor of the same context is returned
    as it is; one of another context of this GPU is copied by a kernel of the
    target context, through its view, after the source context's stream has
    drained, and the target's stream is drained before returning so that the
    source may be released at once. A deferred tensor is forced first (its fill
    runs at most once, whoever asks)."""
    t = unwrap(t)
    if t.context is context:
        return t
    t.context.synchronize()
    out = context.buffer(t.dtype, t.shape)
    context.assign(out, context.with_view(_Foreign(t), t.view))
    context.synchronize()
    return out


class _Foreign:
    """Another context's tensor as an operand: same storage, same dtype."""

    __slots__ = ("buffer", "dtype")

    def __init__(self, t):
        self.buffer, self.dtype = t.buffer, t.dtype


def psum(t):
    """nx_effect.ml:477-479."""
    raise RuntimeError("psum must be used under vmap")
