"""The slice of the Nx frontend that the GPT-2 forward needs, restated over a
backend object (``raven_amd.nx_backend.Backend`` on the GPU, or the CPU oracle's
``OracleBackend`` in tests): every function lowers to the same sequence of
backend primitives as packages/nx/lib/core/frontend.ml does, so a model built
from these calls issues the reference's op mix, one backend call per primitive.

Nothing here computes: shapes are checked, views are built, and the backend is
called. Citations are to packages/nx/lib/core/frontend.ml unless noted.
"""

from __future__ import annotations

from typing import Sequence

import numpy as np

from . import dtype as dt
from .nx_backend import encode_scalar


def _broadcast_shapes(a: Sequence[int], b: Sequence[int]) -> tuple:
    if tuple(a) == tuple(b):
        return tuple(a)
    n = max(len(a), len(b))
    out = []
    for i in range(n):
        x = a[i - (n - len(a))] if i >= n - len(a) else 1
        y = b[i - (n - len(b))] if i >= n - len(b) else 1
        if x != y and x != 1 and y != 1:
            raise ValueError(f"broadcast: cannot broadcast {tuple(a)} with {tuple(b)}")
        out.append(max(x, y) if min(x, y) != 0 else 0)
    return tuple(out)


_ENCODED: dict = {}  # (dtype name, Python value) -> its encoded storage element


class Nx:
    """Frontend functions bound to one backend."""

    def __init__(self, backend):
        self.B = backend

    # ── creation ────────────────────────────────────────────────────────────
    def create(self, dtype: dt.DType, shape, host: np.ndarray):
        """frontend.ml:342-353: fill a host buffer, ``from_host``, reshape."""
        return self.B.reshape(self.B.from_host(np.ascontiguousarray(host), dtype), tuple(shape))

    def scalar(self, dtype: dt.DType, value):
        """frontend.ml:360: ``B.full ctx dt [||] value``."""
        key = (dtype.name, value)
        enc = _ENCODED.get(key)
        if enc is None:
            enc = encode_scalar(dtype, value)
            enc.setflags(write=False)
            if len(_ENCODED) < 1024 and value == value:  # a NaN never equals its own key
                _ENCODED[key] = enc
        return self.B.full(dtype, (), enc)

    def scalar_like(self, x, value):
        return self.scalar(x.dtype, value)

    def arange(self, dtype: dt.DType, start: int, stop: int, step: int = 1):
        """frontend.ml:1246-1290: values are produced on the host."""
        return self.create(dtype, (len(range(start, stop, step)),),
                           np.arange(start, stop, step).astype(dtype.np_storage))

    # ── views ───────────────────────────────────────────────────────────────
    def reshape(self, shape, x):
        return self.B.reshape(x, tuple(shape))

    def broadcast_to(self, shape, x):
        shape = tuple(shape)
        if tuple(x.shape) == shape:
            return x
        pad = len(shape) - len(x.shape)
        if pad > 0 and len(x.shape) > 0:  # a rank-0 view expands to any rank directly (view.ml expand)
            x = self.B.reshape(x, (1,) * pad + tuple(x.shape))
        return self.B.expand(x, shape)

    def broadcasted(self, a, b):
        """frontend.ml:293-296."""
        if a.shape == b.shape:
            return a, b
        s = _broadcast_shapes(a.shape, b.shape)
        return self.broadcast_to(s, a), self.broadcast_to(s, b)

    def swapaxes(self, a1: int, a2: int, x):
        """frontend.ml:981-993."""
        r = len(x.shape)
        a1, a2 = a1 % r, a2 % r
        if a1 == a2:
            return x
        axes = list(range(r))
        axes[a1], axes[a2] = a2, a1
        return self.B.permute(x, axes)

    def transpose(self, x):
        return self.B.permute(x, list(range(len(x.shape)))[::-1])

    def contiguous(self, x):
        return self.B.contiguous(x)

    # ── elementwise (frontend.ml:417-534) ───────────────────────────────────
    def _binop(self, op, a, b):
        a, b = self.broadcasted(a, b)
        return self.B.binary(op, a, b)

    def add(self, a, b):
        return self._binop("add", a, b)

    def sub(self, a, b):
        return self._binop("sub", a, b)

    def mul(self, a, b):
        return self._binop("mul", a, b)

    def div(self, a, b):
        return self._binop("idiv" if a.dtype.is_int else "fdiv", a, b)

    def add_s(self, x, s):
        return self.add(x, self.scalar_like(x, s))

    def mul_s(self, x, s):
        return self.mul(x, self.scalar_like(x, s))

    def less_equal(self, a, b):
        a, b = self.broadcasted(a, b)
        return self.B.compare("cmple", a, b)

    def where(self, cond, if_true, if_false):
        """frontend.ml:612-618."""
        s = _broadcast_shapes(_broadcast_shapes(if_true.shape, if_false.shape), cond.shape)
        return self.B.where(self.broadcast_to(s, cond), self.broadcast_to(s, if_true),
                            self.broadcast_to(s, if_false))

    def sqrt(self, x):
        return self.B.unary("sqrt", x)

    def exp(self, x):
        return self.B.unary("exp", x)

    def tanh(self, x):
        return self.B.unary("tanh", x)

    def cast(self, dtype: dt.DType, x):
        """frontend.ml:324-328: a cast to the same dtype is the identity."""
        return x if x.dtype is dtype else self.B.cast(x, dtype)

    # ── reductions (frontend.ml:642-708) ────────────────────────────────────
    def _reduce(self, op, x, axes, keepdims):
        r = len(x.shape)
        axes = sorted(a % r for a in axes)
        out = self.B.reduce(op, axes, x)
        if keepdims:
            out = self.B.reshape(out, tuple(1 if i in axes else s for i, s in enumerate(x.shape)))
        return out

    def sum(self, x, axes, keepdims=False):
        return self._reduce("sum", x, axes, keepdims)

    def max(self, x, axes, keepdims=False):
        return self._reduce("max", x, axes, keepdims)

    def mean(self, x, axes, keepdims=False):
        """frontend.ml:698-707: sum, then divide by a broadcast scalar."""
        s = self.sum(x, axes, keepdims)
        n = 1
        for a in axes:
            n *= x.shape[a % len(x.shape)]
        divisor = self.broadcast_to(s.shape, self.scalar(x.dtype, float(max(1, n))))
        return self.div(s, divisor)

    def softmax(self, x, axes=(-1,)):
        """frontend.ml:4242-4252 with scale = 1."""
        max_x = self.max(x, axes, keepdims=True)
        e = self.exp(self.sub(x, max_x))
        return self.div(e, self.sum(e, axes, keepdims=True))

    # ── indexing / contraction ──────────────────────────────────────────────
    def take(self, table, indices, axis=0):
        """frontend.ml:1410-1435, mode `raise: a gather with the flattened
        indices broadcast across the other axes of ``table``."""
        tshape = list(table.shape)
        n_idx = 1
        for s in indices.shape:
            n_idx *= s
        flat = self.B.reshape(indices, (n_idx,))
        expanded = [n_idx if i == axis else 1 for i in range(len(tshape))]
        target = list(tshape)
        target[axis] = n_idx
        idx = self.broadcast_to(target, self.B.reshape(flat, expanded))
        return self.B.gather(table, idx, axis)

    def matmul(self, a, b):
        """frontend.ml:2346-2352 for operands of rank >= 2."""
        if len(a.shape) < 2 or len(b.shape) < 2:
            raise ValueError("matmul: this mirror covers operands of rank >= 2")
        if a.shape[-1] != b.shape[-2]:
            raise ValueError(f"dot: cannot contract {tuple(a.shape)} to {tuple(b.shape)}")
        return self.B.matmul(a, b)

