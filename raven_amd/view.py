"""Strided view algebra: shape, element strides and element offset.

Mirrors ``Nx_core.View`` (packages/nx/lib/core/view.ml:43-322): every movement
operation is metadata only; ``reshape`` never copies and raises when the
strides cannot express the new shape. Errors are ``ValueError``, the Python
counterpart of OCaml's ``Invalid_argument``.
"""

from __future__ import annotations

from typing import Sequence, Tuple


def c_contiguous_strides(shape: Sequence[int]) -> Tuple[int, ...]:
    strides = [0] * len(shape)
    acc = 1
    for i in range(len(shape) - 1, -1, -1):
        strides[i] = acc
        acc *= max(shape[i], 1) if shape[i] == 0 else shape[i]
    # Shape.c_contiguous_strides gives 0-size dims the stride of a size-1 dim.
    return tuple(strides)


def numel(shape: Sequence[int]) -> int:
    n = 1
    for s in shape:
        n *= s
    return n


_CONTIGUOUS: dict = {}  # shape -> its C-contiguous, offset-0 view (views are immutable)


class View:
    """Immutable by convention: every operation returns a new view."""

    __slots__ = ("shape", "strides", "offset")

    def __init__(self, shape: Tuple[int, ...], strides: Tuple[int, ...], offset: int = 0):
        self.shape = shape
        self.strides = strides
        self.offset = offset

    def __eq__(self, other):
        return (isinstance(other, View) and self.shape == other.shape and self.strides == other.strides
                and self.offset == other.offset)

    def __hash__(self):
        return hash((self.shape, self.strides, self.offset))

    def __repr__(self):  # pragma: no cover
        return f"View(shape={self.shape}, strides={self.strides}, offset={self.offset})"

    # -- construction (view.ml:43-78) -------------------------------------
    @staticmethod
    def create(shape, strides=None, offset=0) -> "View":
        shape = tuple([int(s) for s in shape])
        if strides is None:
            if offset == 0 or 0 in shape:
                v = _CONTIGUOUS.get(shape)
                if v is None:
                    v = View(shape, c_contiguous_strides(shape), 0)
                    if len(_CONTIGUOUS) < 4096:
                        _CONTIGUOUS[shape] = v
                return v
            strides = c_contiguous_strides(shape)
        else:
            strides = tuple([int(s) for s in strides])
            if len(strides) != len(shape):
                raise ValueError(
                    f"create: strides length {len(strides)} != shape length {len(shape)}")
        if 0 in shape:
            offset = 0
        return View(shape, strides, int(offset))

    @property
    def ndim(self) -> int:
        return len(self.shape)

    @property
    def numel(self) -> int:
        return numel(self.shape)

    def is_c_contiguous(self) -> bool:
        """Row-major strides, ignoring size-1 dims (view.ml:20-41)."""
        expect = 1
        for s, st in zip(reversed(self.shape), reversed(self.strides)):
            if s == 0:
                return True
            if s != 1 and st != expect:
                return False
            expect *= s
        return True

    # -- movement (view.ml:82-322) ----------------------------------------
    def expand(self, new_shape) -> "View":
        new_shape = tuple(int(s) for s in new_shape)
        if self.ndim == 0:
            return View(new_shape, (0,) * len(new_shape), self.offset)
        if len(new_shape) != self.ndim:
            raise ValueError(f"expand: rank mismatch: {len(new_shape)} vs {self.ndim}")
        if any(s == 0 for s in self.shape):
            return View.create(new_shape)
        strides = []
        for i, ns in enumerate(new_shape):
            s = self.shape[i]
            if s == ns:
                strides.append(self.strides[i])
            elif s == 1:
                strides.append(0)
            else:
                raise ValueError(
                    f"expand: dimension {i} (size {s}) cannot expand to size {ns}, "
                    "only singletons expand")
        return View.create(new_shape, strides, self.offset)

    def permute(self, axes) -> "View":
        axes = tuple(int(a) for a in axes)
        n = self.ndim
        if len(axes) != n:
            raise ValueError(f"permute: axes length {len(axes)} != ndim {n}")
        seen = [False] * n
        for ax in axes:
            if ax < 0 or ax >= n:
                raise ValueError(f"permute: axis {ax} out of bounds for {n}D tensor")
            if seen[ax]:
                raise ValueError(f"permute: duplicate axis {ax}")
            seen[ax] = True
        return View.create([self.shape[a] for a in axes],
                           [self.strides[a] for a in axes], self.offset)

    def shrink(self, bounds) -> "View":
        bounds = [(int(b), int(e)) for b, e in bounds]
        if len(bounds) != self.ndim:
            raise ValueError(f"shrink: bounds length {len(bounds)} != ndim {self.ndim}")
        if all(b == 0 and e == s for (b, e), s in zip(bounds, self.shape)):
            return self
        for (b, e), s in zip(bounds, self.shape):
            if b < 0 or e < 0 or b > s or e > s or b >= e:
                raise ValueError("shrink: bounds must be within shape and start < end")
        off = self.offset + sum(b * st for (b, _), st in zip(bounds, self.strides))
        return View.create([e - b for b, e in bounds], self.strides, off)

    def flip(self, flags) -> "View":
        flags = [bool(f) for f in flags]
        if len(flags) != self.ndim:
            raise ValueError(f"flip: boolean array length {len(flags)} != ndim {self.ndim}")
        off = self.offset
        strides = list(self.strides)
        for i, f in enumerate(flags):
            if f and self.shape[i] > 0:
                off += (self.shape[i] - 1) * self.strides[i]
                strides[i] = -strides[i]
        return View.create(self.shape, strides, off)

    def reshape(self, new_shape) -> "View":
        new_shape = tuple(int(s) for s in new_shape)
        if new_shape == self.shape:
            return self
        old_n, new_n = numel(self.shape), numel(new_shape)
        if old_n != new_n and old_n != 0 and new_n != 0:
            raise ValueError(f"reshape: cannot reshape {list(self.shape)} to {list(new_shape)}")
        if 0 in self.shape or 0 in new_shape:
            return View.create(new_shape, offset=0)
        if self.strides == c_contiguous_strides(self.shape) or self.is_c_contiguous():
            return View.create(new_shape, offset=self.offset)
        if len(new_shape) == 0:
            return View.create(new_shape, offset=self.offset)
        if all(s == 0 for s in self.strides):
            return View.create(new_shape, (0,) * len(new_shape), self.offset)
        # squeeze / unsqueeze of size-1 dims only
        old_non1 = [(s, st) for s, st in zip(self.shape, self.strides) if s != 1]
        new_non1 = [s for s in new_shape if s != 1]
        if [s for s, _ in old_non1] == new_non1:
            it = iter(old_non1)
            strides = [0 if s == 1 else next(it)[1] for s in new_shape]
            return View.create(new_shape, strides, self.offset)
        strides = _merge_split(old_non1, new_non1)
        if strides is None:
            raise ValueError(
                f"reshape: cannot reshape {list(self.shape)} to {list(new_shape)}, "
                f"incompatible strides {list(self.strides)} "
                f"(expected {list(c_contiguous_strides(new_shape))}), call contiguous() first")
        it = iter(strides)
        full = [0 if s == 1 else next(it) for s in new_shape]
        return View.create(new_shape, full, self.offset)


def _merge_split(old_dims, new_dims):
    """Strides for ``new_dims`` when each is a split of one old dim or a merge of
    adjacent old dims that compose (view.ml:203-265); None if impossible."""
    old = list(old_dims)
    out = []
    i = 0
    for ns in new_dims:
        if i >= len(old):
            return None
        size, stride = old[i]
        if size == ns:
            out.append(stride)
            i += 1
        elif size > ns and size % ns == 0:
            rem = size // ns
            out.append(stride * rem)
            old[i] = (rem, stride)
        elif ns > size:
            acc, st = size, stride
            j = i + 1
            while acc < ns:
                if j >= len(old):
                    return None
                nsize, nstride = old[j]
                if st != nstride * nsize:
                    return None
                acc *= nsize
                st = nstride
                j += 1
            if acc != ns:
                return None
            out.append(st)
            i = j
        else:
            return None
    if i != len(old):
        return None
    return out
