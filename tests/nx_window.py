"""A deferred-evaluation window in front of a backend: the host-side twin of the library's
own deferred mode (nxh_set_deferred), kept as its cross-check. No binding uses it.

The frontend lowers softmax, layer norm and GELU to a dozen primitives each
(packages/nx/lib/core/frontend.ml:4242-4252, packages/kaun/lib/layer_norm.ml:43-68,
packages/kaun/lib/fn.ml:31-38, packages/kaun/lib/attention.ml:93-108), and an
eager backend makes one pass over memory per primitive. ``Window`` exposes the
same operations as the backend it wraps but only *records* the elementwise
primitives, casts and reductions. The record is executed, in issue order, as
soon as anything else is asked of the backend (any other operation on a tensor,
a host read, a synchronisation) or when it grows past ``limit`` entries. At
that point runs of entries that spell one of the three sequences, and whose
intermediate results nobody can observe any more (every handle to them has
been dropped and their only readers are inside the run), are replaced by one
call of the backend's fused operation; everything else is issued as recorded.

What a caller can observe is unchanged except for two things: an error of a
recorded primitive surfaces when the record is executed rather than at the
call, and a fused float result may differ from the op-by-op one by the order
in which a row's sum is added (every elementwise step is rounded identically).

Handles: a ``WTensor`` is a view over a ``Cell``; the cell holds either the
backend's tensor or the record entry that will produce it. Dropping the last
handle of a pending cell is what makes an intermediate unobservable; the
reference's binding learns the same from its custom-block finalisers
(nx_backend.ml:36-43 keeps one buffer per handle), only later, so there the
window would be executed with more intermediates still alive.
"""

from __future__ import annotations

import weakref
from typing import List, Optional, Sequence

import numpy as np

from raven_amd import dtype as dt
from raven_amd.view import View, c_contiguous_strides, numel

FUSED_FLOATS = ("float16", "bfloat16", "float32", "float64")
ISLAND = ("float16", "bfloat16")  # dtypes whose layer-norm statistics run in float32
MAX_ROW = 1 << 24


class Entry:
    """One recorded primitive."""

    __slots__ = ("kind", "op", "ins", "shape", "dtype", "axes", "cell", "alive", "result", "readers", "fused_into",
                 "value", "tag", "wanted", "__weakref__")

    def __init__(self, kind, op, ins, shape, dtype, axes=None):
        self.kind, self.op, self.ins = kind, op, ins
        self.shape, self.dtype, self.axes = tuple(shape), dtype, axes
        self.cell = None       # weakref to the Cell that will receive the result
        self.alive = True      # False once every handle to the result is gone
        self.result = None     # backend tensor once executed
        self.readers = []      # entries of the window that read this one
        self.fused_into = None
        self.value = None      # kind "full": the encoded element
        self.tag = None        # what is known about the result's contents (("causal", n))
        self.wanted = False    # a caller asked for the result itself (force)


class Operand:
    """An input of an entry: a pending entry or a backend tensor, seen through a view."""

    __slots__ = ("entry", "root", "view", "scalar", "tag")

    def __init__(self, entry, root, view, scalar, tag=None):
        self.entry, self.root, self.view, self.scalar, self.tag = entry, root, view, scalar, tag

    def same(self, other: "Operand") -> bool:
        return self.entry is other.entry and self.root is other.root and self.view == other.view


class Cell:
    """Storage shared by the views of one tensor: the backend's tensor (`root`)
    or the entry that will produce it, plus what the window knows about the
    contents: `scalar` (the encoded element of a one-element full), `host` (a
    small int32 array uploaded with from_host), `tag` (see Entry.tag)."""

    __slots__ = ("root", "entry", "scalar", "host", "tag", "__weakref__")

    def __init__(self, root=None, entry=None, scalar=None, host=None):
        self.root, self.entry, self.scalar, self.host, self.tag = root, entry, scalar, host, None

    def __del__(self):
        e = self.entry
        if e is not None:
            e.alive = False


class WTensor:
    """The window's tensor handle."""

    __slots__ = ("cell", "view", "dtype", "context")

    def __init__(self, cell: Cell, view: View, dtype: dt.DType, context: "Window"):
        self.cell, self.view, self.dtype, self.context = cell, view, dtype, context

    @property
    def shape(self):
        return self.view.shape

    @property
    def strides(self):
        return self.view.strides

    @property
    def offset(self):
        return self.view.offset


def _encode(dtype, value):
    from .nx_backend import encode_scalar

    return encode_scalar(dtype, value)


def _identity(view: View, shape) -> bool:
    return view.offset == 0 and view.shape == tuple(shape) and view.is_c_contiguous()


def _row_broadcast(view: View, shape) -> bool:
    """A keepdims result [..., 1] expanded along the last axis to ``shape``."""
    shape = tuple(shape)
    if view.shape != shape or view.offset != 0 or not shape:
        return False
    if shape[-1] != 1 and view.strides[-1] != 0:
        return False
    outer = c_contiguous_strides(shape[:-1])
    return all(s == 1 or a == b for s, a, b in zip(shape[:-1], view.strides[:-1], outer))


def _all_broadcast(view: View) -> bool:
    return view.offset == 0 and all(s == 1 or st == 0 for s, st in zip(view.shape, view.strides))


def _vector_broadcast(view: View, shape) -> bool:
    """A rank-1 tensor of the row length broadcast over the outer dims."""
    shape = tuple(shape)
    return (view.shape == shape and view.offset == 0 and (shape[-1] == 1 or view.strides[-1] == 1)
            and all(s == 1 or st == 0 for s, st in zip(shape[:-1], view.strides[:-1])))


def _causal_length(op, x: "WTensor", y: "WTensor"):
    """n if ``compare op x y`` is the n x n causal mask of attention.ml:236-243:
    cmple of arange(n) along the columns against arange(n) down the rows, so
    that element [i][j] is (j <= i)."""
    if op != "cmple" or len(x.shape) != 2 or x.shape[0] != x.shape[1]:
        return None
    n = x.shape[0]
    hx, hy = x.cell.host, y.cell.host
    if hx is None or hy is None or hx.size != n or hy.size != n:
        return None
    if (x.view.offset, y.view.offset) != (0, 0) or x.view.strides != (0, 1) or y.view.strides != (1, 0):
        return None
    ar = np.arange(n)
    return n if np.array_equal(hx, ar) and np.array_equal(hy, ar) else None


class Window:
    """``Window(backend)``: same operations, deferred as described above."""

    DEFERRED = ("unary", "binary", "where", "cast", "reduce", "compare", "matmul")

    def __init__(self, backend, limit: int = 512, fuse: bool = True):
        self.B = backend
        self.limit = limit
        self.fuse = fuse
        self.entries: List[Entry] = []
        self.stats = {"recorded": 0, "issued": 0, "softmax_rows": 0, "layer_norm_rows": 0, "gelu_tanh": 0,
                      "attention": 0, "linear": 0, "flushes": 0, "fallbacks": 0}

    # ── handles ─────────────────────────────────────────────────────────────
    def _wrap(self, t, scalar=None) -> WTensor:
        return WTensor(Cell(root=t, scalar=scalar), t.view, t.dtype, self)

    def _is_base_tensor(self, x) -> bool:
        return hasattr(x, "view") and hasattr(x, "dtype") and not isinstance(x, WTensor)

    def force(self, t: WTensor):
        """The backend's tensor for ``t`` (executes the record if ``t`` is pending)."""
        if t.cell.root is None:
            t.cell.entry.wanted = True
            self.flush()
        return self.B.with_view(t.cell.root, t.view)

    def _operand(self, t: WTensor) -> Operand:
        c = t.cell
        if c.root is None:
            return Operand(c.entry, None, t.view, c.scalar, c.entry.tag)
        return Operand(None, c.root, t.view, c.scalar, c.tag)

    def _record(self, kind, op, ins: Sequence[WTensor], shape, dtype, axes=None) -> WTensor:
        e = Entry(kind, op, [self._operand(t) for t in ins], shape, dtype, axes)
        for o in e.ins:
            if o.entry is not None:
                o.entry.readers.append(e)
        cell = Cell(entry=e)
        e.cell = weakref.ref(cell)
        self.entries.append(e)
        self.stats["recorded"] += 1
        out = WTensor(cell, View.create(shape), dtype, self)
        if len(self.entries) >= self.limit:
            self.flush()
        return out

    # ── recorded primitives ─────────────────────────────────────────────────
    @staticmethod
    def _same_shape(op, *ts):
        for t in ts[1:]:
            if tuple(t.shape) != tuple(ts[0].shape):
                raise ValueError(f"{op}: shape mismatch")

    def unary(self, op, x):
        return self._record("unary", op, [x], x.shape, x.dtype)

    def binary(self, op, x, y):
        self._same_shape(op, x, y)
        return self._record("binary", op, [x, y], x.shape, x.dtype)

    def where(self, cond, a, b):
        self._same_shape("where", cond, a, b)
        return self._record("where", None, [cond, a, b], a.shape, a.dtype)

    def cast(self, x, dtype):
        return self._record("cast", None, [x], x.shape, dtype)

    def compare(self, op, x, y):
        self._same_shape(op, x, y)
        out = self._record("compare", op, [x, y], x.shape, dt.bool_)
        n = _causal_length(op, x, y)
        if n is not None and out.cell.entry is not None:
            out.cell.entry.tag = ("causal", n)
        elif n is not None:
            out.cell.tag = ("causal", n)
        return out

    def matmul(self, x, y):
        xs, ys = tuple(x.shape), tuple(y.shape)
        if len(xs) < 2 or len(ys) < 2 or xs[-1] != ys[-2] or x.dtype is not y.dtype:
            self.flush()  # let the backend phrase the error
            return self._lift(self.B.matmul(self.force(x), self.force(y)))
        nd = max(len(xs), len(ys))
        batch = []
        for i in range(nd - 2):
            ai, bi = i - (nd - len(xs)), i - (nd - len(ys))
            a, b = (xs[ai] if ai >= 0 else 1), (ys[bi] if bi >= 0 else 1)
            if a != b and a != 1 and b != 1:
                self.flush()
                return self._lift(self.B.matmul(self.force(x), self.force(y)))
            batch.append(max(a, b) if min(a, b) != 0 else 0)
        return self._record("matmul", None, [x, y], tuple(batch) + (xs[-2], ys[-1]), x.dtype)

    def reduce(self, op, axes, x):
        axes = sorted(int(a) for a in axes)
        if any(a < 0 or a >= len(x.shape) for a in axes) or len(set(axes)) != len(axes):
            raise ValueError(f"reduce_{op}: axes out of range")
        if op in ("max", "min") and any(x.shape[a] == 0 for a in axes):
            raise ValueError(f"reduce_{op}: reduction over an empty axis has no identity")
        shape = [s for i, s in enumerate(x.shape) if i not in axes]
        return self._record("reduce", op, [x], shape, x.dtype, axes)

    # ── views: metadata only ────────────────────────────────────────────────
    def _of_view(self, t, v):
        return WTensor(t.cell, v, t.dtype, self)

    def expand(self, t, shape):
        return self._of_view(t, t.view.expand(shape))

    def reshape(self, t, shape):
        return self._of_view(t, t.view.reshape(shape))

    def permute(self, t, axes):
        return self._of_view(t, t.view.permute(axes))

    def shrink(self, t, bounds):
        return self._of_view(t, t.view.shrink(bounds))

    def flip(self, t, flags):
        return self._of_view(t, t.view.flip(flags))

    def contiguous(self, x):
        if x.view.is_c_contiguous() and x.view.offset == 0:
            return x
        return self.copy(x)

    # ── creation: nothing to wait for ───────────────────────────────────────
    def full(self, dtype, shape, value):
        """A one-element ``full`` is recorded too: the scalars inside a fused
        sequence are then never filled on the device."""
        shape = tuple(int(s) for s in shape)
        if numel(shape) != 1 or dtype.packed:
            return self._wrap(self.B.full(dtype, shape, value))
        scalar = value if isinstance(value, np.ndarray) else _encode(dtype, value)
        scalar = np.array(scalar, copy=True).reshape(1)
        e = Entry("full", None, [], shape, dtype)
        e.value = scalar
        cell = Cell(entry=e, scalar=scalar)
        e.cell = weakref.ref(cell)
        self.entries.append(e)
        return WTensor(cell, View.create(shape), dtype, self)

    def buffer(self, dtype, shape):
        return self._wrap(self.B.buffer(dtype, shape))

    def from_host(self, array, dtype):
        """Small int32 uploads (index vectors: the aranges of a causal mask, token
        ids) are kept on the host until something reads them: a compare of two
        aranges is then recognised as a causal mask, and when the attention kernel
        takes that mask as a flag neither the compare nor the uploads happen."""
        a = np.asarray(array)
        if dtype.name != "int32" or a.nbytes > 65536 or a.size == 0:
            return self._wrap(self.B.from_host(array, dtype))
        host = np.ascontiguousarray(a).reshape(-1).copy()
        e = Entry("upload", None, [], (host.size,), dtype)
        e.value = host
        cell = Cell(entry=e, host=host)
        e.cell = weakref.ref(cell)
        self.entries.append(e)
        return WTensor(cell, View.create((host.size,)), dtype, self)

    # ── everything else: execute the record, then call through ──────────────
    def __getattr__(self, name):
        target = getattr(self.B, name)
        if not callable(target):
            return target

        def call(*args, **kwargs):
            self.flush()
            out = target(*[self._lower(a) for a in args], **{k: self._lower(v) for k, v in kwargs.items()})
            return self._lift(out)

        return call

    def _lower(self, a):
        if isinstance(a, WTensor):
            return self.force(a)
        if isinstance(a, (list, tuple)):
            return type(a)(self._lower(x) for x in a)
        return a

    def _lift(self, out):
        if self._is_base_tensor(out):
            return self._wrap(out)
        if isinstance(out, (list, tuple)):
            return type(out)(self._lift(x) for x in out)
        return out

    # ── executing the record ────────────────────────────────────────────────
    def _tensor_of(self, o: Operand):
        e = o.entry
        if e is not None and e.result is None and e.kind in ("full", "upload"):
            self._issue(e)  # a scalar or an upload that something still reads
        root = e.result if e is not None else o.root
        return self.B.with_view(root, o.view)

    def _issue(self, e: Entry):
        if e.kind == "full":
            self._deliver(e, self.B.full(e.dtype, e.shape, e.value))
            return
        if e.kind == "upload":
            self._deliver(e, self.B.from_host(e.value, e.dtype))
            return
        ins = [self._tensor_of(o) for o in e.ins]
        if e.kind == "unary":
            r = self.B.unary(e.op, ins[0])
        elif e.kind == "binary":
            r = self.B.binary(e.op, ins[0], ins[1])
        elif e.kind == "where":
            r = self.B.where(ins[0], ins[1], ins[2])
        elif e.kind == "cast":
            r = self.B.cast(ins[0], e.dtype)
        elif e.kind == "compare":
            r = self.B.compare(e.op, ins[0], ins[1])
        elif e.kind == "matmul":
            r = self.B.matmul(ins[0], ins[1])
            if r.view != View.create(e.shape):  # rows with a padded pitch: the record promised a plain block
                r = self.B.contiguous(r)
        else:
            r = self.B.reduce(e.op, e.axes, ins[0])
        self.stats["issued"] += 1
        self._deliver(e, r)

    @staticmethod
    def _deliver(e: Entry, r):
        e.result = r
        cell = e.cell() if e.cell is not None else None
        if cell is not None:
            cell.root = r
            cell.entry = None
            cell.tag = e.tag

    def flush(self):
        entries, self.entries = self.entries, []
        if not entries:
            return
        self.stats["flushes"] += 1
        plans = {}
        if self.fuse:
            for e in reversed(entries):
                if e.fused_into is not None or id(e) in plans:
                    continue
                plan = _match(self, e)
                if plan is not None:
                    plans[id(e)] = plan
                    for inner in plan.interior:
                        inner.fused_into = e
        carried = []
        try:
            for e in entries:
                if e.fused_into is not None:
                    continue
                if e.kind == "compare" and e.tag is not None and e.result is None and not e.wanted:
                    # A causal mask whose readers all went into fused runs that take it as a
                    # flag: nobody has needed its elements yet. It stays recorded (with the
                    # uploads it reads) until a reader outside a fused run or a caller wants
                    # it, and is dropped once its last handle is gone.
                    if all(r.fused_into is not None and _takes_flag(plans, r) for r in e.readers):
                        if e.alive:
                            carried += [o.entry for o in e.ins if o.entry is not None and o.entry.result is None]
                            carried.append(e)
                        continue
                if e.kind == "upload":
                    # uploaded when a reader is issued or a caller wants it; kept while a handle is left
                    if e.result is None:
                        if e.wanted:
                            self._issue(e)
                        elif e.alive:
                            carried.append(e)
                    continue
                if e.kind == "full":
                    # filled only if a handle is left or, later, when a reader is issued
                    if e.alive and e.result is None:
                        self._issue(e)
                    continue
                plan = plans.get(id(e))
                if plan is None:
                    self._issue(e)
                    continue
                try:
                    r = plan.run(self)
                except RuntimeError:
                    # the backend declined the fused form: issue the run as recorded
                    self.stats["fallbacks"] += 1
                    for inner in plan.interior:
                        self._issue(inner)
                    self._issue(e)
                    continue
                self.stats[plan.name] += 1
                self._deliver(e, r)
        finally:
            keep = set(map(id, carried))
            for e in entries:  # drop the graph: results stay alive through their cells only
                if id(e) in keep:
                    e.readers = []
                else:
                    e.ins, e.readers, e.result = [], [], None
            seen = set()
            self.entries = [e for e in carried if not (id(e) in seen or seen.add(id(e)))] + self.entries

    def synchronize(self):
        self.flush()
        return self.B.synchronize()

    def timer_start(self):
        self.flush()
        return self.B.timer_start()

    def timer_stop(self):
        self.flush()
        return self.B.timer_stop()


# ── recognising the three sequences ──────────────────────────────────────────

class Plan:
    def __init__(self, name, interior, run):
        self.name, self.interior, self.run = name, interior, run


def _producer(o: Operand, kind, op=None, identity=True) -> Optional[Entry]:
    e = o.entry
    if e is None or e.kind != kind or (op is not None and e.op != op) or e.fused_into is not None:
        return None
    if identity and not _identity(o.view, e.shape):
        return None
    return e


def _takes_flag(plans, reader: Entry) -> bool:
    """The fused run `reader` went into replaces its mask operand by a flag."""
    plan = plans.get(id(reader.fused_into))
    return plan is not None and plan.name == "attention" and getattr(plan, "causal", False)


def _hidden(interior: Sequence[Entry], anchor: Entry) -> bool:
    """No handle to an interior result is left and all its readers are inside the run."""
    inside = set(map(id, interior)) | {id(anchor)}
    return all((not e.alive) and all(id(r) in inside for r in e.readers) for e in interior)


def _scalar_of(o: Operand, dtype) -> Optional[np.ndarray]:
    if (o.entry is not None and o.entry.kind != "full") or o.scalar is None or not _all_broadcast(o.view):
        return None
    if o.scalar.dtype != dtype.np_storage:
        return None
    return o.scalar


def _rows_ok(o: Operand, shape) -> bool:
    """The operand's rows are contiguous (what the fused kernels need of x)."""
    if not shape or shape[-1] > MAX_ROW or len(shape) > 9:
        return False
    if o.view.shape != tuple(shape):
        return False
    return shape[-1] == 1 or o.view.strides[-1] == 1


def _match(w: Window, e: Entry) -> Optional[Plan]:
    """Tries the runs that can END in an entry of e's kind."""
    if e.kind == "matmul":
        matchers = (_match_attention,)
    elif e.kind == "cast":
        matchers = (_match_softmax,)
    elif e.kind == "binary":
        if e.op == "add":
            matchers = (_match_linear, _match_layer_norm)
        elif e.op == "mul":
            matchers = (_match_gelu,)
        elif e.op == "fdiv":
            matchers = (_match_softmax,)
        else:
            return None
    else:
        return None
    for m in matchers:
        p = m(w, e)
        if p is not None:
            return p
    return None


def _softmax_parts(anchor: Entry):
    """The softmax run ending in `anchor` (the final division, or the cast behind
    it): (interior, x, scale, mask, masked_value, shape), or None. `x` is the
    operand the run starts from, behind the optional scale and mask."""
    interior = []
    d = anchor
    if anchor.kind == "cast":
        d = _producer(anchor.ins[0], "binary", "fdiv")
        if d is None or d.dtype.name != "float32" or anchor.dtype.name not in ("float16", "bfloat16"):
            return None
        interior.append(d)
    if d.kind != "binary" or d.op != "fdiv" or d.dtype.name not in FUSED_FLOATS or not d.shape:
        return None
    shape, last = d.shape, [len(d.shape) - 1]
    ex = _producer(d.ins[0], "unary", "exp")
    s = d.ins[1].entry
    if ex is None or s is None or s.kind != "reduce" or s.op != "sum" or s.axes != last or s.fused_into is not None:
        return None
    if not _row_broadcast(d.ins[1].view, shape) or _producer(s.ins[0], "unary", "exp") is not ex:
        return None
    sub = _producer(ex.ins[0], "binary", "sub")
    if sub is None:
        return None
    mx = sub.ins[1].entry
    if (mx is None or mx.kind != "reduce" or mx.op != "max" or mx.axes != last or mx.fused_into is not None
            or not _row_broadcast(sub.ins[1].view, shape) or not mx.ins[0].same(sub.ins[0])):
        return None
    interior += [ex, s, sub, mx]
    x = sub.ins[0]
    scale = mask = masked = None
    # the mask and scale in front (attention.ml:93-101), each only if it can be hidden too
    wh = _producer(x, "where")
    if wh is not None and _hidden(interior + [wh], anchor):
        fill = _scalar_of(wh.ins[2], wh.dtype)
        m = wh.ins[0]
        if fill is not None and m.view.shape == tuple(shape) and (shape[-1] == 1 or m.view.strides[-1] in (0, 1)):
            interior.append(wh)
            mask, masked, x = m, fill, wh.ins[1]
    mul = _producer(x, "binary", "mul")
    if mul is not None and _hidden(interior + [mul], anchor):
        sc = _scalar_of(mul.ins[1], mul.dtype)
        if sc is not None:
            interior.append(mul)
            scale, x = sc, mul.ins[0]
    if not _hidden(interior, anchor):
        return None
    return interior, x, scale, mask, masked, shape


def _match_softmax(w: Window, anchor: Entry) -> Optional[Plan]:
    parts = _softmax_parts(anchor)
    if parts is None:
        return None
    interior, x, scale, mask, masked, shape = parts
    if not _rows_ok(x, shape):
        return None
    out_dtype = anchor.dtype

    def run(win: Window):
        return win.B.softmax_rows(win._tensor_of(x), scale, win._tensor_of(mask) if mask is not None else None,
                                  masked, out_dtype)

    return Plan("softmax_rows", interior, run)


def _match_attention(w: Window, anchor: Entry) -> Optional[Plan]:
    """kaun/lib/attention.ml:67-110 for 16-bit operands: cast q and k to float32,
    Q K^T, [scale], [mask], softmax, cast back, probs x V."""
    if anchor.kind != "matmul" or anchor.dtype.name not in ISLAND or len(anchor.shape) < 2:
        return None
    dtype = anchor.dtype
    probs = _producer(anchor.ins[0], "cast")
    if probs is None or probs.dtype is not dtype:
        return None
    parts = _softmax_parts(probs)
    if parts is None:
        return None
    interior, x, scale, mask, masked, sshape = parts
    scores = _producer(x, "matmul")
    if scores is None or scores.dtype.name != "float32":
        return None
    cq = _producer(scores.ins[0], "cast")
    kt = scores.ins[1]
    ck = kt.entry
    if cq is None or ck is None or ck.kind != "cast" or ck.fused_into is not None or len(ck.shape) < 2:
        return None
    r = len(ck.shape)
    axes = list(range(r))
    axes[-1], axes[-2] = axes[-2], axes[-1]
    if kt.view != View.create(ck.shape).permute(axes):
        return None
    q, k, v = cq.ins[0], ck.ins[0], anchor.ins[1]
    dt_of = lambda o: o.entry.dtype if o.entry is not None else o.root.dtype
    if dt_of(q) is not dtype or dt_of(k) is not dtype or dt_of(v) is not dtype:
        return None
    qs, ks, vs = q.view.shape, k.view.shape, v.view.shape
    if (len(qs) != r or len(vs) != r or qs[:-2] != ks[:-2] or qs[:-2] != vs[:-2] or ks != vs or qs[-1] != ks[-1]
            or qs[-1] not in (32, 64, 128) or tuple(anchor.shape) != qs or len(qs) > 6
            or any(o.view.strides[-1] != 1 for o in (q, k, v))):
        return None
    interior = interior + [probs, scores, cq, ck]
    if not _hidden(interior, anchor):
        return None
    causal = False
    if mask is not None:
        n = qs[-2]
        flat = tuple(0 if s_ != 1 else st for s_, st in zip(sshape[:-2], mask.view.strides[:-2]))
        neg_inf = masked is not None and float(np.asarray(masked, dtype=np.float32).reshape(-1)[0]) == float("-inf")
        if (neg_inf and mask.tag == ("causal", n) and ks[-2] == n and mask.view.offset == 0 and mask.view.strides[-2:] == (n, 1)
                and all(st == 0 or s_ == 1 for s_, st in zip(sshape[:-2], mask.view.strides[:-2]))):
            causal, mask = True, None  # the kernel takes the mask as a flag (see Window.flush for the compare)
        del flat
    as_f32 = lambda a: None if a is None else np.asarray(a, dtype=np.float32).reshape(1)

    def run(win: Window):
        return win.B.attention(win._tensor_of(q), win._tensor_of(k), win._tensor_of(v), as_f32(scale),
                               win._tensor_of(mask) if mask is not None else None, as_f32(masked), causal)

    plan = Plan("attention", interior, run)
    plan.causal = causal
    return plan


def _match_linear(w: Window, anchor: Entry) -> Optional[Plan]:
    """kaun/lib/linear.ml:50-52 and the residual add around it (gpt2.ml:165-176):
    add(matmul(x, w), bias), optionally inside add(residual, .), as one GEMM with
    the adds in its epilogue."""
    if anchor.kind != "binary" or anchor.op != "add" or anchor.dtype.name not in ("float16", "bfloat16", "float32"):
        return None
    shape = anchor.shape
    if len(shape) < 2:
        return None

    def biased(o: Operand):
        """(matmul entry, bias operand) if `o` is add(matmul, broadcast vector)."""
        e = _producer(o, "binary", "add")
        if e is None:
            return None
        mm = _producer(e.ins[0], "matmul")
        b = e.ins[1]
        if mm is None or b.entry is not None or not _vector_broadcast(b.view, shape):
            return None
        return e, mm, b

    interior, bias, residual, mm = None, None, None, None
    # residual + (matmul + bias), either operand order; then matmul + bias; then residual + matmul
    for inner, other in ((anchor.ins[1], anchor.ins[0]), (anchor.ins[0], anchor.ins[1])):
        hit = biased(inner)
        if hit is not None and _hidden([hit[0], hit[1]], anchor) and other.view.shape == tuple(shape):
            interior, mm, bias, residual = [hit[0], hit[1]], hit[1], hit[2], other
            break
    if interior is None:
        m0 = _producer(anchor.ins[0], "matmul")
        if m0 is not None and anchor.ins[1].entry is None and _vector_broadcast(anchor.ins[1].view, shape) \
                and _hidden([m0], anchor):
            interior, mm, bias = [m0], m0, anchor.ins[1]
    if interior is None:
        for inner, other in ((anchor.ins[1], anchor.ins[0]), (anchor.ins[0], anchor.ins[1])):
            m0 = _producer(inner, "matmul")
            if m0 is not None and _hidden([m0], anchor) and other.view.shape == tuple(shape):
                interior, mm, residual = [m0], m0, other
                break
    if interior is None or tuple(mm.shape) != tuple(shape):
        return None
    if residual is not None and shape[-1] > 1 and residual.view.strides[-1] != 1:
        return None
    x, wt = mm.ins

    def vector(win: Window, o: Operand):
        t = win._tensor_of(o)
        return win.B.with_view(t, View.create((shape[-1],), (o.view.strides[-1] if shape[-1] > 1 else 1,), o.view.offset))

    def run(win: Window):
        return win.B.linear(win._tensor_of(x), win._tensor_of(wt), vector(win, bias) if bias is not None else None,
                            win._tensor_of(residual) if residual is not None else None)

    return Plan("linear", interior, run)


def _match_layer_norm(w: Window, anchor: Entry) -> Optional[Plan]:
    # anchor: add(mul(normalized, gamma), beta)   (layer_norm.ml:66-68)
    if anchor.kind != "binary" or anchor.op != "add" or anchor.dtype.name not in FUSED_FLOATS or not anchor.shape:
        return None
    shape, last, dtype = anchor.shape, [len(anchor.shape) - 1], anchor.dtype
    g = _producer(anchor.ins[0], "binary", "mul")
    beta = anchor.ins[1]
    if g is None or beta.entry is not None or not _vector_broadcast(beta.view, shape):
        return None
    gamma = g.ins[1]
    if gamma.entry is not None or not _vector_broadcast(gamma.view, shape):
        return None
    interior = [g]
    island = dtype.name in ISLAND
    n_op = g.ins[0]
    stat = dtype
    if island:
        c_out = _producer(n_op, "cast")
        if c_out is None:
            return None
        interior.append(c_out)
        n_op = c_out.ins[0]
        stat = dt.float32
    nrm = _producer(n_op, "binary", "fdiv")
    if nrm is None or nrm.dtype is not stat:
        return None
    xc = _producer(nrm.ins[0], "binary", "sub")
    rt = nrm.ins[1].entry
    if (xc is None or rt is None or rt.kind != "unary" or rt.op != "sqrt" or rt.fused_into is not None
            or not _row_broadcast(nrm.ins[1].view, shape)):
        return None
    keep = tuple(shape[:-1]) + (1,)
    add = _producer(rt.ins[0], "binary", "add")
    if add is None or add.shape != keep:
        return None
    eps = _scalar_of(add.ins[1], stat)
    var = _producer(add.ins[0], "binary", "fdiv")
    if eps is None or var is None:
        return None
    s2, cnt2 = var.ins[0].entry, _scalar_of(var.ins[1], stat)
    if (s2 is None or s2.kind != "reduce" or s2.op != "sum" or s2.axes != last or cnt2 is None
            or not _identity(var.ins[0].view, keep)):
        return None
    sq = _producer(s2.ins[0], "binary", "mul")
    if sq is None or _producer(sq.ins[0], "binary", "sub") is not xc or _producer(sq.ins[1], "binary", "sub") is not xc:
        return None
    mu = xc.ins[1].entry
    if (mu is None or mu.kind != "binary" or mu.op != "fdiv" or mu.fused_into is not None
            or not _row_broadcast(xc.ins[1].view, shape)):
        return None
    s1, cnt1 = mu.ins[0].entry, _scalar_of(mu.ins[1], stat)
    if (s1 is None or s1.kind != "reduce" or s1.op != "sum" or s1.axes != last or cnt1 is None
            or not _identity(mu.ins[0].view, keep) or not s1.ins[0].same(xc.ins[0])):
        return None
    count = float(shape[-1])
    as_float = lambda a: float(a.astype(np.float64)[0])
    if as_float(cnt1) != count or as_float(cnt2) != count or float(np.float32(count)) != count:
        return None
    interior += [nrm, rt, add, var, s2, sq, xc, mu, s1]
    x = xc.ins[0]
    if island:
        c_in = _producer(x, "cast")
        if c_in is None or c_in.ins[0].view.shape != tuple(shape):
            return None
        interior.append(c_in)
        x = c_in.ins[0]
        src_dtype = x.entry.dtype if x.entry is not None else x.root.dtype
        if src_dtype is not dtype:
            return None
    eps_value = as_float(eps)
    if not (eps_value >= 0) or not _hidden(interior, anchor) or not _rows_ok(x, shape):
        return None

    def vector(win: Window, o: Operand):
        # back to the rank-1 parameter: the last axis of the broadcast view
        t = win._tensor_of(o)
        v = View.create((shape[-1],), (o.view.strides[-1] if shape[-1] > 1 else 1,), o.view.offset)
        return win.B.with_view(t, v)

    def run(win: Window):
        return win.B.layer_norm_rows(win._tensor_of(x), vector(win, gamma), vector(win, beta), eps_value)

    return Plan("layer_norm_rows", interior, run)


def _match_gelu(w: Window, anchor: Entry) -> Optional[Plan]:
    # fn.ml:31-38, outermost first
    if anchor.kind != "binary" or anchor.op != "mul" or anchor.dtype.name not in FUSED_FLOATS:
        return None
    d = anchor.dtype
    c3 = _scalar_of(anchor.ins[1], d)
    wv = _producer(anchor.ins[0], "binary", "mul")
    if c3 is None or wv is None:
        return None
    x = wv.ins[0]
    u = _producer(wv.ins[1], "binary", "add")
    if u is None:
        return None
    c2 = _scalar_of(u.ins[1], d)
    th = _producer(u.ins[0], "unary", "tanh")
    if c2 is None or th is None:
        return None
    inner = _producer(th.ins[0], "binary", "mul")
    if inner is None:
        return None
    c1 = _scalar_of(inner.ins[1], d)
    q = _producer(inner.ins[0], "binary", "add")
    if c1 is None or q is None or not q.ins[0].same(x):
        return None
    p = _producer(q.ins[1], "binary", "mul")
    if p is None:
        return None
    c0 = _scalar_of(p.ins[1], d)
    x3 = _producer(p.ins[0], "binary", "mul")
    if c0 is None or x3 is None or not x3.ins[0].same(x):
        return None
    x2 = _producer(x3.ins[1], "binary", "mul")
    if x2 is None or not x2.ins[0].same(x) or not x2.ins[1].same(x):
        return None
    interior = [wv, u, th, inner, q, p, x3, x2]
    if not _hidden(interior, anchor) or not x.view.is_c_contiguous() or x.view.shape != tuple(anchor.shape):
        return None
    consts = np.concatenate([c0, c1, c2, c3])

    def run(win: Window):
        return win.B.gelu_tanh(win._tensor_of(x), consts)

    return Plan("gelu_tanh", interior, run)
