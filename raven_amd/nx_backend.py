"""Host-side mirror of the Nx backend binding, on top of the libnxhip C ABI.

This is what ``nx_backend.ml`` of an ``nx_hip`` library does, written in Python
because this image has no OCaml toolchain: it allocates each result, unpacks
tensor handles into ``nxh_tensor`` descriptors and makes one C call per
primitive. Operation names, argument meaning and error kinds follow
``Nx_core.Backend_intf.S`` (packages/nx/lib/core/backend_intf.ml:77-721) and
the reference binding (packages/nx/lib/backend_c/nx_backend.ml):

* a tensor is ``{buffer; shape; strides; offset; dtype; context}``; movement ops
  only rewrite the view and share the buffer (nx_backend.ml:36-84);
* compute ops allocate a fresh C-contiguous, offset-0 result
  (nx_backend.ml:170-183);
* ``ValueError`` stands for OCaml's ``Invalid_argument``, ``RuntimeError`` for
  ``Failure`` (nx_c_engine.c:1345-1351).

There is no CPU fallback: constructing a ``Backend`` without a GPU or without
the built library raises.
"""

from __future__ import annotations

import ctypes as C
from typing import Sequence

import numpy as np

from . import _ffi
from . import dtype as dt
from ._ffi import BINARY_OPS, COMPARE_OPS, REDUCE_OPS, UNARY_OPS, NxhTensor, make_tensor
from .view import View, numel


class DeviceBuffer:
    """One device allocation, shared by every view of a tensor. Returned to the
    context's caching allocator when the last handle goes away (the OCaml
    binding does the same from a custom-block finaliser)."""

    __slots__ = ("ctx", "ptr", "nbytes", "__weakref__")

    def __init__(self, ctx: "Backend", nbytes: int):
        p = C.c_void_p()
        ctx._check(ctx._lib.nxh_alloc(ctx._h, nbytes, C.byref(p)))
        self.ctx = ctx
        self.ptr = p.value
        self.nbytes = nbytes

    def __del__(self):
        ctx = getattr(self, "ctx", None)
        if ctx is not None and ctx._h and self.ptr:
            ctx._lib.nxh_free(ctx._h, self.ptr)
            self.ptr = None


class Tensor:
    """The backend's tensor handle (nx_backend.ml:36-43)."""

    __slots__ = ("buffer", "view", "dtype", "context")

    def __init__(self, buffer: DeviceBuffer, view: View, dtype: dt.DType, context: "Backend"):
        self.buffer = buffer
        self.view = view
        self.dtype = dtype
        self.context = context

    @property
    def shape(self):
        return self.view.shape

    @property
    def strides(self):
        return self.view.strides

    @property
    def offset(self):
        return self.view.offset

    def _desc(self):
        v = self.view
        return make_tensor(self.buffer.ptr, self.dtype.tag, v.shape, v.strides, v.offset)

    def __repr__(self):  # pragma: no cover
        return f"Tensor({self.dtype.name}, shape={self.shape}, strides={self.strides}, offset={self.offset})"


def encode_scalar(dtype: dt.DType, value) -> np.ndarray:
    """Host encoding of a ``full`` value, as ``Nx_buffer.fill`` stores it
    (packages/nx/lib/buffer/nx_buffer_stubs.h:70-302): one storage element."""
    if dtype is dt.bfloat16:
        u = np.asarray(value, dtype=np.float32).reshape(1).view(np.uint32)
        nan = (u & 0x7FFFFFFF) > 0x7F800000
        r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
        return np.where(nan, ((u >> 16) | 0x40).astype(np.uint16), r)
    if dtype in (dt.float8_e4m3, dt.float8_e5m2):
        raise NotImplementedError("encode fp8 scalars with cast from float32")
    if dtype.packed:
        return np.asarray(int(value) & 0xF, dtype=np.uint8).reshape(1)
    if dtype is dt.bool_:
        return np.asarray(1 if value else 0, dtype=np.uint8).reshape(1)
    with np.errstate(all="ignore"):
        return np.asarray(value).astype(dtype.np_storage).reshape(1)


class Graph:
    """Launches recorded between Backend.capture_begin and capture_end. Tensors
    created in between keep their storage: `launch` recomputes them in place
    from what the older tensors they were computed from hold at that time."""

    def __init__(self, backend, handle):
        self._backend, self._h = backend, handle

    def launch(self):
        b = self._backend
        b._check(b._lib.nxh_graph_launch(b._h, self._h))

    def destroy(self):
        if self._h:
            b = self._backend
            b._check(b._lib.nxh_graph_destroy(b._h, self._h))
            self._h = None


class Backend:
    """An execution context (``create_context``, nx_backend.mli:32-39) plus the
    operations of ``Backend_intf.S``."""

    def __init__(self):
        self._lib = _ffi.load()
        self._gelu_constants = {}
        h = C.c_void_p()
        rc = self._lib.nxh_context_create(C.byref(h))
        self._h = h.value
        if rc != _ffi.NXH_OK:
            self._h = None
            raise RuntimeError(self._lib.nxh_last_error(None).decode())

    def close(self):
        if self._h:
            self._lib.nxh_context_destroy(self._h)
            self._h = None

    # ── plumbing ────────────────────────────────────────────────────────────
    def _check(self, rc: int):
        if rc == _ffi.NXH_OK:
            return
        msg = self._lib.nxh_last_error(self._h).decode()
        if rc == _ffi.NXH_INVALID_ARGUMENT:
            raise ValueError(msg)
        raise RuntimeError(msg)

    def device_info(self):
        dev, cus = C.c_int(), C.c_int()
        name = C.create_string_buffer(128)
        self._check(self._lib.nxh_device_info(self._h, C.byref(dev), name, 128, C.byref(cus)))
        return {"device": dev.value, "name": name.value.decode(), "compute_units": cus.value}

    def synchronize(self):
        self._check(self._lib.nxh_synchronize(self._h))

    def last_path(self) -> str:
        return self._lib.nxh_last_path(self._h).decode()

    # -- recorded sequences: no counterpart in Backend_intf.S, whose calls run as they are made --
    def capture_begin(self):
        """From here to capture_end every call records its launches instead of
        running them; to_host / synchronize raise until then."""
        self._check(self._lib.nxh_capture_begin(self._h))

    def capture_end(self) -> "Graph":
        g = C.c_void_p()
        self._check(self._lib.nxh_capture_end(self._h, C.byref(g)))
        return Graph(self, g)

    # -- deferred evaluation: primitives are recorded and fused below the C ABI --
    DEFER_STATS = ("recorded", "issued", "flushes", "fallbacks", "softmax_rows", "layer_norm_rows", "gelu_tanh",
                   "attention", "linear", "postponed", "materialised", "linear_gelu", "grouped")

    def set_deferred(self, on: bool):
        """With the mode on, unary / binary / compare / where / cast / reduce / matmul and
        one-element fills are recorded by the library and executed (fused where a run spells
        softmax, layer norm, GELU, attention or a linear layer whose intermediates have died)
        by the next call of anything else, a host read included."""
        self._check(self._lib.nxh_set_deferred(self._h, int(bool(on))))

    def deferred_stats(self):
        v = (C.c_uint64 * len(self.DEFER_STATS))()
        self._check(self._lib.nxh_deferred_stats(self._h, v, len(self.DEFER_STATS)))
        return dict(zip(self.DEFER_STATS, (int(x) for x in v)))

    def set_cache_policy(self, mode: int):
        """Bit 0 allows streaming (non-temporal) loads, bit 1 streaming stores, of blocks whose
        history says they are not touched again while cached; 0 turns the policy off."""
        self._check(self._lib.nxh_set_cache_policy(self._h, int(mode)))

    def cache_policy_stats(self):
        a, b = C.c_uint64(), C.c_uint64()
        self._check(self._lib.nxh_cache_policy_stats(self._h, C.byref(a), C.byref(b)))
        return {"streaming_in": a.value, "streaming_out": b.value}

    def memory_stats(self):
        v = [C.c_uint64() for _ in range(4)]
        self._check(self._lib.nxh_memory_stats(self._h, *[C.byref(x) for x in v]))
        return dict(zip(("in_use", "cached", "reserved", "driver_allocs"), (x.value for x in v)))

    def trim(self):
        self._check(self._lib.nxh_trim(self._h))

    def timer_start(self):
        self._check(self._lib.nxh_timer_start(self._h))

    def timer_stop(self) -> float:
        ms = C.c_float()
        self._check(self._lib.nxh_timer_stop(self._h, C.byref(ms)))
        return ms.value

    # ── creation (backend_intf.ml:120-145) ──────────────────────────────────
    def buffer(self, dtype: dt.DType, shape: Sequence[int]) -> Tensor:
        """Uninitialised C-contiguous tensor."""
        shape = tuple(int(s) for s in shape)
        buf = DeviceBuffer(self, dtype.nbytes(numel(shape)))
        return Tensor(buf, View.create(shape), dtype, self)

    def full(self, dtype: dt.DType, shape: Sequence[int], value) -> Tensor:
        """Every element is ``value`` (a Python number, or one already-encoded
        storage element as a numpy array)."""
        out = self.buffer(dtype, shape)
        enc = value if isinstance(value, np.ndarray) else encode_scalar(dtype, value)
        enc = np.ascontiguousarray(enc.reshape(1))
        d = out._desc()
        self._check(self._lib.nxh_fill(self._h, C.byref(d), enc.ctypes.data))
        return out

    def from_host(self, array: np.ndarray, dtype: dt.DType) -> Tensor:
        """Copies a flat, C-contiguous host buffer to the device; the result is
        rank 1 (nx_backend.ml:66-69). The host array may be reused on return."""
        flat = np.ascontiguousarray(array).reshape(-1)
        if flat.dtype.itemsize != dtype.np_storage.itemsize:
            raise ValueError("from_host: host array does not hold this dtype's storage type")
        n = flat.size * 2 if dtype.packed else flat.size
        buf = DeviceBuffer(self, flat.nbytes)
        self._check(self._lib.nxh_memcpy_h2d(self._h, buf.ptr, flat.ctypes.data, flat.nbytes))
        return Tensor(buf, View.create((n,)), dtype, self)

    def to_host(self, t: Tensor) -> np.ndarray:
        """The WHOLE backing storage as a flat host array, to be read through
        the tensor's view (backend_intf.ml:108-116). Waits for the stream."""
        count = t.buffer.nbytes // t.dtype.np_storage.itemsize
        host = np.empty(count, dtype=t.dtype.np_storage)
        self._check(self._lib.nxh_memcpy_d2h(self._h, host.ctypes.data, t.buffer.ptr, host.nbytes))
        return host

    # ── movement: views only (nx_backend.ml:77-84) ──────────────────────────
    def _of_view(self, t: Tensor, v: View) -> Tensor:
        return Tensor(t.buffer, v, t.dtype, self)

    def with_view(self, t: Tensor, v: View) -> Tensor:
        """``t``'s storage seen through ``v`` (any view the storage can hold)."""
        return Tensor(t.buffer, v, t.dtype, self)

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

    # ── map family (nx_backend.ml:170-234) ──────────────────────────────────
    def unary(self, op: str, x: Tensor) -> Tensor:
        out = self.buffer(x.dtype, x.shape)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_unary(self._h, UNARY_OPS.index(op), C.byref(o), C.byref(a)))
        return out

    def binary(self, op: str, x: Tensor, y: Tensor) -> Tensor:
        out = self.buffer(x.dtype, x.shape)
        o, a, b = out._desc(), x._desc(), y._desc()
        self._check(self._lib.nxh_binary(self._h, BINARY_OPS.index(op), C.byref(o), C.byref(a), C.byref(b)))
        return out

    def compare(self, op: str, x: Tensor, y: Tensor) -> Tensor:
        out = self.buffer(dt.bool_, x.shape)
        o, a, b = out._desc(), x._desc(), y._desc()
        self._check(self._lib.nxh_compare(self._h, COMPARE_OPS.index(op), C.byref(o), C.byref(a), C.byref(b)))
        return out

    def where(self, cond: Tensor, if_true: Tensor, if_false: Tensor) -> Tensor:
        out = self.buffer(if_true.dtype, if_true.shape)
        o, c, a, b = out._desc(), cond._desc(), if_true._desc(), if_false._desc()
        self._check(self._lib.nxh_where(self._h, C.byref(o), C.byref(c), C.byref(a), C.byref(b)))
        return out

    def cast(self, x: Tensor, dtype: dt.DType) -> Tensor:
        out = self.buffer(dtype, x.shape)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_cast(self._h, C.byref(o), C.byref(a)))
        return out

    # ── move family (nx_backend.ml:349-357, 399-402) ────────────────────────
    def copy(self, x: Tensor) -> Tensor:
        out = self.buffer(x.dtype, x.shape)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_copy(self._h, C.byref(o), C.byref(a)))
        return out

    def contiguous(self, x: Tensor) -> Tensor:
        """``x`` itself iff C-contiguous AND offset 0, else a copy."""
        if x.view.is_c_contiguous() and x.view.offset == 0:
            return x
        return self.copy(x)

    def assign(self, dst: Tensor, src: Tensor) -> None:
        """Writes ``src`` through ``dst``'s strides (visible through every view
        sharing dst's buffer)."""
        o, a = dst._desc(), src._desc()
        self._check(self._lib.nxh_copy(self._h, C.byref(o), C.byref(a)))

    def gather(self, data: Tensor, indices: Tensor, axis: int) -> Tensor:
        out = self.buffer(data.dtype, indices.shape)
        o, d, i = out._desc(), data._desc(), indices._desc()
        self._check(self._lib.nxh_gather(self._h, C.byref(o), C.byref(d), C.byref(i), axis))
        return out

    # ── scatter / pad / cat / scan / threefry (nx_backend.ml:309-319, 362-416, 474-477)
    def scatter(self, mode: str, unique_indices: bool, template: Tensor, indices: Tensor, updates: Tensor,
                axis: int) -> Tensor:
        """``mode`` is "set" or "add"; ``unique_indices`` is accepted and ignored,
        as in the reference binding. The result starts as a copy of ``template``."""
        out = self.copy(template)
        o, i, u = out._desc(), indices._desc(), updates._desc()
        self._check(self._lib.nxh_scatter(self._h, C.byref(o), C.byref(i), C.byref(u), axis,
                                          {"set": 0, "add": 1}[mode]))
        return out

    def pad(self, x: Tensor, padding: Sequence[Sequence[int]], fill_value) -> Tensor:
        out = self.buffer(x.dtype, [s + int(b) + int(a) for s, (b, a) in zip(x.shape, padding)])
        enc = fill_value if isinstance(fill_value, np.ndarray) else encode_scalar(x.dtype, fill_value)
        enc = np.ascontiguousarray(enc.reshape(1))
        before = (C.c_int64 * max(len(padding), 1))(*[int(b) for b, _ in padding])
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_pad(self._h, C.byref(o), C.byref(a), enc.ctypes.data, before))
        return out

    def cat(self, tensors: Sequence[Tensor], axis: int) -> Tensor:
        if not tensors:
            raise ValueError("cat: empty tensor list")
        first = tensors[0]
        axis = axis + len(first.shape) if axis < 0 else axis
        if not 0 <= axis < len(first.shape):
            raise ValueError("cat: axis out of range")
        shape = list(first.shape)
        shape[axis] = sum(t.shape[axis] for t in tensors)
        out = self.buffer(first.dtype, shape)
        descs = [t._desc() for t in tensors]
        arr = (C.POINTER(NxhTensor) * len(descs))(*[C.pointer(d) for d in descs])
        o = out._desc()
        self._check(self._lib.nxh_cat(self._h, C.byref(o), arr, len(descs), axis))
        return out

    def associative_scan(self, axis: int, op: str, x: Tensor) -> Tensor:
        out = self.buffer(x.dtype, x.shape)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_scan(self._h, REDUCE_OPS.index(op), C.byref(o), C.byref(a), axis))
        return out

    def threefry(self, key: Tensor, counter: Tensor) -> Tensor:
        out = self.buffer(dt.int32, counter.shape)
        o, k, c = out._desc(), key._desc(), counter._desc()
        self._check(self._lib.nxh_threefry(self._h, C.byref(o), C.byref(k), C.byref(c)))
        return out

    # ── sort (nx_backend.ml:330-338) ─────────────────────────────────────────
    def sort(self, x: Tensor, axis: int, descending: bool) -> Tensor:
        out = self.buffer(x.dtype, x.shape)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_sort(self._h, C.byref(o), C.byref(a), axis, int(descending)))
        return out

    def argsort(self, x: Tensor, axis: int, descending: bool) -> Tensor:
        out = self.buffer(dt.int32, x.shape)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_argsort(self._h, C.byref(o), C.byref(a), axis, int(descending)))
        return out

    # ── windows (nx_backend.ml:427-464) ──────────────────────────────────────
    @staticmethod
    def _window_params(op, in_shape, kernel_size, stride, dilation, padding):
        k = len(kernel_size)
        if not (len(stride) == len(dilation) == len(padding) == k) or k < 1 or len(in_shape) < k:
            raise ValueError(f"{op}: shape mismatch")
        spatial = in_shape[len(in_shape) - k:]
        windows, taps = 1, 1
        for i in range(k):
            padded = spatial[i] + padding[i][0] + padding[i][1]
            extent = dilation[i] * (kernel_size[i] - 1) + 1
            windows *= (padded - extent) // stride[i] + 1
            taps *= kernel_size[i]
        arr = lambda v: (C.c_int64 * len(v))(*[int(a) for a in v])
        flat = [int(v) for pair in padding for v in pair]
        return taps, windows, (arr(kernel_size), arr(stride), arr(dilation), arr(flat))

    def unfold(self, x: Tensor, kernel_size, stride, dilation, padding) -> Tensor:
        taps, windows, params = self._window_params("unfold", x.shape, kernel_size, stride, dilation, padding)
        out = self.buffer(x.dtype, tuple(x.shape[:len(x.shape) - len(kernel_size)]) + (taps, windows))
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_unfold(self._h, C.byref(o), C.byref(a), len(kernel_size), *params))
        return out

    def fold(self, x: Tensor, output_size, kernel_size, stride, dilation, padding) -> Tensor:
        if len(x.shape) < 2:
            raise ValueError("fold: shape mismatch")
        oshape = tuple(x.shape[:-2]) + tuple(int(s) for s in output_size)
        _, _, params = self._window_params("fold", oshape, kernel_size, stride, dilation, padding)
        out = self.buffer(x.dtype, oshape)
        osz = (C.c_int64 * len(output_size))(*[int(s) for s in output_size])
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_fold(self._h, C.byref(o), C.byref(a), len(kernel_size), osz, *params))
        return out

    # ── Fourier transforms (nx_backend.ml:502-548): unnormalised, the frontend owns 1/n ──
    @staticmethod
    def _axes_arg(axes):
        axes = [int(a) for a in axes]
        return (C.c_int32 * max(len(axes), 1))(*axes), len(axes)

    def fft(self, x: Tensor, axes, inverse: bool = False) -> Tensor:
        out = self.buffer(x.dtype, x.shape)
        ax, n = self._axes_arg(axes)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_fft(self._h, C.byref(o), C.byref(a), ax, n, int(inverse)))
        return out

    def ifft(self, x: Tensor, axes) -> Tensor:
        return self.fft(x, axes, inverse=True)

    def rfft(self, x: Tensor, dtype: dt.DType, axes) -> Tensor:
        ax, n = self._axes_arg(axes)
        if n < 1 or not 0 <= ax[n - 1] < len(x.shape):
            raise ValueError("rfft: axis out of range")
        shape = list(x.shape)
        shape[ax[n - 1]] = shape[ax[n - 1]] // 2 + 1
        out = self.buffer(dtype, shape)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_rfft(self._h, C.byref(o), C.byref(a), ax, n))
        return out

    def irfft(self, x: Tensor, dtype: dt.DType, axes, s=None) -> Tensor:
        ax, n = self._axes_arg(axes)
        if n < 1 or not 0 <= ax[n - 1] < len(x.shape):
            raise ValueError("irfft: axis out of range")
        size = int(s[n - 1]) if s is not None else (x.shape[ax[n - 1]] - 1) * 2
        shape = list(x.shape)
        shape[ax[n - 1]] = size
        out = self.buffer(dtype, shape)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_irfft(self._h, C.byref(o), C.byref(a), ax, n, size if s is not None else 0))
        return out

    # ── linear algebra (nx_backend.ml:550-707): the binding allocates every result ──
    def cholesky(self, x: Tensor, upper: bool = False) -> Tensor:
        out = self.buffer(x.dtype, x.shape)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_cholesky(self._h, C.byref(o), C.byref(a), int(upper)))
        return out

    def triangular_solve(self, a: Tensor, b: Tensor, upper: bool, transpose: bool, unit_diag: bool) -> Tensor:
        vector = len(b.shape) == len(a.shape) - 1
        bm = self.reshape(b, tuple(b.shape) + (1,)) if vector else b
        out = self.buffer(b.dtype, bm.shape)
        flags = int(upper) | (int(transpose) << 1) | (int(unit_diag) << 2)
        o, da, db = out._desc(), a._desc(), bm._desc()
        self._check(self._lib.nxh_triangular_solve(self._h, C.byref(o), C.byref(da), C.byref(db), flags))
        return self.reshape(out, b.shape) if vector else out

    def qr(self, x: Tensor, reduced: bool = True):
        if len(x.shape) < 2:
            raise ValueError("qr: shape mismatch")
        *batch, m, n = x.shape
        k = min(m, n)
        q = self.buffer(x.dtype, (*batch, m, k if reduced else m))
        r = self.buffer(x.dtype, (*batch, k if reduced else m, n))
        dq, dr, a = q._desc(), r._desc(), x._desc()
        self._check(self._lib.nxh_qr(self._h, C.byref(dq), C.byref(dr), C.byref(a), int(reduced)))
        return q, r

    def _eigh(self, x: Tensor, vectors: bool):
        if len(x.shape) < 2:
            raise ValueError("eigh: shape mismatch")
        w = self.buffer(dt.float64, tuple(x.shape[:-2]) + (x.shape[-1],))
        v = self.buffer(x.dtype, x.shape) if vectors else None
        dw, a = w._desc(), x._desc()
        dv = v._desc() if vectors else None
        self._check(self._lib.nxh_eigh(self._h, C.byref(dw), C.byref(dv) if vectors else None, C.byref(a)))
        return w, v

    def eigh(self, x: Tensor):
        return self._eigh(x, True)

    def eigvalsh(self, x: Tensor) -> Tensor:
        return self._eigh(x, False)[0]

    def svd(self, x: Tensor, full_matrices: bool = False):
        if len(x.shape) < 2:
            raise ValueError("svd: shape mismatch")
        *batch, m, n = x.shape
        k = min(m, n)
        u = self.buffer(x.dtype, (*batch, m, m if full_matrices else k))
        s = self.buffer(dt.float64, (*batch, k))
        vt = self.buffer(x.dtype, (*batch, n if full_matrices else k, n))
        du, ds, dv, a = u._desc(), s._desc(), vt._desc(), x._desc()
        self._check(self._lib.nxh_svd(self._h, C.byref(du), C.byref(ds), C.byref(dv), C.byref(a)))
        return u, s, vt

    def _eig(self, x: Tensor, vectors: bool):
        if len(x.shape) < 2:
            raise ValueError("eig: shape mismatch")
        w = self.buffer(dt.complex128, tuple(x.shape[:-2]) + (x.shape[-1],))
        v = self.buffer(dt.complex128, x.shape) if vectors else None
        dw, a = w._desc(), x._desc()
        dv = v._desc() if vectors else None
        self._check(self._lib.nxh_eig(self._h, C.byref(dw), C.byref(dv) if vectors else None, C.byref(a)))
        return w, v

    def eig(self, x: Tensor):
        return self._eig(x, True)

    def eigvals(self, x: Tensor) -> Tensor:
        return self._eig(x, False)[0]

    # ── fused sequences of primitives (no counterpart in Backend_intf.S) ────
    def _scalar_arg(self, dtype: dt.DType, value):
        if value is None:
            return None, None
        enc = value if isinstance(value, np.ndarray) else encode_scalar(dtype, value)
        enc = np.ascontiguousarray(enc.reshape(-1))
        return enc, enc.ctypes.data

    def softmax_rows(self, x: Tensor, scale=None, mask: Tensor | None = None, masked_value=None,
                     out_dtype: dt.DType | None = None) -> Tensor:
        """softmax over the last axis of ``x * scale`` with masked-out elements
        replaced by ``masked_value`` first, optionally cast: the sequence mul,
        where, max, sub, exp, sum, div, cast in one kernel. Scalars are Python
        numbers or already-encoded storage elements."""
        out = self.buffer(out_dtype or x.dtype, x.shape)
        keep_s, ps = self._scalar_arg(x.dtype, scale)
        keep_m, pm = self._scalar_arg(x.dtype, masked_value)
        o, a = out._desc(), x._desc()
        m = mask._desc() if mask is not None else None
        self._check(self._lib.nxh_softmax_rows(self._h, C.byref(o), C.byref(a), ps,
                                               C.byref(m) if m is not None else None, pm))
        return out

    def layer_norm_rows(self, x: Tensor, gamma: Tensor | None, beta: Tensor | None, eps: float) -> Tensor:
        out = self.buffer(x.dtype, x.shape)
        o, a = out._desc(), x._desc()
        g = gamma._desc() if gamma is not None else None
        b = beta._desc() if beta is not None else None
        self._check(self._lib.nxh_layer_norm_rows(self._h, C.byref(o), C.byref(a),
                                                  C.byref(g) if g is not None else None,
                                                  C.byref(b) if b is not None else None, float(eps)))
        return out

    def gelu_tanh(self, x: Tensor, constants=(0.044715, 0.7978845608028654, 1.0, 0.5)) -> Tensor:
        """``constants`` are four Python numbers or one array of four encoded
        storage elements."""
        out = self.buffer(x.dtype, x.shape)
        if isinstance(constants, np.ndarray):
            enc = np.ascontiguousarray(constants.reshape(4))
        else:
            key = (x.dtype.tag, tuple(constants))
            enc = self._gelu_constants.get(key)
            if enc is None:  # (encoding four scalars costs more host time than the kernel takes)
                enc = self._gelu_constants[key] = np.concatenate([encode_scalar(x.dtype, c) for c in constants])
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_gelu_tanh(self._h, C.byref(o), C.byref(a), enc.ctypes.data))
        return out

    def linear(self, x: Tensor, w: Tensor, bias: Tensor | None = None, residual: Tensor | None = None) -> Tensor:
        """``(matmul x w + bias) + residual`` in the GEMM's epilogue, every step
        rounded to the dtype as the primitives would (kaun/lib/linear.ml:50-52)."""
        xs, ws = x.shape, w.shape
        nd = max(len(xs), len(ws))
        batch = []
        for i in range(nd - 2):
            ai, bi = i - (nd - len(xs)), i - (nd - len(ws))
            batch.append(max(xs[ai] if ai >= 0 else 1, ws[bi] if bi >= 0 else 1))
        out = self.buffer(x.dtype, batch + [xs[-2], ws[-1]])
        o, a, b = out._desc(), x._desc(), w._desc()
        bd = bias._desc() if bias is not None else None
        rd = residual._desc() if residual is not None else None
        self._check(self._lib.nxh_linear(self._h, C.byref(o), C.byref(a), C.byref(b),
                                         C.byref(bd) if bd is not None else None,
                                         C.byref(rd) if rd is not None else None))
        return out

    def linear_gelu_tanh(self, x: Tensor, w: Tensor, bias: Tensor | None = None,
                         constants=(0.044715, 0.7978845608028654, 1.0, 0.5)) -> Tensor:
        """``gelu_tanh(matmul x w + bias)`` with the GELU in the GEMM's epilogue: the bits of
        ``linear`` followed by ``gelu_tanh``. Raises for anything but bfloat16 / float16 products made
        of whole 128 x 128 (or 128 x 192) tiles (the caller then issues the two calls)."""
        out = self.buffer(x.dtype, list(x.shape[:-1]) + [w.shape[-1]])
        if isinstance(constants, np.ndarray):
            enc = np.ascontiguousarray(constants.reshape(4))
        else:
            enc = np.concatenate([encode_scalar(x.dtype, c) for c in constants])
        o, a, b = out._desc(), x._desc(), w._desc()
        bd = bias._desc() if bias is not None else None
        self._check(self._lib.nxh_linear_gelu_tanh(self._h, C.byref(o), C.byref(a), C.byref(b),
                                                   C.byref(bd) if bd is not None else None, enc.ctypes.data))
        return out

    def attention(self, q: Tensor, k: Tensor, v: Tensor, scale=None, mask: Tensor | None = None,
                  masked_value=None, causal: bool = False) -> Tensor:
        """Scaled dot-product attention of f16 / bf16 operands in one kernel
        (the sequence of kaun/lib/attention.ml:67-110). ``scale`` and
        ``masked_value`` are float32 scalars."""
        out = self.buffer(q.dtype, q.shape)
        keep_s, ps = self._scalar_arg(dt.float32, scale)
        keep_m, pm = self._scalar_arg(dt.float32, masked_value)
        o, a, b, c = out._desc(), q._desc(), k._desc(), v._desc()
        m = mask._desc() if mask is not None else None
        self._check(self._lib.nxh_attention(self._h, C.byref(o), C.byref(a), C.byref(b), C.byref(c), ps,
                                            C.byref(m) if m is not None else None, pm, int(causal)))
        return out

    # ── fold family (nx_backend.ml:266-307) ─────────────────────────────────
    def reduce(self, op: str, axes: Sequence[int], x: Tensor) -> Tensor:
        axes = sorted(int(a) for a in axes)
        if op in ("max", "min"):
            for a in axes:
                if x.shape[a] == 0:
                    raise ValueError(f"reduce_{op}: reduction over an empty axis has no identity")
        oshape = [s for i, s in enumerate(x.shape) if i not in axes]
        out = self.buffer(x.dtype, oshape)
        arr = (C.c_int32 * max(len(axes), 1))(*axes)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_reduce(self._h, REDUCE_OPS.index(op), C.byref(o), C.byref(a), arr, len(axes)))
        return out

    def reduce_noalloc(self, op: str, axes: Sequence[int], x: Tensor, out: Tensor) -> Tensor:
        """`reduce` into a result the caller allocated beforehand, through the entry
        point that neither allocates nor frees device memory (its split partials
        live in the library's static per-device workspace)."""
        axes = sorted(int(a) for a in axes)
        arr = (C.c_int32 * max(len(axes), 1))(*axes)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_reduce_noalloc(self._h, REDUCE_OPS.index(op), C.byref(o), C.byref(a), arr, len(axes)))
        return out

    def _argreduce(self, is_min: bool, x: Tensor, axis: int, keepdims: bool) -> Tensor:
        name = "argmin" if is_min else "argmax"
        if x.shape[axis] == 0:
            raise ValueError(f"{name}: argument reduction over an empty axis")
        if keepdims:
            oshape = [1 if i == axis else s for i, s in enumerate(x.shape)]
        else:
            oshape = [s for i, s in enumerate(x.shape) if i != axis]
        out = self.buffer(dt.int32, oshape)
        o, a = out._desc(), x._desc()
        self._check(self._lib.nxh_argreduce(self._h, int(is_min), C.byref(o), C.byref(a), axis))
        return out

    def argmax(self, x: Tensor, axis: int, keepdims: bool = False) -> Tensor:
        return self._argreduce(False, x, axis, keepdims)

    def argmin(self, x: Tensor, axis: int, keepdims: bool = False) -> Tensor:
        return self._argreduce(True, x, axis, keepdims)

    # ── matmul (nx_backend.ml:485-500) ──────────────────────────────────────
    def matmul(self, x: Tensor, y: Tensor) -> Tensor:
        xs, ys = x.shape, y.shape
        nd = max(len(xs), len(ys))
        batch = []
        for i in range(nd - 2):
            ai, bi = i - (nd - len(xs)), i - (nd - len(ys))
            batch.append(max(xs[ai] if ai >= 0 else 1, ys[bi] if bi >= 0 else 1))
        out = self._matmul_result(x.dtype, batch + [xs[-2], ys[-1]])
        o, a, b = out._desc(), x._desc(), y._desc()
        self._check(self._lib.nxh_matmul(self._h, C.byref(o), C.byref(a), C.byref(b)))
        return out

    def _matmul_result(self, dtype: dt.DType, shape) -> Tensor:
        """The fresh result of a matmul. The reference allocates it C-contiguous
        (nx_backend.ml:485-500); here a long row that is no whole number of 128-byte
        memory lines (GPT-2's 50257 logits per token) gets a row pitch rounded up to
        whole lines, and the result is the [..., n] view of that block. Every row of
        the GEMM's output tile then starts on a line and is written with whole aligned
        vectors (the head GEMM of GPT-2 small: 0.82 -> 0.73 ms)."""
        n = int(shape[-1])
        line = 128 // dtype.itemsize if not dtype.packed else 0
        if line == 0 or n < 4096 or n % line == 0 or 0 in shape:
            return self.buffer(dtype, shape)
        pitch = (n + line - 1) // line * line
        block = self.buffer(dtype, list(shape[:-1]) + [pitch])
        return self.shrink(block, [(0, int(s)) for s in shape])


def logical(t: Tensor) -> np.ndarray:
    """Host copy of the tensor's logical contents (storage dtype), read through
    its view from the full backing storage."""
    if t.dtype.packed:
        raise NotImplementedError("packed tensors have no element-addressable host view")
    storage = t.context.to_host(t)
    v = t.view
    if v.numel == 0:
        return np.zeros(v.shape, dtype=storage.dtype)
    es = storage.dtype.itemsize
    return np.lib.stride_tricks.as_strided(storage[v.offset:], shape=v.shape,
                                           strides=[s * es for s in v.strides]).copy()
