"""numpy-facing wrapper of the CPU parity oracle (``libnxoracle.so``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by the smoke check and by the
``cpu_baseline`` leg of ``bench.py`` — never by the product package.

``OracleBackend`` has the same operation names as ``raven_amd.nx_backend`` (and
therefore as ``Nx_core.Backend_intf.S``), but tensors are host numpy storage
plus a ``View``; it restates what the reference binding does around each C call
(packages/nx/lib/backend_c/nx_backend.ml).
"""

from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

from raven_amd import dtype as dt
from raven_amd._ffi import (BINARY_OPS, COMPARE_OPS, NXH_INVALID_ARGUMENT, REDUCE_OPS,
                            UNARY_OPS, NxhTensor, make_tensor)
from raven_amd.view import View, c_contiguous_strides, numel

HERE = Path(__file__).resolve().parent
LIB = HERE / "libnxoracle.so"


def build(force: bool = False) -> Path:
    src = HERE / "nx_oracle.c"
    if force or not LIB.exists() or LIB.stat().st_mtime < src.stat().st_mtime:
        subprocess.run(["make", "-C", str(HERE), "-B" if force else "-s"], check=True,
                       capture_output=True)
    return LIB


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(str(LIB))
        T = C.POINTER(NxhTensor)
        L.nxo_last_error.restype = C.c_char_p
        for name, args in {
            "nxo_unary": [C.c_int, T, T],
            "nxo_binary": [C.c_int, T, T, T],
            "nxo_compare": [C.c_int, T, T, T],
            "nxo_where": [T, T, T, T],
            "nxo_cast": [T, T],
            "nxo_copy": [T, T],
            "nxo_fill": [T, C.c_void_p],
            "nxo_reduce": [C.c_int, T, T, C.POINTER(C.c_int32), C.c_int],
            "nxo_argreduce": [C.c_int, T, T, C.c_int],
            "nxo_matmul": [T, T, T],
            "nxo_gather": [T, T, T, C.c_int],
            "nxo_pad": [T, T, C.c_void_p, C.POINTER(C.c_int64)],
            "nxo_cat": [T, C.POINTER(T), C.c_int, C.c_int],
            "nxo_scan": [C.c_int, T, T, C.c_int],
            "nxo_threefry": [T, T, T],
            "nxo_scatter": [T, T, T, C.c_int, C.c_int],
            "nxo_sort": [T, T, C.c_int, C.c_int],
            "nxo_argsort": [T, T, C.c_int, C.c_int],
            "nxo_unfold": [T, T, C.c_int] + [C.POINTER(C.c_int64)] * 4,
            "nxo_fold": [T, T, C.c_int] + [C.POINTER(C.c_int64)] * 5,
        }.items():
            getattr(L, name).argtypes = args
            getattr(L, name).restype = C.c_int
        L.nxo_f32_to_f16.argtypes = [C.c_float]
        L.nxo_f32_to_f16.restype = C.c_uint16
        L.nxo_f32_to_bf16.argtypes = [C.c_float]
        L.nxo_f32_to_bf16.restype = C.c_uint16
        L.nxo_f16_to_f32.argtypes = [C.c_uint16]
        L.nxo_f16_to_f32.restype = C.c_float
        L.nxo_bf16_to_f32.argtypes = [C.c_uint16]
        L.nxo_bf16_to_f32.restype = C.c_float
        for n in ("nxo_f32_to_f8e4m3", "nxo_f32_to_f8e5m2"):
            getattr(L, n).argtypes = [C.c_float]
            getattr(L, n).restype = C.c_uint8
        for n in ("nxo_f8e4m3_to_f32", "nxo_f8e5m2_to_f32"):
            getattr(L, n).argtypes = [C.c_uint8]
            getattr(L, n).restype = C.c_float
        L.nxo_set_threads.argtypes = [C.c_int]
        L.nxo_last_threads.restype = C.c_int
        L.nxo_ncores.restype = C.c_int
        _lib = L
    return _lib


class OTensor:
    """Host tensor: flat numpy storage + view + dtype."""

    def __init__(self, storage: np.ndarray, view: View, dtype: dt.DType):
        self.storage = storage
        self.view = view
        self.dtype = dtype

    @property
    def shape(self):
        return self.view.shape

    def desc(self) -> NxhTensor:
        return make_tensor(self.storage.ctypes.data, self.dtype.tag, self.view.shape,
                           self.view.strides, self.view.offset)


def _check(rc: int, op: str):
    if rc == 0:
        return
    msg = f"{op}: {lib().nxo_last_error().decode()}"
    if rc == NXH_INVALID_ARGUMENT:
        raise ValueError(msg)
    raise RuntimeError(msg)


class OracleBackend:
    """Same surface as raven_amd.nx_backend.Backend, on the host."""

    # creation ------------------------------------------------------------
    def buffer(self, dtype: dt.DType, shape) -> OTensor:
        n = numel(shape)
        storage = np.zeros(dtype.nbytes(n) // max(dtype.np_storage.itemsize, 1)
                           if not dtype.packed else (n + 1) // 2, dtype=dtype.np_storage)
        return OTensor(storage, View.create(shape), dtype)

    def from_host(self, array: np.ndarray, dtype: dt.DType) -> OTensor:
        flat = np.ascontiguousarray(array).reshape(-1).view(dtype.np_storage).copy()
        n = flat.size * 2 if dtype.packed else flat.size
        return OTensor(flat, View.create((n,)), dtype)

    def to_host(self, t: OTensor) -> np.ndarray:
        return t.storage

    def full(self, dtype: dt.DType, shape, value_storage: np.ndarray) -> OTensor:
        out = self.buffer(dtype, shape)
        v = np.ascontiguousarray(value_storage, dtype=dtype.np_storage).reshape(1)
        _check(lib().nxo_fill(out.desc(), v.ctypes.data), "full")
        return out

    # movement ------------------------------------------------------------
    def _mv(self, t, v):
        return OTensor(t.storage, v, t.dtype)

    def with_view(self, t, v):
        return OTensor(t.storage, v, t.dtype)

    def expand(self, t, shape):
        return self._mv(t, t.view.expand(shape))

    def reshape(self, t, shape):
        return self._mv(t, t.view.reshape(shape))

    def permute(self, t, axes):
        return self._mv(t, t.view.permute(axes))

    def shrink(self, t, bounds):
        return self._mv(t, t.view.shrink(bounds))

    def flip(self, t, flags):
        return self._mv(t, t.view.flip(flags))

    # map family ------------------------------------------------------------
    def unary(self, op: str, x):
        out = self.buffer(x.dtype, x.shape)
        _check(lib().nxo_unary(UNARY_OPS.index(op), out.desc(), x.desc()), op)
        return out

    def binary(self, op: str, x, y):
        out = self.buffer(x.dtype, x.shape)
        _check(lib().nxo_binary(BINARY_OPS.index(op), out.desc(), x.desc(), y.desc()), op)
        return out

    def compare(self, op: str, x, y):
        out = self.buffer(dt.bool_, x.shape)
        _check(lib().nxo_compare(COMPARE_OPS.index(op), out.desc(), x.desc(), y.desc()), op)
        return out

    def where(self, cond, a, b):
        out = self.buffer(a.dtype, a.shape)
        _check(lib().nxo_where(out.desc(), cond.desc(), a.desc(), b.desc()), "where")
        return out

    def cast(self, x, dtype):
        out = self.buffer(dtype, x.shape)
        _check(lib().nxo_cast(out.desc(), x.desc()), "cast")
        return out

    def copy(self, x):
        out = self.buffer(x.dtype, x.shape)
        _check(lib().nxo_copy(out.desc(), x.desc()), "copy")
        return out

    def contiguous(self, x):
        if x.view.is_c_contiguous() and x.view.offset == 0:
            return x
        return self.copy(x)

    def assign(self, dst, src):
        _check(lib().nxo_copy(dst.desc(), src.desc()), "copy")

    # fold family -----------------------------------------------------------
    def reduce(self, op: str, axes, x):
        axes = sorted(int(a) for a in axes)
        if op in ("max", "min"):
            for a in axes:
                if x.shape[a] == 0:
                    raise ValueError(
                        f"reduce_{op}: reduction over an empty axis has no identity")
        oshape = [s for i, s in enumerate(x.shape) if i not in axes]
        out = self.buffer(x.dtype, oshape)
        arr = (C.c_int32 * max(len(axes), 1))(*axes)
        _check(lib().nxo_reduce(REDUCE_OPS.index(op), out.desc(), x.desc(), arr, len(axes)),
               f"reduce_{op}")
        return out

    def _arg(self, is_min, axis, keepdims, x):
        name = "argmin" if is_min else "argmax"
        if x.shape[axis] == 0:
            raise ValueError(f"{name}: argument reduction over an empty axis")
        oshape = [1 if i == axis else s for i, s in enumerate(x.shape)] if keepdims else \
            [s for i, s in enumerate(x.shape) if i != axis]
        out = self.buffer(dt.int32, oshape)
        _check(lib().nxo_argreduce(int(is_min), out.desc(), x.desc(), axis), name)
        return out

    def argmax(self, x, axis, keepdims=False):
        return self._arg(False, axis, keepdims, x)

    def argmin(self, x, axis, keepdims=False):
        return self._arg(True, axis, keepdims, x)

    # matmul / gather ---------------------------------------------------------
    def matmul(self, x, y):
        xs, ys = x.shape, y.shape
        nd = max(len(xs), len(ys))
        batch = []
        for i in range(nd - 2):
            ai, bi = i - (nd - len(xs)), i - (nd - len(ys))
            batch.append(max(xs[ai] if ai >= 0 else 1, ys[bi] if bi >= 0 else 1))
        out = self.buffer(x.dtype, batch + [xs[-2], ys[-1]])
        _check(lib().nxo_matmul(out.desc(), x.desc(), y.desc()), "matmul")
        return out

    def gather(self, data, indices, axis):
        out = self.buffer(data.dtype, indices.shape)
        _check(lib().nxo_gather(out.desc(), data.desc(), indices.desc(), axis), "gather")
        return out

    # materialising movement, scan, random, scatter -------------------------
    def pad(self, x, padding, fill_storage: np.ndarray):
        out = self.buffer(x.dtype, [s + b + a for s, (b, a) in zip(x.shape, padding)])
        fill = np.ascontiguousarray(fill_storage, dtype=x.dtype.np_storage).reshape(1)
        before = (C.c_int64 * max(len(padding), 1))(*[b for b, _ in padding])
        _check(lib().nxo_pad(out.desc(), x.desc(), fill.ctypes.data, before), "pad")
        return out

    def cat(self, tensors, axis):
        if not tensors:
            raise ValueError("cat: empty tensor list")
        first = tensors[0]
        axis = axis + len(first.shape) if axis < 0 else axis
        if not 0 <= axis < len(first.shape):
            raise ValueError("cat: axis out of range")
        shape = list(first.shape)
        shape[axis] = sum(t.shape[axis] for t in tensors)
        out = self.buffer(first.dtype, shape)
        descs = [t.desc() for t in tensors]
        arr = (C.POINTER(NxhTensor) * len(descs))(*[C.pointer(d) for d in descs])
        _check(lib().nxo_cat(out.desc(), arr, len(descs), axis), "cat")
        return out

    def associative_scan(self, axis, op: str, x):
        out = self.buffer(x.dtype, x.shape)
        _check(lib().nxo_scan(REDUCE_OPS.index(op), out.desc(), x.desc(), axis),
               {"sum": "cumsum", "prod": "cumprod", "max": "cummax", "min": "cummin"}[op])
        return out

    def threefry(self, key, counter):
        out = self.buffer(dt.int32, counter.shape)
        _check(lib().nxo_threefry(out.desc(), key.desc(), counter.desc()), "threefry")
        return out

    def scatter(self, mode: str, unique_indices: bool, template, indices, updates, axis):
        out = self.copy(template)
        _check(lib().nxo_scatter(out.desc(), indices.desc(), updates.desc(), axis,
                                 {"set": 0, "add": 1}[mode]), "scatter")
        return out

    # sort, windows -----------------------------------------------------------
    def sort(self, x, axis: int, descending: bool):
        out = self.buffer(x.dtype, x.shape)
        _check(lib().nxo_sort(out.desc(), x.desc(), axis, int(descending)), "sort")
        return out

    def argsort(self, x, axis: int, descending: bool):
        out = self.buffer(dt.int32, x.shape)
        _check(lib().nxo_argsort(out.desc(), x.desc(), axis, int(descending)), "argsort")
        return out

    def unfold(self, x, kernel_size, stride, dilation, padding):
        shape, params = window_shapes(x.shape, kernel_size, stride, dilation, padding)
        out = self.buffer(x.dtype, shape)
        _check(lib().nxo_unfold(out.desc(), x.desc(), len(kernel_size), *params), "unfold")
        return out

    def fold(self, x, output_size, kernel_size, stride, dilation, padding):
        _, params = window_shapes(tuple(x.shape[:-2]) + tuple(output_size), kernel_size, stride, dilation, padding)
        out = self.buffer(x.dtype, tuple(x.shape[:-2]) + tuple(int(s) for s in output_size))
        osz = (C.c_int64 * len(output_size))(*[int(s) for s in output_size])
        _check(lib().nxo_fold(out.desc(), x.desc(), len(kernel_size), osz, *params), "fold")
        return out

    # Fourier transforms ------------------------------------------------------
    # nx_c_fft.c computes every 1-D pass in double precision from the DFT's
    # definition (unnormalised; -sign forward, +sign inverse) and rounds to the
    # output dtype once per pass (nx_c_fft.c:30-32, 869-894). numpy's transform is
    # double precision too; its 1/n on the inverse is multiplied back out.
    def _from_array(self, a: np.ndarray, d: dt.DType):
        return self.reshape(self.from_host(np.ascontiguousarray(a.astype(d.np_storage)), d), a.shape)

    def fft(self, x, axes, inverse: bool = False):
        cur = logical(x)
        for ax in axes:  # nx_c_fft.c:940-956: one pass per listed axis, rounded to the dtype in between
            wide = cur.astype(np.complex128)
            y = np.fft.ifft(wide, axis=ax) * wide.shape[ax] if inverse else np.fft.fft(wide, axis=ax)
            cur = y.astype(x.dtype.np_storage)
        return self._from_array(cur, x.dtype)

    def ifft(self, x, axes):
        return self.fft(x, axes, inverse=True)

    def rfft(self, x, dtype, axes):
        axes = [int(a) for a in axes]
        last = axes[-1]
        a = logical(x).astype(np.float64)
        n = a.shape[last]
        full = np.fft.fft(a.astype(np.complex128), axis=last)  # nx_c_fft.c:968-972: full transform, keep n/2+1 bins
        cur = np.take(full, range(n // 2 + 1), axis=last).astype(dtype.np_storage)
        for ax in axes[:-1]:
            cur = np.fft.fft(cur.astype(np.complex128), axis=ax).astype(dtype.np_storage)
        return self._from_array(cur, dtype)

    def irfft(self, x, dtype, axes, s=None):
        axes = [int(a) for a in axes]
        last = axes[-1]
        tmp = logical(x).astype(np.complex128)
        for ax in axes[:-1]:  # nx_c_fft.c:1101-1114, complex128 throughout
            tmp = np.fft.ifft(tmp, axis=ax) * tmp.shape[ax]
        in_half = tmp.shape[last]
        size = int(s[len(axes) - 1]) if s is not None else 2 * (in_half - 1)
        half = min(in_half, size // 2 + 1)
        g = np.moveaxis(tmp, last, -1)
        f = np.zeros(g.shape[:-1] + (size,), np.complex128)
        f[..., :half] = g[..., :half]
        for k in range(1, half):  # nx_c_fft.c:1013-1023
            if size - k != k:
                f[..., size - k] = np.conj(g[..., k])
        y = (np.fft.ifft(f, axis=-1) * size).real if size else np.zeros(f.shape)
        return self._from_array(np.moveaxis(y, -1, last), dtype)

    # linear algebra ------------------------------------------------------------
    # The reference factors with its own LAPACK-style kernels in the storage's
    # compute type (nx_c_tri.c, nx_c_qr.c, nx_c_eigh.c, nx_c_svd.c, nx_c_eig.c);
    # its tests accept any factorisation that reconstructs the matrix
    # (backend_contract.ml:2075-2311). Here numpy / LAPACK in double precision
    # stands for it: same conventions (lower triangle read, real R diagonal,
    # ascending / descending order, unit-norm vectors), results rounded to the
    # result dtype by the oracle's own cast.
    def _wide(self, x):
        return logical(self.cast(x, dt.complex128 if x.dtype.is_complex else dt.float64))

    def _narrow(self, a, d):
        wide = dt.complex128 if np.iscomplexobj(a) else dt.float64
        t = self._from_array(np.asarray(a), wide)
        return t if d is wide else self.cast(t, d)

    @staticmethod
    def _check_float(op, x):
        if not (x.dtype.is_float or x.dtype.is_complex):
            raise RuntimeError(f"{op}: linalg requires a float or complex dtype")

    def cholesky(self, x, upper: bool = False):
        self._check_float("cholesky", x)
        a = self._wide(x)
        low = np.tril(a)
        herm = low + np.swapaxes(np.tril(a, -1), -1, -2).conj()  # nx_c_tri.c:11-16: only the lower triangle is read
        try:
            if not np.all(np.isfinite(herm)):
                raise np.linalg.LinAlgError
            l = np.linalg.cholesky(herm)
        except np.linalg.LinAlgError:
            raise RuntimeError("cholesky: matrix is not positive definite") from None
        return self._narrow(np.swapaxes(l, -1, -2).conj() if upper else l, x.dtype)

    def triangular_solve(self, a, b, upper: bool, transpose: bool, unit_diag: bool):
        import scipy.linalg

        self._check_float("triangular_solve", a)
        A, Bm = self._wide(a), self._wide(b)
        vector = Bm.ndim == A.ndim - 1
        if vector:
            Bm = Bm[..., None]
        out = np.empty(Bm.shape, np.result_type(A, Bm))
        n = A.shape[-1]
        for idx in np.ndindex(*A.shape[:-2]):
            if not unit_diag and np.any(np.diagonal(A[idx]) == 0):  # nx_c_tri.c:113-118: exact zero only
                raise RuntimeError("triangular_solve: triangular matrix is singular")
            out[idx] = (scipy.linalg.solve_triangular(A[idx], Bm[idx], lower=not upper, trans="C" if transpose else "N",
                                                      unit_diagonal=unit_diag, check_finite=False)
                        if n else Bm[idx])
        return self._narrow(out[..., 0] if vector else out, b.dtype)

    @staticmethod
    def _householder_qr(a, reduced):
        """nx_c_qr.c:44-110 restated: LAPACK's reflectors (real beta = -sign(re alpha) |x|,
        tau = ((beta - re alpha) / beta, -im alpha / beta), H_j^H applied while factoring,
        Q = H_0 H_1 ...), except that a column with nothing below the diagonal takes no
        reflector even when its diagonal element is complex (LAPACK would rotate it real)."""
        m, n = a.shape
        k = min(m, n)
        A = a.copy()
        tau = np.zeros(k, A.dtype)
        for j in range(k):
            x = A[j + 1:, j]
            xnorm2 = float(np.sum(x.real ** 2 + x.imag ** 2))
            alpha = A[j, j]
            if xnorm2 == 0.0:
                continue
            anorm = np.sqrt(alpha.real ** 2 + alpha.imag ** 2 + xnorm2)
            beta = -anorm if alpha.real >= 0 else anorm
            tau[j] = complex((beta - alpha.real) / beta, -alpha.imag / beta) if np.iscomplexobj(A) else (beta - alpha) / beta
            A[j + 1:, j] = x / (alpha - beta)
            A[j, j] = beta
            v = np.concatenate([[1.0], A[j + 1:, j]])
            w = np.conj(tau[j]) * (v.conj() @ A[j:, j + 1:])
            A[j:, j + 1:] -= np.outer(v, w)
        nq = k if reduced else m
        Q = np.eye(m, nq, dtype=A.dtype)
        for j in range(k - 1, -1, -1):
            v = np.concatenate([[1.0], A[j + 1:, j]])
            w = tau[j] * (v.conj() @ Q[j:, j:])
            Q[j:, j:] -= np.outer(v, w)
        return Q, np.triu(A[:(k if reduced else m), :])

    def qr(self, x, reduced: bool = True):
        self._check_float("qr", x)
        a = self._wide(x)
        m, n = a.shape[-2:]
        k = min(m, n)
        q = np.empty(a.shape[:-2] + (m, k if reduced else m), a.dtype)
        r = np.empty(a.shape[:-2] + (k if reduced else m, n), a.dtype)
        for idx in np.ndindex(*a.shape[:-2]):
            q[idx], r[idx] = self._householder_qr(a[idx], reduced)
        return self._narrow(q, x.dtype), self._narrow(r, x.dtype)

    def eigh(self, x):
        self._check_float("eigh", x)
        w, v = np.linalg.eigh(self._wide(x), UPLO="L")  # nx_c_eigh.c:14-21: lower triangle, ascending
        return self._narrow(w, dt.float64), self._narrow(v, x.dtype)

    def eigvalsh(self, x):
        self._check_float("eigvalsh", x)
        return self._narrow(np.linalg.eigvalsh(self._wide(x), UPLO="L"), dt.float64)

    def svd(self, x, full_matrices: bool = False):
        self._check_float("svd", x)
        u, s, vt = np.linalg.svd(self._wide(x), full_matrices=full_matrices)
        return self._narrow(u, x.dtype), self._narrow(s, dt.float64), self._narrow(vt, x.dtype)

    def eig(self, x):
        self._check_float("eig", x)
        w, v = np.linalg.eig(self._wide(x))  # unit 2-norm columns, as nx_c_eig.c:56
        return self._narrow(w.astype(np.complex128), dt.complex128), self._narrow(v.astype(np.complex128), dt.complex128)

    def eigvals(self, x):
        self._check_float("eigvals", x)
        return self._narrow(np.linalg.eigvals(self._wide(x)).astype(np.complex128), dt.complex128)


def window_shapes(in_shape, kernel_size, stride, dilation, padding):
    """Result shape of unfold (nx_backend.ml:427-445) and the K-long parameter
    arrays as C int64 arrays (padding flattened to [before0, after0, ...])."""
    k = len(kernel_size)
    if not (len(stride) == len(dilation) == len(padding) == k) or k < 1 or len(in_shape) < k:
        raise ValueError("unfold: shape mismatch")
    lead, spatial = tuple(in_shape[:len(in_shape) - k]), in_shape[len(in_shape) - k:]
    windows = 1
    for i in range(k):
        padded = spatial[i] + padding[i][0] + padding[i][1]
        extent = dilation[i] * (kernel_size[i] - 1) + 1
        windows *= (padded - extent) // stride[i] + 1
    kp = 1
    for s in kernel_size:
        kp *= s
    arr = lambda v: (C.c_int64 * len(v))(*[int(a) for a in v])
    flat = [int(v) for pair in padding for v in pair]
    return lead + (kp, windows), (arr(kernel_size), arr(stride), arr(dilation), arr(flat))


def logical(t: OTensor) -> np.ndarray:
    """The tensor's logical contents as a numpy array of its storage dtype."""
    if t.dtype.packed:
        raise NotImplementedError
    es = t.storage.dtype.itemsize
    v = t.view
    if v.numel == 0:
        return np.zeros(v.shape, dtype=t.storage.dtype)
    return np.lib.stride_tricks.as_strided(
        t.storage[v.offset:] if all(s >= 0 for s in v.strides) else
        _neg_base(t.storage, v), shape=v.shape,
        strides=[s * es for s in v.strides]).copy()


def _neg_base(storage, v):
    return storage[v.offset:]
