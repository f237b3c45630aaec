#!/usr/bin/env python3
"""Benchmark of the Nx eager hot path on one MI355X.

A "step" is one pass of BASELINE.json's config 2 (broadcast / strided
elementwise) over synthetic input already resident in HBM:

  f32:   a[64,512,512] viewed through permute(0,2,1); b[1,512,1] expanded
         t = add a' b ; u = mul t 0.5 ; v = cast f16 u
  int32: add a' b ; mul a' b ; m = cmplt b a' ; where m a' b

`value` is the algorithmic GB/s of that step (unique input elements read once +
outputs written once: 832 MiB + the small broadcast operands). The same JSON
line carries `roofline` for the dominant kernel (the LDS-turned elementwise
kernel, timed alone with HIP events on the context's stream), `cpu_baseline`
(the CPU oracle — a restatement of the reference's C backend — on the same
workload, rank 0, host cores), and `ops`: every op of configs 1-4 timed alone
(GB/s or TFLOP/s and its fraction of the 8 TB/s / MFMA peak).

Calls go straight through the C ABI with pre-built descriptors and
pre-allocated outputs ("output first"), so the timed region holds kernel
launches only: no allocation, no host<->device copies.
"""

from __future__ import annotations

import argparse
import ctypes as C
import json
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

from raven_amd import _ffi  # noqa: E402
from raven_amd import dtype as dt  # noqa: E402
from raven_amd.nx_backend import Backend, logical  # noqa: E402

MIB = 1 << 20
PEAK_HBM_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "f16": 2500.0, "f32": 157.3}
METRIC = "Nx op GB/s (elementwise/reduce) + GEMM TFLOP/s, as % of MI355X roofline"


# HBM bytes per launch of the headline step's dominant kernel (map_tiled add, f32,
# [64,512,512]), from rocprofv3 --pmc FETCH_SIZE and --pmc WRITE_SIZE runs of
# `bench.py --only-step --no-cpu --pmc-calibration`: 32 817 KiB fetched x 1.9990 (a plain
# 64 MiB copy reads 32 784 KiB on the same counter) + 65 536 KiB written x 1.0000.
DOMINANT_KERNEL_HBM_TRAFFIC = 134285312


class Op:
    """One pre-built C-ABI call: name, thunk, algorithmic bytes / flops."""

    def __init__(self, name, fn, args, nbytes=0, flops=0, keep=()):
        self.name, self.fn, self.args, self.nbytes, self.flops, self.keep = name, fn, args, nbytes, flops, keep

    def __call__(self):
        rc = self.fn(*self.args)
        if rc != 0:
            raise RuntimeError(f"{self.name}: status {rc}")


def ref(t):
    d = t._desc()
    return d, C.byref(d)


class Workloads:
    def __init__(self, hip: Backend):
        self.hip, self.lib, self.h = hip, hip._lib, hip._h
        self.keep = []

    def dev(self, arr, d, shape=None):
        t = self.hip.from_host(arr, d)
        return self.hip.reshape(t, shape if shape is not None else arr.shape)

    def mk(self, name, fn, tensors, extra=(), pre=(), nbytes=0, flops=0):
        descs = [ref(t) for t in tensors]
        self.keep.append((tensors, descs))
        args = (self.h, *pre, *[p for _, p in descs], *extra)
        return Op(name, fn, args, nbytes, flops)

    def unary(self, op, out, x, nbytes):
        return self.mk(op, self.lib.nxh_unary, [out, x], pre=(_ffi.UNARY_OPS.index(op),), nbytes=nbytes)

    def binary(self, op, out, x, y, nbytes, name=None):
        return self.mk(name or op, self.lib.nxh_binary, [out, x, y], pre=(_ffi.BINARY_OPS.index(op),), nbytes=nbytes)

    def compare(self, op, out, x, y, nbytes):
        return self.mk(op, self.lib.nxh_compare, [out, x, y], pre=(_ffi.COMPARE_OPS.index(op),), nbytes=nbytes)

    def reduce(self, op, out, x, axes, nbytes, name):
        arr = (C.c_int32 * len(axes))(*axes)
        self.keep.append(arr)
        return self.mk(name, self.lib.nxh_reduce, [out, x], pre=(_ffi.REDUCE_OPS.index(op),),
                       extra=(arr, len(axes)), nbytes=nbytes)

    # -- config 2: the headline step ------------------------------------------
    def config2(self):
        hip = self.hip
        rng = [np.random.default_rng(s) for s in (4, 5, 6, 7)]
        shp = (64, 512, 512)
        n = 64 * 512 * 512
        a = self.dev(rng[0].standard_normal(shp).astype(np.float32), dt.float32)
        b = self.dev(rng[1].standard_normal((1, 512, 1)).astype(np.float32), dt.float32)
        ai = self.dev(rng[2].integers(-1000, 1001, shp).astype(np.int32), dt.int32)
        bi = self.dev(rng[3].integers(-1000, 1001, (1, 512, 1)).astype(np.int32), dt.int32)
        ap, aip = hip.permute(a, (0, 2, 1)), hip.permute(ai, (0, 2, 1))
        bx, bix = hip.expand(b, shp), hip.expand(bi, shp)
        half = hip.expand(hip.full(dt.float32, (), 0.5), shp)
        t, u = hip.buffer(dt.float32, shp), hip.buffer(dt.float32, shp)
        v = hip.buffer(dt.float16, shp)
        ti, ui = hip.buffer(dt.int32, shp), hip.buffer(dt.int32, shp)
        m, w = hip.buffer(dt.bool_, shp), hip.buffer(dt.int32, shp)
        small = 512 * 4
        ops = [
            self.binary("add", t, ap, bx, 8 * n + small, "cfg2 f32 add(permuted a, broadcast b)"),
            self.binary("mul", u, t, half, 8 * n + 4, "cfg2 f32 mul(t, scalar 0.5)"),
            self.mk("cfg2 cast f32->f16", self.lib.nxh_cast, [v, u], nbytes=6 * n),
            self.binary("add", ti, aip, bix, 8 * n + small, "cfg2 i32 add(permuted a, broadcast b)"),
            self.binary("mul", ui, aip, bix, 8 * n + small, "cfg2 i32 mul(permuted a, broadcast b)"),
            self.compare("cmplt", m, bix, aip, 5 * n + small),
            self.mk("cfg2 i32 where(m, permuted a, broadcast b)", self.lib.nxh_where, [w, m, aip, bix],
                    nbytes=9 * n + small),
        ]
        ops[5].name = "cfg2 i32 cmplt(broadcast b, permuted a)"
        self.cfg2_out = {"v": v, "w": w, "m": m}
        return ops

    # -- config 1: the CPU-runnable chain --------------------------------------
    def config1(self):
        hip = self.hip
        n = 4096
        a, b, c = (self.dev(np.random.default_rng(s).uniform(-1, 1, (n, n)).astype(np.float32), dt.float32)
                   for s in (1, 2, 3))
        t1, t2, t3 = (hip.buffer(dt.float32, (n, n)) for _ in range(3))
        z = hip.buffer(dt.float32, (n,))
        e = n * n * 4
        self.cfg1 = (a, b, c, z)
        return [
            self.binary("mul", t1, a, b, 3 * e, "cfg1 f32 mul"),
            self.unary("sin", t2, c, 2 * e),
            self.binary("add", t3, t1, t2, 3 * e, "cfg1 f32 add"),
            self.reduce("sum", z, t3, [1], e + n * 4, "cfg1 f32 reduce_sum axis 1"),
        ]

    # -- config 3: reductions ---------------------------------------------------
    def config3(self):
        hip = self.hip
        n = 8192
        x = self.dev(np.random.default_rng(8).standard_normal((n, n)).astype(np.float32), dt.float32)
        xi = self.dev(np.random.default_rng(9).integers(-1000, 1001, (n, n)).astype(np.int32), dt.int32)
        e = n * n * 4 + n * 4
        ops = []
        for axis in (1, 0):
            of, oi, oa = hip.buffer(dt.float32, (n,)), hip.buffer(dt.int32, (n,)), hip.buffer(dt.int32, (n,))
            ops.append(self.reduce("sum", of, x, [axis], e, f"cfg3 f32 sum axis {axis}"))
            ops.append(self.reduce("max", hip.buffer(dt.float32, (n,)), x, [axis], e, f"cfg3 f32 max axis {axis}"))
            ops.append(self.mk(f"cfg3 f32 argmax axis {axis}", self.lib.nxh_argreduce, [oa, x], pre=(0,),
                               extra=(axis,), nbytes=e))
            ops.append(self.reduce("sum", oi, xi, [axis], e, f"cfg3 i32 sum axis {axis}"))
        return ops

    # -- config 4: GEMM -----------------------------------------------------------
    def config4(self):
        hip = self.hip
        ops = []
        a = self.dev((np.random.default_rng(10).standard_normal((2048, 2048)) * 0.02).astype(np.float32), dt.float32)
        b = self.dev((np.random.default_rng(11).standard_normal((2048, 2048)) * 0.02).astype(np.float32), dt.float32)
        ops.append(self.mk("cfg4 f32 matmul 2048^3", self.lib.nxh_matmul, [hip.buffer(dt.float32, (2048, 2048)), a, b],
                           flops=2 * 2048 ** 3, nbytes=3 * 2048 * 2048 * 4))
        # bf16 inputs are generated on the device: f32 noise cast to bf16 (RNE)
        rng = np.random.default_rng(12)
        base = (rng.standard_normal((4096, 4096)) * 0.02).astype(np.float32)
        ab = hip.cast(hip.expand(hip.reshape(self.dev(base, dt.float32), (1, 4096, 4096)), (16, 4096, 4096)), dt.bfloat16)
        base2 = (np.random.default_rng(13).standard_normal((4096, 4096)) * 0.02).astype(np.float32)
        bb = hip.cast(hip.expand(hip.reshape(self.dev(base2, dt.float32), (1, 4096, 4096)), (16, 4096, 4096)), dt.bfloat16)
        ops.append(self.mk("cfg4 bf16 matmul [16,4096,4096]^2", self.lib.nxh_matmul,
                           [hip.buffer(dt.bfloat16, (16, 4096, 4096)), ab, bb],
                           flops=2 * 16 * 4096 ** 3, nbytes=3 * 16 * 4096 * 4096 * 2))
        for d, nm in ((dt.bfloat16, "bf16"), (dt.float32, "f32")):
            sa = hip.cast(self.dev((np.random.default_rng(14).standard_normal((8, 4096)) * 0.02).astype(np.float32),
                                   dt.float32), d)
            sb = hip.cast(self.dev((np.random.default_rng(15).standard_normal((4096, 16384)) * 0.02).astype(np.float32),
                                   dt.float32), d)
            es = d.itemsize
            ops.append(self.mk(f"cfg4 {nm} skinny [8,4096]x[4096,16384]", self.lib.nxh_matmul,
                               [hip.buffer(d, (8, 16384)), sa, sb], flops=2 * 8 * 4096 * 16384,
                               nbytes=(8 * 4096 + 4096 * 16384 + 8 * 16384) * es))
        return ops


def next_ops(hip, W, linalg=False):
    """The operations beside the named hot path (pad, cat, scan, threefry,
    scatter, sort, unfold, fold), timed through the Python mirror with HIP events."""
    rng = np.random.default_rng(20)
    out = []

    def timed(name, fn, nbytes, iters=20):
        for _ in range(3):
            r = fn()
            del r
        hip.synchronize()
        hip.timer_start()
        for _ in range(iters):
            r = fn()
            del r
        ms = hip.timer_stop() / iters
        out.append({"op": name, "ms": round(ms, 5), "GB/s": round(nbytes / (ms * 1e-3) / 1e9, 1),
                    "frac_hbm": round(nbytes / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "bound": "hbm"})

    x = W.dev(rng.standard_normal((2048, 4100)).astype(np.float32), dt.float32)
    timed("pad [2048,4100] f32 by ((3,5),(7,1))", lambda: hip.pad(x, [(3, 5), (7, 1)], -2.5),
          2048 * 4100 * 4 + 2056 * 4108 * 4)
    parts = [W.dev(rng.standard_normal((1024, 4096)).astype(np.float32), dt.float32) for _ in range(4)]
    timed("cat 4 x [1024,4096] f32 along axis 0", lambda: hip.cat(parts, 0), 2 * 4 * 1024 * 4096 * 4)
    timed("cat 4 x [1024,4096] f32 along axis 1", lambda: hip.cat(parts, 1), 2 * 4 * 1024 * 4096 * 4)
    y = W.dev(rng.standard_normal((4096, 8192)).astype(np.float32), dt.float32)
    timed("cumsum [4096,8192] f32 axis 1 (scan_rows)", lambda: hip.associative_scan(1, "sum", y), 2 * 4096 * 8192 * 4)
    timed("cumsum [4096,8192] f32 axis 0 (scan_chunks: 3 passes over the data)", lambda: hip.associative_scan(0, "sum", y), 2 * 4096 * 8192 * 4)
    n = 1 << 24
    ctr = W.dev(np.arange(2 * n, dtype=np.int64).astype(np.int32).reshape(n, 2), dt.int32)
    key = hip.expand(W.dev(np.array([[1234, -99]], np.int32), dt.int32), (n, 2))
    timed("threefry 2^24 vectors (one key)", lambda: hip.threefry(key, ctr), 2 * n * 8)
    vocab, dim, ntok = 50257, 768, 8192
    ids = W.dev(rng.integers(0, vocab, (ntok, 1)).astype(np.int32), dt.int32)
    idx = hip.expand(ids, (ntok, dim))
    upd = W.dev(rng.standard_normal((ntok, dim)).astype(np.float32), dt.float32)
    table = hip.full(dt.float32, (vocab, dim), 0.0)
    # template copy (read + write of the table) + indices + updates + read-modify-write of the touched rows
    timed("scatter-add [8192,768] f32 rows into [50257,768] (embedding gradient)",
          lambda: hip.scatter("add", False, table, idx, upd, 0),
          2 * vocab * dim * 4 + ntok * 4 + 3 * ntok * dim * 4, iters=5)
    del table, upd, idx, ctr, key, y, parts, x
    # sort moves each element once in and once out; the network in between is
    # compare-exchange work, so the rate is quoted in keys per second too
    rows = W.dev(rng.standard_normal((16384, 1024)).astype(np.float32), dt.float32)
    timed("sort [16384,1024] f32 axis 1 (sort_lds)", lambda: hip.sort(rows, 1, False), 2 * 16384 * 1024 * 4)
    out[-1]["Mkeys/s"] = round(16384 * 1024 / out[-1]["ms"] / 1e3, 1)
    timed("argsort [16384,1024] f32 axis 1, descending (sort_lds)", lambda: hip.argsort(rows, 1, True),
          2 * 16384 * 1024 * 4)
    out[-1]["Mkeys/s"] = round(16384 * 1024 / out[-1]["ms"] / 1e3, 1)
    one = W.dev(rng.standard_normal(1 << 24).astype(np.float32), dt.float32)
    timed("sort 2^24 f32, one slice (sort_global)", lambda: hip.sort(one, 0, False), 2 * (1 << 24) * 4, iters=5)
    out[-1]["Mkeys/s"] = round((1 << 24) / out[-1]["ms"] / 1e3, 1)
    for rec in out[-3:]:
        rec["bound"] = "lds"  # compare-exchange steps through LDS, not bytes, set the time
    del rows, one
    img = W.dev(rng.standard_normal((8, 64, 128, 128)).astype(np.float32), dt.float32)
    geo = ([3, 3], [1, 1], [1, 1], [(1, 1), (1, 1)])
    nin, ncols = 8 * 64 * 128 * 128 * 4, 9 * 8 * 64 * 128 * 128 * 4
    timed("unfold [8,64,128,128] f32, 3x3 same (im2col)", lambda: hip.unfold(img, *geo), nin + ncols)
    cols = hip.unfold(img, *geo)
    timed("fold back to [8,64,128,128] (col2im, 9 taps per output)", lambda: hip.fold(cols, [128, 128], *geo), nin + ncols)
    del img, cols
    # fused attention and the row kernels at GPT-2-small's shapes (bf16, batch 8, seq 1024)
    bf = lambda shape: W.dev((rng.standard_normal(shape).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16),
                             dt.bfloat16)
    b, h, sq, hd = 8, 12, 1024, 64
    q, k, v = (hip.permute(hip.reshape(bf((b, sq, h * hd)), (b, sq, h, hd)), (0, 2, 1, 3)) for _ in range(3))
    timed("attention [8,12,1024,64] bf16, causal, head-split views (attention_fused)",
          lambda: hip.attention(q, k, v, 0.125, causal=True, masked_value=float("-inf")), 4 * b * sq * h * hd * 2)
    useful = 4 * b * h * sq * (sq + 1) // 2 * hd  # Q K^T and probs x V over the visible half
    # bound by the per-score VALU work (two expf, an exact division, a narrowing), not by the MFMAs
    out[-1].update({"bound": "valu", "TFLOP/s": round(useful / (out[-1]["ms"] * 1e-3) / 1e12, 1)})
    scores = W.dev(rng.standard_normal((b * h * sq, sq)).astype(np.float32), dt.float32)
    timed("softmax_rows [98304,1024] f32 -> bf16 with scale (fused)",
          lambda: hip.softmax_rows(scores, 0.125, None, None, dt.bfloat16), b * h * sq * sq * 6)
    del scores
    x = bf((b * sq, 768))
    gam, bet = bf((768,)), bf((768,))
    timed("layer_norm_rows [8192,768] bf16 (fused)", lambda: hip.layer_norm_rows(x, gam, bet, 1e-5), 2 * b * sq * 768 * 2)
    y = bf((b * sq, 3072))
    timed("gelu_tanh [8192,3072] bf16 (fused)", lambda: hip.gelu_tanh(y), 2 * b * sq * 3072 * 2)
    del x, y, gam, bet, q, k, v
    # Fourier transforms: one pass reads and writes the tensor once; the butterflies run in LDS
    cplx = lambda shape: W.dev((rng.standard_normal(shape) + 1j * rng.standard_normal(shape)).astype(np.complex64),
                               dt.complex64)
    z = cplx((16384, 1024))
    timed("fft [16384,1024] complex64 axis 1 (fft_lines, four radix-2 stages per LDS pass)", lambda: hip.fft(z, [1]), 2 * 16384 * 1024 * 8)
    out[-1]["GFLOP/s"] = round(5 * 16384 * 1024 * 10 / out[-1]["ms"] / 1e6, 1)
    z2 = cplx((4096, 4096))
    timed("fft [4096,4096] complex64 axis 0 (strided lines)", lambda: hip.fft(z2, [0]), 2 * 4096 * 4096 * 8)
    z3 = cplx((8192, 1000))
    timed("fft [8192,1000] complex64 axis 1 (Bluestein in LDS, M = 2048)", lambda: hip.fft(z3, [1]), 2 * 8192 * 1000 * 8)
    r = W.dev(rng.standard_normal((16384, 2048)).astype(np.float32), dt.float32)
    timed("rfft [16384,2048] f32 -> complex64 axis 1", lambda: hip.rfft(r, dt.complex64, [1]),
          16384 * 2048 * 4 + 16384 * 1025 * 8)
    big = cplx((4, 1 << 20))
    timed("fft [4,2^20] complex64 axis 1 (four-step through a workspace)", lambda: hip.fft(big, [1]),
          2 * 4 * (1 << 20) * 8, iters=5)
    for rec in out[-5:]:
        rec["bound"] = "lds"
    del z, z2, z3, r, big
    if not linalg:
        return out

    # linear algebra (only with --only-next: thousands of short launches that would drown a
    # kernel-time profile of the hot path): correctness first, times only
    def la(name, fn, iters=3):
        timed(name, fn, 0, iters=iters)
        for key in ("GB/s", "frac_hbm"):
            out[-1].pop(key)
        out[-1]["bound"] = "latency"

    g = rng.standard_normal((256, 64, 64)).astype(np.float32)
    spd = W.dev(g @ g.transpose(0, 2, 1) + 64 * np.eye(64, dtype=np.float32), dt.float32)
    gen = W.dev(g, dt.float32)
    la("cholesky [256,64,64] f32", lambda: hip.cholesky(spd))
    la("qr [256,64,64] f32, reduced", lambda: hip.qr(gen))
    la("eigh [256,64,64] f32 (Jacobi)", lambda: hip.eigh(spd))
    la("svd [256,64,64] f32 (one-sided Jacobi)", lambda: hip.svd(gen))
    la("eig [256,64,64] f32 (Hessenberg + shifted QR)", lambda: hip.eig(gen))
    one = rng.standard_normal((1, 512, 512)).astype(np.float32)
    big_spd = W.dev(one @ one.transpose(0, 2, 1) + 512 * np.eye(512, dtype=np.float32), dt.float32)
    la("cholesky [1,512,512] f32", lambda: hip.cholesky(big_spd))
    la("eigh [1,512,512] f32 (Jacobi)", lambda: hip.eigh(big_spd), iters=1)
    return out


def time_ops(hip, ops, iters, warmup):
    """Average milliseconds per pass of `ops`, HIP events on the context stream."""
    for _ in range(warmup):
        for op in ops:
            op()
    hip.synchronize()
    hip.timer_start()
    for _ in range(iters):
        for op in ops:
            op()
    return hip.timer_stop() / iters


def op_record(op, ms):
    rec = {"op": op.name, "ms": round(ms, 5)}
    gbs = op.nbytes / (ms * 1e-3) / 1e9
    if op.flops and "skinny" not in op.name:
        dtype = "bf16" if "bf16" in op.name else "f32"
        tf = op.flops / (ms * 1e-3) / 1e12
        rec.update({"TFLOP/s": round(tf, 2), "frac_mfma": round(tf / PEAK_TFLOPS[dtype], 4), "bound": "mfma"})
    else:
        rec.update({"GB/s": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4), "bound": "hbm"})
        if op.flops:
            rec["TFLOP/s"] = round(op.flops / (ms * 1e-3) / 1e12, 3)
    return rec


def cpu_baseline(seconds_budget=20.0):
    """The oracle (CPU restatement of the reference C backend) on config 2, with
    the reference's own thread policy, on this host's cores."""
    from oracle.nx_oracle import OracleBackend, lib

    B = OracleBackend()
    rng = [np.random.default_rng(s) for s in (4, 5, 6, 7)]
    shp = (64, 512, 512)
    n = 64 * 512 * 512
    mk = lambda arr, d: B.reshape(B.from_host(arr, d), arr.shape)  # noqa: E731
    a = mk(rng[0].standard_normal(shp).astype(np.float32), dt.float32)
    b = mk(rng[1].standard_normal((1, 512, 1)).astype(np.float32), dt.float32)
    ai = mk(rng[2].integers(-1000, 1001, shp).astype(np.int32), dt.int32)
    bi = mk(rng[3].integers(-1000, 1001, (1, 512, 1)).astype(np.int32), dt.int32)
    ap, aip = B.permute(a, (0, 2, 1)), B.permute(ai, (0, 2, 1))
    bx, bix = B.expand(b, shp), B.expand(bi, shp)
    half = B.expand(B.full(dt.float32, (), np.array([0.5], np.float32)), shp)
    threads = set()

    def step():
        t = B.binary("add", ap, bx)
        threads.add(lib().nxo_last_threads())
        u = B.binary("mul", t, half)
        v = B.cast(u, dt.float16)
        B.binary("add", aip, bix)
        B.binary("mul", aip, bix)
        m = B.compare("cmplt", bix, aip)
        w = B.where(m, aip, bix)
        return v, w

    step()  # warm: first touch of fresh pages is not the steady state
    t0 = time.perf_counter()
    reps = 0
    while reps < 3 or (time.perf_counter() - t0 < seconds_budget and reps < 40):
        out = step()
        reps += 1
    dtm = (time.perf_counter() - t0) / reps
    total_bytes = 832 * MIB + 5 * 2048 + 4
    return {
        "value": round(total_bytes / dtm / 1e9, 3), "unit": "GB/s", "cores": max(threads),
        "kind": "port",
        "sample": f"{reps} full passes of config 2 ([64,512,512] f32 + int32 chain, 832 MiB algorithmic), "
                  f"{dtm * 1e3:.1f} ms per pass; host has {lib().nxo_ncores()} cores online; threads per op "
                  "follow the reference policy (bytes/32 MiB, capped by cores)",
    }, out


class CountingBackend:
    """Forwards to the backend and counts the calls that launch work."""

    LAUNCHING = ("unary", "binary", "compare", "where", "cast", "copy", "contiguous", "gather", "reduce",
                 "matmul", "full", "from_host", "softmax_rows", "layer_norm_rows", "gelu_tanh", "attention", "linear")

    def __init__(self, inner):
        self._inner, self.calls = inner, {}

    def __getattr__(self, name):
        attr = getattr(self._inner, name)
        if name not in self.LAUNCHING:
            return attr

        def counted(*a, **k):
            self.calls[name] = self.calls.get(name, 0) + 1
            return attr(*a, **k)

        return counted


def cpu_configs():
    """The CPU oracle on bounded samples of the other configurations, on this
    host's cores with the reference's thread policy: the CPU path beside each
    GPU figure. Every sample is named in its record."""
    from oracle.nx_oracle import OracleBackend, lib

    B = OracleBackend()
    out = []
    mk = lambda arr, d: B.reshape(B.from_host(arr, d), arr.shape)  # noqa: E731

    def timed(name, fn, nbytes=0, flops=0, budget=4.0):
        fn()
        t0, reps = time.perf_counter(), 0
        while reps < 2 or (time.perf_counter() - t0 < budget and reps < 20):
            fn()
            reps += 1
        sec = (time.perf_counter() - t0) / reps
        rec = {"op": name, "ms": round(sec * 1e3, 3), "threads": lib().nxo_last_threads()}
        if nbytes:
            rec["GB/s"] = round(nbytes / sec / 1e9, 2)
        if flops:
            rec["GFLOP/s"] = round(flops / sec / 1e9, 1)
        out.append(rec)

    n = 4096
    a, b, c = (mk(np.random.default_rng(s).uniform(-1, 1, (n, n)).astype(np.float32), dt.float32) for s in (1, 2, 3))
    e = n * n * 4
    timed("cfg1 f32 mul [4096,4096]", lambda: B.binary("mul", a, b), 3 * e)
    timed("cfg1 f32 sin [4096,4096]", lambda: B.unary("sin", c), 2 * e)
    timed("cfg1 f32 reduce_sum axis 1 [4096,4096]", lambda: B.reduce("sum", [1], a), e)
    del a, b, c
    n = 8192
    x = mk(np.random.default_rng(8).standard_normal((n, n)).astype(np.float32), dt.float32)
    e = n * n * 4
    for axis in (1, 0):
        timed(f"cfg3 f32 sum axis {axis} [8192,8192]", lambda: B.reduce("sum", [axis], x), e)
        timed(f"cfg3 f32 argmax axis {axis} [8192,8192]", lambda: B.argmax(x, axis), e)
    del x
    m = 2048
    fa, fb = (mk((np.random.default_rng(s).standard_normal((m, m)) * 0.02).astype(np.float32), dt.float32) for s in (10, 11))
    timed("cfg4 f32 matmul 2048^3", lambda: B.matmul(fa, fb), flops=2 * m ** 3, budget=8.0)
    ba, bb = B.cast(B.reshape(fa, (1, m, m)), dt.bfloat16), B.cast(B.reshape(fb, (1, m, m)), dt.bfloat16)
    timed("cfg4 bf16 matmul, sample [1,2048,2048]^2 of [16,4096,4096]^2", lambda: B.matmul(ba, bb), flops=2 * m ** 3,
          budget=8.0)
    sa = mk((np.random.default_rng(14).standard_normal((8, 4096)) * 0.02).astype(np.float32), dt.float32)
    sb = mk((np.random.default_rng(15).standard_normal((4096, 16384)) * 0.02).astype(np.float32), dt.float32)
    timed("cfg4 f32 skinny [8,4096]x[4096,16384]", lambda: B.matmul(sa, sb), nbytes=(8 * 4096 + 4096 * 16384 + 8 * 16384) * 4,
          flops=2 * 8 * 4096 * 16384)
    del fa, fb, ba, bb, sa, sb
    # config 5: the eager GPT-2-small forward at batch 1 x seq 128 (1/64 of the tokens of the GPU run)
    from raven_amd.kaun_gpt2 import Config, Gpt2, host_params, upload
    from raven_amd.nx_frontend import Nx

    cfg = Config.small()
    enc = lambda v, d: ((np.ascontiguousarray(v, np.float32).view(np.uint32) + 0x7FFF  # noqa: E731
                         + ((np.ascontiguousarray(v, np.float32).view(np.uint32) >> 16) & 1)) >> 16).astype(np.uint16)
    nx = Nx(B)
    params = upload(nx, host_params(cfg, seed=16), dt.bfloat16, enc)
    ids = nx.create(dt.int32, (1, 128), np.random.default_rng(17).integers(0, cfg.vocab_size, (1, 128)).astype(np.int32))
    model = Gpt2(nx, cfg)
    t0 = time.perf_counter()
    model.logits(params, ids)
    sec = time.perf_counter() - t0
    out.append({"op": "cfg5 GPT-2 small forward, bf16, sample batch 1 x seq 128 (one pass)", "ms": round(sec * 1e3, 1),
                "tokens/s": round(128 / sec, 1)})
    return {"host_cores": lib().nxo_ncores(), "ops": out}


def config5(hip, iters=3, warmup=1, window=False, graph=False):
    """GPT-2-small-shaped forward (12 layers, d 768, 12 heads, FFN 3072, vocab
    50257, batch 8 x seq 1024, bf16 random-init weights): tokens/s. Eager: one
    backend call per primitive. With ``window``: the same frontend calls go
    through the deferred-evaluation window, which replaces the softmax, layer
    norm and GELU sequences by the fused row kernels. With ``graph`` too: the
    windowed forward is recorded once and each timed step is one replay."""
    from raven_amd.kaun_gpt2 import Config, Gpt2, host_params, upload
    from raven_amd.nx_frontend import Nx
    from raven_amd.nx_window import Window

    cfg = Config.small()
    batch, seq = 8, 1024

    def enc(a, d):  # f32 -> bf16 storage, round to nearest even
        u = np.ascontiguousarray(a, np.float32).view(np.uint32)
        return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)

    counter = CountingBackend(hip)
    front = Window(counter) if window else counter
    nx = Nx(front)
    params = upload(nx, host_params(cfg, seed=16), dt.bfloat16, enc)
    ids = nx.create(dt.int32, (batch, seq),
                    np.random.default_rng(17).integers(0, cfg.vocab_size, (batch, seq)).astype(np.int32))
    model = Gpt2(nx, cfg)
    for _ in range(warmup):
        out = model.logits(params, ids)
        del out
    front.synchronize()
    recorded = None
    if graph:
        front.capture_begin()
        try:
            out = front.force(model.logits(params, ids))
        finally:
            recorded = front.capture_end()
    counter.calls.clear()
    t0 = time.perf_counter()
    front.timer_start()
    for _ in range(iters):
        if recorded is not None:
            recorded.launch()
        else:
            out = model.logits(params, ids)
            del out
    ev_ms = front.timer_stop() / iters
    front.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / iters
    calls = {k: v // iters for k, v in counter.calls.items()}
    if recorded is not None:
        del out
        recorded.destroy()
    flops = 284812800 * batch * seq  # matmul FLOPs per forward
    how = ("the windowed forward recorded once, each step one graph replay" if graph else
           "deferred-evaluation window: attention, layer norm, GELU and linear sequences as fused kernels" if window
           else "eager, one backend call per primitive")
    rec = {"op": f"cfg5 GPT-2 small forward, bf16, batch 8 x seq 1024 ({how})",
           "ms": round(ms, 3), "tokens/s": round(batch * seq / (ms * 1e-3), 1), "hip_event_ms": round(ev_ms, 3),
           "matmul_TFLOP/s": round(flops / (ms * 1e-3) / 1e12, 1), "backend_calls": sum(calls.values()),
           "calls_by_kind": calls}
    del params, ids, model, nx, front
    hip.trim()
    return rec


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--only-step", action="store_true", help="time the headline step only")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also launch 20 plain 64 MiB copies (scale for rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--only-config", type=int, choices=(1, 2, 3, 4), default=0,
                    help="time the operations of one configuration only and print their records")
    ap.add_argument("--only-next", action="store_true",
                    help="time the operations beside the hot path only (pad ... fft), the linear-algebra family included")
    ap.add_argument("--only-gpt2", action="store_true", help="run the GPT-2 forward leg only and print its record")
    ap.add_argument("--cpu-configs", action="store_true",
                    help="time the CPU oracle on bounded samples of configurations 1, 3, 4, 5 and print the records")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this backend has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    if args.cpu_configs:
        print(json.dumps({"cpu_configs": cpu_configs()}))
        return
    hip = Backend()
    info = hip.device_info()
    if args.only_gpt2:
        print(json.dumps(config5(hip)))
        print(json.dumps(config5(hip, window=True)))
        print(json.dumps(config5(hip, window=True, graph=True, iters=10)))
        return
    if args.only_next:
        print(json.dumps({"ops": next_ops(hip, Workloads(hip), linalg=True)}))
        return
    if args.only_config:
        # one configuration's operations, each timed alone (for profiling runs)
        W = Workloads(hip)
        group = {1: W.config1, 2: W.config2, 3: W.config3, 4: W.config4}[args.only_config]
        recs = [op_record(op, time_ops(hip, [op], 10 if "16,4096" in op.name else 50, 3)) for op in group()]
        print(json.dumps({"config": args.only_config, "ops": recs}))
        return
    W = Workloads(hip)
    step_ops = W.config2()
    step_bytes = sum(o.nbytes for o in step_ops)

    # headline: W warm-up steps, then exactly K timed steps, synchronised on both sides
    for _ in range(args.warmup):
        for op in step_ops:
            op()
    hip.synchronize()
    t0 = time.perf_counter()
    hip.timer_start()
    for _ in range(args.steps):
        for op in step_ops:
            op()
    ev_ms = hip.timer_stop()
    hip.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = wall_ms / args.steps
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    # the same step recorded once and replayed: what the launch gaps between the seven calls cost
    hip.capture_begin()
    try:
        for op in step_ops:
            op()
    finally:
        recorded = hip.capture_end()
    for _ in range(args.warmup):
        recorded.launch()
    hip.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        recorded.launch()
    hip.synchronize()
    replay_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    recorded.destroy()

    # parity of what was just timed, against the oracle on the same seeded inputs
    cpu, parity = None, None
    if not args.no_cpu:
        cpu, (ov, ow) = cpu_baseline()
        from oracle.nx_oracle import logical as ological

        parity = bool(np.array_equal(logical(W.cfg2_out["v"]).view(np.uint16), ological(ov).view(np.uint16))
                      and np.array_equal(logical(W.cfg2_out["w"]), ological(ow)))

    # dominant kernel alone (the LDS-turned add), for the roofline object
    dom = step_ops[0]
    dom_ms = time_ops(hip, [dom], 200, 10)
    dom_path = hip.last_path()
    roofline = {
        "kernel": f"{dom_path}_kernel<BinaryF<OpAdd, f32>, 64> ({dom.name})",
        "bound": "hbm", "achieved": round(dom.nbytes / (dom_ms * 1e-3) / 1e9, 1), "peak": PEAK_HBM_GBS,
        "unit": "GB/s", "frac": round(dom.nbytes / (dom_ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
        "bytes_per_launch": dom.nbytes, "avg_launch_ms": round(dom_ms, 5), "traffic": DOMINANT_KERNEL_HBM_TRAFFIC,
    }

    ops_out = []
    if args.pmc_calibration:
        # a plain contiguous copy of known size (64 MiB read, 64 MiB written) in the same process:
        # hardware-counter readings of the step's kernels are scaled by what the counters show here
        src, dst = hip.full(dt.float32, (64, 512, 512), 1.0), hip.buffer(dt.float32, (64, 512, 512))
        cal = W.mk("calibration copy 64 MiB", W.lib.nxh_copy, [dst, src], nbytes=2 * 64 * 512 * 512 * 4)
        for _ in range(20):
            cal()
        hip.synchronize()
    if not args.only_step:
        for op in step_ops:
            ops_out.append(op_record(op, time_ops(hip, [op], 100, 5)))
        for group in (W.config1, W.config3, W.config4):
            ops = group()
            for op in ops:
                iters = 10 if "16,4096" in op.name else 50
                ops_out.append(op_record(op, time_ops(hip, [op], iters, 3)))
            if group == W.config1:
                ms = time_ops(hip, ops, 50, 3)
                ops_out.append({"op": "cfg1 chain (4 ops, 576 MiB)", "ms": round(ms, 5),
                                "GB/s": round(603996160 / (ms * 1e-3) / 1e9, 1),
                                "frac_hbm": round(603996160 / (ms * 1e-3) / 1e9 / PEAK_HBM_GBS, 4), "bound": "hbm"})
            del ops
            W.keep.clear()
            hip.trim()
        ops_out.append(config5(hip))
        ops_out.append(config5(hip, window=True))
        ops_out.append(config5(hip, window=True, graph=True, iters=10))
        ops_out.extend(next_ops(hip, W))

    line = {
        "metric": METRIC, "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32+i32", "data": "synthetic",
        "config": {"workload": "config 2: broadcast/strided elementwise, [64,512,512] f32 (add permuted+broadcast, "
                               "mul scalar, cast f16) and int32 (add, mul, cmplt, where); 7 backend calls per step",
                   "algorithmic_bytes_per_step": step_bytes, "device": info["name"].strip(),
                   "compute_units": info["compute_units"], "hip_event_ms_per_step": round(ev_ms / args.steps, 5),
                   "frac_of_hbm_peak": round(value / PEAK_HBM_GBS, 4), "parity_vs_oracle": parity,
                   "graph_replay": {"ms_per_step": round(replay_ms, 5),
                                    "GB/s": round(step_bytes / (replay_ms * 1e-3) / 1e9, 1),
                                    "note": "the step recorded with nxh_capture_begin/_end and replayed with "
                                            "nxh_graph_launch; not the headline value"}},
        "roofline": roofline, "cpu_baseline": cpu, "ops": ops_out,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
