"""Concurrent callers. The reference serialises its parallel regions and releases the runtime
lock around them (nx_c_engine.c:443-465), so operations may be issued from several OCaml domains
at once. Here every context has one stream and one lock: two host threads that issue map, reduce,
matmul, gather and sort calls (each with its allocations and frees) on ONE context, and on TWO
contexts of the one GPU, must get, call for call, the bits a single thread gets. ctypes releases
the interpreter lock for the duration of each library call, so the calls really overlap."""

import threading

import numpy as np
import pytest

from helpers import logical, same_bits
from raven_amd import dtype as dt
from raven_amd.nx_backend import Backend
from raven_amd.nx_frontend import Nx

pytestmark = pytest.mark.gpu

ROUNDS = 40


def workload(hip, seed, deferred=False):
    """A chain of calls of every family on inputs of its own; returns the host copy of each round's
    results. Every intermediate is dropped at once, so blocks go back to the allocator and are
    handed out again while the other thread is allocating."""
    rng = np.random.default_rng(seed)
    nx = Nx(hip)
    a = rng.standard_normal((96, 160)).astype(np.float32)
    b = rng.standard_normal((160, 64)).astype(np.float32)
    n = rng.integers(-1000, 1000, (96, 160)).astype(np.int32)
    idx = rng.integers(0, 96, (40, 160)).astype(np.int32)
    ta, tb, tn, ti = (hip.reshape(hip.from_host(x, d), x.shape) for x, d in
                      ((a, dt.float32), (b, dt.float32), (n, dt.int32), (idx, dt.int32)))
    out = []
    for r in range(ROUNDS):
        s = nx.add(nx.mul_s(ta, 1.0 + r), hip.permute(hip.permute(ta, (1, 0)), (1, 0)))   # map
        e = nx.exp(nx.mul_s(s, 0.01))
        row = hip.reduce("sum", [1], e)                                                   # fold
        col = hip.reduce("max", [0], tn)
        mm = nx.matmul(e, tb)                                                             # matmul
        g = hip.gather(s, ti, 0)                                                          # move
        srt = hip.sort(tn, 1, bool(r & 1))
        sm = nx.softmax(mm)                                                               # five primitives (fused when deferred)
        out.append([logical(t) for t in (row, col, mm, g, srt, sm)])
        del s, e, row, col, mm, g, srt, sm
    hip.synchronize()
    return out


def run_threads(contexts, seeds):
    results, errors = [None] * len(seeds), []

    def body(i):
        try:
            results[i] = workload(contexts[i], seeds[i])
        except BaseException as exc:  # noqa: BLE001 - reported by the main thread
            errors.append((i, repr(exc)))

    threads = [threading.Thread(target=body, args=(i,)) for i in range(len(seeds))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=110)
    assert not any(t.is_alive() for t in threads), "a caller did not return"
    assert not errors, errors
    return results


def compare(got, want, who):
    for r, (g_round, w_round) in enumerate(zip(got, want)):
        for name, g, w in zip(("sum", "max", "matmul", "gather", "sort", "softmax"), g_round, w_round):
            same_bits(g, w, f"{who}, round {r}, {name}")  # stops at the first mismatch


def test_two_threads_on_one_context(hip):
    serial = [workload(hip, 41), workload(hip, 42)]
    got = run_threads([hip, hip], [41, 42])
    compare(got[0], serial[0], "thread 0 on the shared context")
    compare(got[1], serial[1], "thread 1 on the shared context")
    before = hip.memory_stats()["in_use"]
    hip.synchronize()
    assert hip.memory_stats()["in_use"] == before


def test_two_threads_on_two_contexts(hip):
    other = Backend()
    serial = [workload(hip, 43), workload(hip, 44)]
    got = run_threads([hip, other], [43, 44])
    compare(got[0], serial[0], "thread 0 on its own context")
    compare(got[1], serial[1], "thread 1 on its own context")


def test_two_threads_record_into_two_contexts(hip):
    """The deferred mode keeps one record per context: two threads, each with its own context in
    that mode, fuse their own runs and see their own results."""
    other = Backend()
    serial = [workload(hip, 45), workload(hip, 46)]
    for c in (hip, other):
        c.set_deferred(True)
    try:
        before = [c.deferred_stats()["softmax_rows"] for c in (hip, other)]
        got = run_threads([hip, other], [45, 46])
        fused = [c.deferred_stats()["softmax_rows"] - b for c, b in zip((hip, other), before)]
    finally:
        for c in (hip, other):
            c.set_deferred(False)
    assert fused == [ROUNDS, ROUNDS]
    for i in range(2):
        for r in range(ROUNDS):
            for name, g, w in zip(("sum", "max", "matmul", "gather", "sort"), got[i][r], serial[i][r]):
                same_bits(g, w, f"context {i}, round {r}, {name}")
            # the fused row sum may add in another order than the five primitives
            assert np.allclose(got[i][r][5], serial[i][r][5], rtol=2e-6, atol=1e-9)
