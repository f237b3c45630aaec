"""Recorded sequences (nxh_capture_begin / nxh_capture_end / nxh_graph_launch):
a replay must give what the same calls give eagerly, bit for bit, on every
replay, with other work of the same context between the replays, and after its
inputs were rewritten in place."""

import numpy as np
import pytest

from helpers import decode, encode, logical, same_bits
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu


class capture:
    """Closes the capture even when the recorded calls raise, so that a failing
    test leaves the shared context usable."""

    def __init__(self, backend):
        self.B, self.graph = backend, None

    def __enter__(self):
        self.B.capture_begin()
        return self

    def __exit__(self, *exc):
        self.graph = self.B.capture_end()
        return False


def chain(B, a, b, idx):
    """Map, strided view, reduction with a scratch buffer, scan, sort, GEMM and a
    gather: one launch of most kernel families, with temporaries that die."""
    c = B.binary("add", a, b)
    d = B.binary("mul", c, B.permute(c, (1, 0)))
    s = B.reduce("sum", [0], d)
    m = B.matmul(d, c)
    k = B.associative_scan(1, "max", m)
    o = B.sort(B.binary("sub", k, B.expand(B.reshape(s, (1, 192)), (192, 192))), 1, True)
    return B.gather(o, idx, 0)


def inputs(seed):
    rng = np.random.default_rng(seed)
    a = (rng.integers(-8, 8, (192, 192)) / 4).astype(np.float32)  # quarter-integers: sums are exact in any order
    b = (rng.integers(-8, 8, (192, 192)) / 4).astype(np.float32)
    idx = rng.integers(0, 192, (64, 192)).astype(np.int32)
    return a, b, idx


def test_replays_match_eager_results_between_other_work(hip, oracle):
    a0, b0, i0 = inputs(1)
    ta, tb = (hip.reshape(hip.from_host(x, dt.float32), x.shape) for x in (a0, b0))
    ti = hip.reshape(hip.from_host(i0, dt.int32), i0.shape)
    chain(hip, ta, tb, ti)  # warm every entry point once
    before = hip.memory_stats()["in_use"]
    with capture(hip) as cap:
        out = chain(hip, ta, tb, ti)
    g = cap.graph
    try:
        for seed in (1, 2, 3, 4):
            a, b, i = inputs(seed)
            # rewrite the inputs in place, then run unrelated eager work that allocates and frees
            for t, x, d in ((ta, a, dt.float32), (tb, b, dt.float32), (ti, i, dt.int32)):
                hip.assign(t, hip.reshape(hip.from_host(x, d), x.shape))
            junk = hip.binary("mul", hip.full(dt.float32, (257, 129), 3.0), hip.full(dt.float32, (257, 129), 2.0))
            assert float(logical(hip.reduce("max", [0, 1], junk))) == 6.0
            g.launch()
            eager = chain(hip, ta, tb, ti)
            oa, ob = (oracle.reshape(oracle.from_host(x, dt.float32), x.shape) for x in (a, b))
            want = chain(oracle, oa, ob, oracle.reshape(oracle.from_host(i, dt.int32), i.shape))
            same_bits(logical(out), logical(eager), f"replay {seed} against eager")
            same_bits(logical(out), logical(want), f"replay {seed} against the oracle")
    finally:
        g.destroy()
    del out, eager, junk
    assert hip.memory_stats()["in_use"] == before


def test_matmul_forms_with_temporaries_replay(hip, oracle):
    """The matmul forms that take a pooled block inside the call (the f32 cut along K with its
    partial sums, the padded copies of ragged operands) and the float64 kernel, recorded once:
    every replay gives the bits of the eager call on the inputs of the moment."""
    rng = np.random.default_rng(77)

    def make(seed):
        r = np.random.default_rng(seed)
        return (r.standard_normal((256, 2048)).astype(np.float32), r.standard_normal((2048, 256)).astype(np.float32),
                encode(r.standard_normal((1, 256, 576)), dt.bfloat16, oracle),
                encode(r.standard_normal((8, 576, 196)), dt.bfloat16, oracle),
                r.standard_normal((300, 100)), r.standard_normal((100, 200)))

    def dev(x, d):
        return hip.reshape(hip.from_host(x, d), x.shape)

    kinds = (dt.float32, dt.float32, dt.bfloat16, dt.bfloat16, dt.float64, dt.float64)
    ts = [dev(x, d) for x, d in zip(make(0), kinds)]

    def run():
        outs = [hip.matmul(ts[0], ts[1])]
        paths = [hip.last_path()]
        outs.append(hip.matmul(hip.expand(ts[2], (8, 256, 576)), ts[3]))
        paths.append(hip.last_path())
        outs.append(hip.matmul(ts[4], ts[5]))
        paths.append(hip.last_path())
        return outs, paths

    _, paths = run()  # warm
    assert paths == ["gemm_tile_64x64_splitk", "gemm_tile_padded", "gemm_f64_32x32"], paths
    with capture(hip) as cap:
        outs, _ = run()
    g = cap.graph
    try:
        for seed in (1, 2, 3):
            for t, x, d in zip(ts, make(seed), kinds):
                hip.assign(t, dev(x, d))
            junk = hip.matmul(dev(rng.standard_normal((128, 1024)).astype(np.float32), dt.float32),
                              dev(rng.standard_normal((1024, 64)).astype(np.float32), dt.float32))  # takes and frees a block
            g.launch()
            eager, _ = run()
            for o, e, name in zip(outs, eager, paths):
                same_bits(logical(o), logical(e), f"replay {seed}: {name}")
            del junk, eager
    finally:
        g.destroy()


def test_uploads_are_replayed_and_host_reads_are_refused(hip):
    x = hip.from_host(np.arange(1000, dtype=np.int32), dt.int32)
    with capture(hip) as cap:
        y = hip.from_host(np.full(1000, 5, np.int32), dt.int32)  # recorded with its own copy of the bytes
        z = hip.binary("add", x, y)
        with pytest.raises(RuntimeError, match="while a graph is being captured"):
            hip.to_host(z)
        with pytest.raises(RuntimeError, match="while a graph is being captured"):
            hip.synchronize()
        with pytest.raises(RuntimeError, match="256 KiB"):
            hip.from_host(np.zeros(1 << 20, np.uint8), dt.uint8)
    g = cap.graph
    try:
        for k in range(3):
            hip.assign(x, hip.from_host(np.arange(1000, dtype=np.int32) * k, dt.int32))
            hip.assign(y, hip.from_host(np.zeros(1000, np.int32), dt.int32))  # the replay uploads the fives again
            g.launch()
            same_bits(logical(z), np.arange(1000, dtype=np.int32) * k + 5, f"replay {k}")
    finally:
        g.destroy()
    with pytest.raises(RuntimeError, match="no capture in progress"):
        hip.capture_end()


def test_index_fault_of_a_replay_surfaces_at_synchronize(hip):
    data = hip.reshape(hip.from_host(np.arange(64, dtype=np.float32), dt.float32), (8, 8))
    idx = hip.reshape(hip.from_host(np.zeros(8, np.int32), dt.int32), (1, 8))
    hip.gather(data, idx, 0)
    with capture(hip) as cap:
        out = hip.gather(data, idx, 0)
    g = cap.graph
    try:
        g.launch()
        hip.synchronize()
        same_bits(logical(out), np.arange(8, dtype=np.float32).reshape(1, 8))
        hip.assign(idx, hip.reshape(hip.from_host(np.full(8, 8, np.int32), dt.int32), (1, 8)))
        g.launch()
        with pytest.raises(RuntimeError, match="index out of bounds"):
            hip.synchronize()
        hip.synchronize()  # reported once
        # an eager gather issued behind a faulting replay reports the replay's fault as the
        # replay's (before its own launch) and then answers for itself only
        g.launch()
        good = hip.reshape(hip.from_host(np.full(8, 3, np.int32), dt.int32), (1, 8))
        with pytest.raises(RuntimeError, match="replayed gather or scatter"):
            hip.gather(data, good, 0)
        same_bits(logical(hip.gather(data, good, 0)), np.arange(24, 32, dtype=np.float32).reshape(1, 8))
        hip.synchronize()
        hip.assign(idx, hip.reshape(hip.from_host(np.full(8, 7, np.int32), dt.int32), (1, 8)))
        g.launch()
        same_bits(logical(out), np.arange(56, 64, dtype=np.float32).reshape(1, 8))
    finally:
        g.destroy()


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16], ids=lambda d: d.name)
def test_captured_gpt2_forward_replays_the_windowed_forward(hip, oracle, d):
    """The whole windowed forward as one graph: new token ids are written into
    the captured input tensor and each replay equals the eager windowed result."""
    from raven_amd.kaun_gpt2 import Config, Gpt2, host_params, upload
    from raven_amd.nx_frontend import Nx
    from nx_window import Window

    cfg = Config(vocab_size=1031, n_positions=128, n_embd=256, n_layer=2, n_head=4, n_inner=1024)
    hp = host_params(cfg, seed=16, stddev=0.05)
    win = Window(hip)
    nx = Nx(win)
    params = upload(nx, hp, d, lambda a, dd: encode(a, dd, oracle))
    model = Gpt2(nx, cfg)
    ids = [np.random.default_rng(40 + k).integers(0, cfg.vocab_size, (2, 96)).astype(np.int32) for k in range(3)]
    t_ids = nx.create(dt.int32, ids[0].shape, ids[0])
    win.force(t_ids)  # the window uploads small index tensors on first use: the input must exist before the capture
    eager = [logical(win.force(model.logits(params, nx.create(dt.int32, i.shape, i)))) for i in ids]
    with capture(win) as cap:
        out = win.force(model.logits(params, t_ids))
    g = cap.graph
    try:
        for k in (0, 1, 2, 1):
            hip.assign(win.force(t_ids), hip.reshape(hip.from_host(ids[k], dt.int32), ids[k].shape))
            g.launch()
            same_bits(logical(out), eager[k], f"replay with ids {k}")
            # eager work of the same context between replays
            assert logical(win.force(model.logits(params, nx.create(dt.int32, ids[k].shape, ids[k])))).shape == eager[k].shape
    finally:
        g.destroy()
    assert np.all(np.isfinite(decode(eager[0], d, oracle)))


def test_a_transform_length_is_never_first_used_inside_a_capture(hip, oracle):
    """The twiddle / chirp tables of a transform are filled by kernels on the
    context's stream. Inside a capture such a fill would only be recorded, and the
    table would count as present while still empty: the first use of a length is
    refused there, and the same length then works eagerly and in a later capture."""
    rng = np.random.default_rng(77)
    for n in (1536, 2 * 3 * 5 * 7 * 11):  # lengths no other test uses: a power-of-two-free one takes the chirp tables too
        a = (rng.standard_normal((4, n)) + 1j * rng.standard_normal((4, n))).astype(np.complex64)
        x = hip.reshape(hip.from_host(a, dt.complex64), a.shape)
        ox = oracle.reshape(oracle.from_host(a, dt.complex64), a.shape)
        with pytest.raises(RuntimeError, match="run it once eagerly"):
            with capture(hip):
                hip.fft(x, [1])
        want = logical(oracle.fft(ox, [1]))
        eager = logical(hip.fft(x, [1]))
        assert np.all(np.abs(eager - want) <= 1e-4 * (1 + np.abs(want))), n
        with capture(hip) as c:
            out = hip.fft(x, [1])
        for _ in range(2):
            c.graph.launch()
            hip.synchronize()
            same_bits(logical(out), eager, f"replayed fft {n}")
        c.graph.destroy()
