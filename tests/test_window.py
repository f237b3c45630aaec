"""The deferred-evaluation window on the CPU: recorded primitives are executed in
issue order, the three sequences are recognised exactly when their
intermediates cannot be observed, and everything a caller can see is what the
eager backend gives.

The wrapped backend here is the CPU oracle with the three fused operations
defined as the primitive sequences themselves, so a window result must equal
the eager result bit for bit and the test isolates the recording, matching and
ordering logic (the fused GPU kernels have their own parity tests)."""

import numpy as np
import pytest

from helpers import encode, pair
from oracle.nx_oracle import OracleBackend
from oracle.nx_oracle import logical as ological
from raven_amd import dtype as dt
from raven_amd.kaun_gpt2 import Config, Gpt2, LayerNorm, host_params, upload
from raven_amd.nx_frontend import Nx
from nx_window import Window

TINY = Config(vocab_size=97, n_positions=16, n_embd=128, n_layer=2, n_head=4, n_inner=256)  # head dim 32


class SequencedOracle(OracleBackend):
    """The oracle plus the fused operations, each spelled as its sequence."""

    def __init__(self):
        self.calls = []


    def softmax_rows(self, x, scale=None, mask=None, masked_value=None, out_dtype=None):
        self.calls.append("softmax_rows")
        nx = Nx(self)
        t = x
        if scale is not None:
            t = nx.mul(t, self.full(x.dtype, (), scale))
        if mask is not None:
            t = nx.where(mask, t, self.full(x.dtype, (), masked_value))
        t = nx.softmax(t)
        return self.cast(t, out_dtype) if out_dtype is not None and out_dtype is not x.dtype else t

    def layer_norm_rows(self, x, gamma, beta, eps):
        self.calls.append("layer_norm_rows")
        return Gpt2(Nx(self), TINY).layer_norm(LayerNorm(gamma, beta), x, eps)

    def attention(self, q, k, v, scale=None, mask=None, masked_value=None, causal=False):
        self.calls.append("attention_causal" if causal else "attention")
        nx = Nx(self)
        r = len(q.shape)
        sc = nx.matmul(nx.cast(dt.float32, q), nx.swapaxes(r - 2, r - 1, nx.cast(dt.float32, k)))
        if scale is not None:
            sc = nx.mul(sc, self.full(dt.float32, (), scale))
        if causal:
            n = q.shape[-2]
            idx = nx.arange(dt.int32, 0, n, 1)
            mask = nx.less_equal(nx.reshape((1, n), idx), nx.reshape((n, 1), idx))
        if mask is not None:
            sc = nx.where(mask, sc, self.full(dt.float32, (), masked_value))
        return nx.matmul(nx.cast(q.dtype, nx.softmax(sc)), v)

    def linear(self, x, w, bias=None, residual=None):
        self.calls.append("linear")
        nx = Nx(self)
        y = nx.matmul(x, w)
        if bias is not None:
            y = nx.add(y, bias)
        return nx.add(residual, y) if residual is not None else y

    def gelu_tanh(self, x, constants):
        self.calls.append("gelu_tanh")
        nx = Nx(self)
        c = [self.full(x.dtype, (), constants[i:i + 1]) for i in range(4)]
        x3 = nx.mul(x, nx.mul(x, x))
        inner = nx.mul(nx.add(x, nx.mul(x3, c[0])), c[1])
        return nx.mul(nx.mul(x, nx.add(nx.tanh(inner), c[2])), c[3])


def value(win, t):
    return ological(win.force(t))


@pytest.fixture
def win():
    return Window(SequencedOracle())


class Counting:
    """Counts what the window asks of the backend (not what the backend's own
    sequences call internally)."""

    def __init__(self, inner):
        self._inner, self.asked = inner, {}

    def __getattr__(self, name):
        attr = getattr(self._inner, name)
        if not callable(attr):
            return attr

        def counted(*a, **k):
            self.asked[name] = self.asked.get(name, 0) + 1
            return attr(*a, **k)

        return counted


def forward(backend, hp, ids, d, oracle):
    nx = Nx(backend)
    params = upload(nx, hp, d, lambda a, dd: encode(a, dd, oracle))
    return Gpt2(nx, TINY).logits(params, nx.create(dt.int32, ids.shape, ids.astype(np.int32)))


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16], ids=lambda d: d.name)
def test_gpt2_forward_through_the_window_fuses_every_sequence(oracle, d):
    hp = host_params(TINY, seed=11, stddev=0.2)
    ids = np.random.default_rng(12).integers(0, TINY.vocab_size, (2, 8))
    want = ological(forward(oracle, hp, ids, d, oracle))
    base = SequencedOracle()
    asked = Counting(base)
    w = Window(asked)
    got = value(w, forward(w, hp, ids, d, oracle))
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))
    L = TINY.n_layer
    assert w.stats["layer_norm_rows"] == 2 * L + 1
    assert w.stats["gelu_tanh"] == L
    assert w.stats["fallbacks"] == 0
    if d is dt.bfloat16:
        # the whole attention core is one call, recognised as causal from the aranges of its mask
        assert (w.stats["attention"], w.stats["softmax_rows"]) == (L, 0)
        assert base.calls.count("attention_causal") == L
    else:
        # float32 has no float32 island: the softmax alone is fused
        assert (w.stats["attention"], w.stats["softmax_rows"]) == (0, L)
        assert base.calls.count("softmax_rows") == L
    # the six linears of a block take their bias add, and two of them the residual
    # add, into the GEMM; what is left op by op per block is, for float32, the mask
    # compare and the two attention matmuls (the causal attention kernel takes the
    # mask as a flag: neither its compare nor the two aranges it reads are ever
    # issued); outside the blocks the embedding add and the head matmul
    assert w.stats["linear"] == 6 * L and base.calls.count("linear") == 6 * L
    per_block = 0 if d is dt.bfloat16 else 3
    assert w.stats["issued"] == L * per_block + 2
    assert asked.asked.get("compare", 0) == (0 if d is dt.bfloat16 else L)
    n_params = 4 + 16 * L  # wte, wpe, ln_f (2) and 16 leaves per block
    # ids and positions, and for float32 the arange of each mask
    assert asked.asked["from_host"] - n_params == (2 if d is dt.bfloat16 else 2 + L)
    # with fusion switched off the window only defers
    w2 = Window(SequencedOracle(), fuse=False)
    got2 = value(w2, forward(w2, hp, ids, d, oracle))
    assert np.array_equal(got2.view(np.uint8), want.view(np.uint8))
    assert w2.stats["issued"] == w2.stats["recorded"] and w2.stats["softmax_rows"] == 0


def test_an_observable_intermediate_blocks_the_fusion(win, oracle):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((4, 16)).astype(np.float32)
    nx, onx = Nx(win), Nx(oracle)
    wx = nx.create(dt.float32, x.shape, x)
    ox = onx.create(dt.float32, x.shape, x)
    # same calls as Nx.softmax, but the exponentials stay referenced
    mx = nx.max(wx, [1], keepdims=True)
    e = nx.exp(nx.sub(wx, mx))
    del mx
    y = nx.div(e, nx.sum(e, [1], keepdims=True))
    want = ological(onx.softmax(ox))
    assert np.array_equal(value(win, y), want)
    assert win.stats["softmax_rows"] == 0 and win.stats["issued"] == 5
    oe = onx.exp(onx.sub(ox, onx.max(ox, [1], keepdims=True)))
    assert np.array_equal(value(win, e), ological(oe))
    # once the handle is gone the same calls fuse
    del e, y
    y = nx.softmax(wx)
    assert np.array_equal(value(win, y), want)
    assert win.stats["softmax_rows"] == 1


def test_a_reader_outside_the_run_blocks_the_fusion(win, oracle):
    x = np.random.default_rng(2).standard_normal((3, 8)).astype(np.float32)
    nx = Nx(win)
    wx = nx.create(dt.float32, x.shape, x)
    mx = nx.max(wx, [1], keepdims=True)
    shifted = nx.sub(wx, mx)
    extra = nx.add(shifted, shifted)       # reads an interior value
    e = nx.exp(shifted)
    del shifted, mx
    y = nx.div(e, nx.sum(e, [1], keepdims=True))
    del e
    onx = Nx(oracle)
    ox = onx.create(dt.float32, x.shape, x)
    assert np.array_equal(value(win, y), ological(onx.softmax(ox)))
    sh = onx.sub(ox, onx.max(ox, [1], keepdims=True))
    assert np.array_equal(value(win, extra), ological(onx.add(sh, sh)))
    assert win.stats["softmax_rows"] == 0


def test_scale_mask_and_cast_join_the_softmax(win, oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 3, 8, 8)).astype(np.float32)
    tri = np.tril(np.ones((8, 8), np.uint8))

    def weights(B):
        nx = Nx(B)
        t = nx.create(dt.float32, x.shape, x)
        m = B.expand(B.reshape(B.from_host(tri, dt.bool_), (1, 1, 8, 8)), x.shape)
        s = nx.mul_s(t, 0.125)
        s = nx.where(m, s, nx.scalar_like(s, float("-inf")))
        return nx.cast(dt.bfloat16, nx.softmax(s))

    got = value(win, weights(win))
    assert np.array_equal(got, ological(weights(oracle)))
    assert win.stats["softmax_rows"] == 1 and win.stats["issued"] == 0
    assert win.B.calls == ["softmax_rows"]


def test_attention_run_and_what_blocks_it(oracle):
    rng = np.random.default_rng(8)
    b, h, s, hd = 2, 3, 16, 32
    d = dt.bfloat16
    q, k, v = (encode(rng.standard_normal((b, h, s, hd)), d, oracle) for _ in range(3))
    rnd = (rng.random((s, s)) < 0.6).astype(np.uint8)
    rnd[:, 0] = 1

    def run(B, mask_kind, keep=None):
        nx = Nx(B)
        tq, tk, tv = (nx.create(d, a.shape, a) for a in (q, k, v))
        if mask_kind == "causal":
            idx = nx.arange(dt.int32, 0, s, 1)
            mask = nx.less_equal(nx.reshape((1, s), idx), nx.reshape((s, 1), idx))
        elif mask_kind == "random":
            mask = nx.create(dt.bool_, (s, s), rnd)
        else:
            mask = None
        model = Gpt2(nx, TINY)
        if keep is None:
            return model.scaled_dot_product_attention(tq, tk, tv, mask)
        # the same calls with the probabilities kept alive
        sc = nx.mul_s(nx.matmul(nx.cast(dt.float32, tq), nx.swapaxes(2, 3, nx.cast(dt.float32, tk))), 0.25)
        sc = nx.where(mask, sc, nx.scalar_like(sc, float("-inf")))
        keep.append(nx.cast(d, nx.softmax(sc)))
        return nx.matmul(keep[-1], tv)

    for kind, expect in (("causal", "attention_causal"), ("random", "attention"), (None, "attention")):
        base = SequencedOracle()
        w = Window(base)
        got = value(w, run(w, kind))
        assert np.array_equal(got, ological(run(oracle, kind))), kind
        assert base.calls == [expect] and w.stats["attention"] == 1, (kind, base.calls)
    # a finite fill gives the hidden keys a weight: the run still fuses, but with the mask
    # tensor, never with the flag that lets the kernel skip the keys above the diagonal
    def finite(B):
        nx = Nx(B)
        tq, tk, tv = (nx.create(d, a.shape, a) for a in (q, k, v))
        idx = nx.arange(dt.int32, 0, s, 1)
        mask = nx.less_equal(nx.reshape((1, s), idx), nx.reshape((s, 1), idx))
        sc = nx.mul_s(nx.matmul(nx.cast(dt.float32, tq), nx.swapaxes(2, 3, nx.cast(dt.float32, tk))), 0.25)
        sc = nx.where(mask, sc, nx.scalar_like(sc, -1.5))
        return nx.matmul(nx.cast(d, nx.softmax(sc)), tv)

    base = SequencedOracle()
    w = Window(base)
    got = value(w, finite(w))
    assert np.array_equal(got, ological(finite(oracle)))
    assert base.calls == ["attention"] and w.stats["attention"] == 1, base.calls
    base = SequencedOracle()
    w = Window(base)
    kept = []
    got = value(w, run(w, "causal", kept))
    okept = []
    want = ological(run(oracle, "causal", okept))
    assert np.array_equal(got, want) and np.array_equal(value(w, kept[0]), ological(okept[0]))
    assert w.stats["attention"] == 0 and base.calls == ["softmax_rows"]   # the softmax alone still fuses


def test_gelu_and_layer_norm_alone(win, oracle):
    rng = np.random.default_rng(4)
    for d in (dt.float32, dt.bfloat16):
        x = encode(rng.standard_normal((5, 24)), d, oracle)
        g = encode(rng.standard_normal(24) + 1, d, oracle)
        b = encode(rng.standard_normal(24), d, oracle)
        before = dict(win.stats)
        res = []
        for B in (win, oracle):
            nx = Nx(B)
            model = Gpt2(nx, TINY)
            tx, tg, tb = (nx.create(d, a.shape, a) for a in (x, g, b))
            res.append((model.gelu_approx(tx), model.layer_norm(LayerNorm(tg, tb), tx, 1e-5)))
        assert np.array_equal(value(win, res[0][0]), ological(res[1][0]))
        assert np.array_equal(value(win, res[0][1]), ological(res[1][1]))
        assert win.stats["gelu_tanh"] == before["gelu_tanh"] + 1
        assert win.stats["layer_norm_rows"] == before["layer_norm_rows"] + 1
        assert win.stats["issued"] == before["issued"]


def test_a_write_through_assign_is_ordered_behind_the_record(win, oracle):
    a = np.arange(6, dtype=np.float32)
    nx = Nx(win)
    ta = nx.create(dt.float32, (6,), a)
    tb = nx.create(dt.float32, (6,), np.ones(6, np.float32))
    s = nx.add(ta, tb)                       # recorded, reads ta
    win.assign(ta, nx.create(dt.float32, (6,), np.zeros(6, np.float32)))  # overwrites ta afterwards
    assert np.array_equal(value(win, s), a + 1)
    assert np.array_equal(value(win, ta), np.zeros(6, np.float32))


def test_errors_and_limits(oracle):
    win = Window(SequencedOracle(), limit=4)
    nx = Nx(win)
    x = nx.create(dt.float32, (2, 3), np.ones((2, 3), np.float32))
    with pytest.raises(ValueError, match="shape mismatch"):
        win.binary("add", x, nx.create(dt.float32, (3, 2), np.ones((3, 2), np.float32)))
    with pytest.raises(ValueError, match="empty axis"):
        win.reduce("max", [1], nx.create(dt.float32, (2, 0), np.ones((2, 0), np.float32)))
    t = x
    for _ in range(9):                       # the record is executed every 4 entries
        t = nx.add(t, x)
    assert win.stats["flushes"] == 2 and len(win.entries) == 1
    assert np.array_equal(value(win, t), np.full((2, 3), 10, np.float32))
    # views of a pending result share it
    u = nx.add(t, t)
    v = win.permute(u, (1, 0))
    assert np.array_equal(value(win, v), np.full((3, 2), 20, np.float32))
    assert np.array_equal(value(win, u), np.full((2, 3), 20, np.float32))
    # rows too long for the fused kernels are declined by the matcher itself
    wide = nx.create(dt.float32, (1, 9000), np.zeros((1, 9000), np.float32))
    y = nx.softmax(wide)
    assert np.allclose(value(win, y), 1 / 9000)
    assert win.stats["softmax_rows"] == 0


def test_linear_runs(oracle):
    rng = np.random.default_rng(21)
    x = rng.standard_normal((2, 6, 16)).astype(np.float32)
    wt = rng.standard_normal((16, 8)).astype(np.float32)
    b = rng.standard_normal(8).astype(np.float32)
    r = rng.standard_normal((2, 6, 8)).astype(np.float32)

    def run(B, form, keep=None):
        nx = Nx(B)
        tx, tw, tb, tr = (nx.create(dt.float32, a.shape, a) for a in (x, wt, b, r))
        y = nx.matmul(tx, tw)
        if form in ("bias", "both", "both-flipped"):
            y = nx.add(y, tb)
        if keep is not None:
            keep.append(y)
        if form == "both":
            y = nx.add(tr, y)
        elif form in ("both-flipped", "residual"):
            y = nx.add(y, tr)
        return y

    for form, calls in (("bias", 1), ("both", 1), ("both-flipped", 1), ("residual", 1), ("plain", 0)):
        base = SequencedOracle()
        w = Window(base)
        got = value(w, run(w, form))
        assert np.array_equal(got, ological(run(oracle, form))), form
        assert base.calls.count("linear") == calls and w.stats["linear"] == calls, (form, base.calls)
    # the biased product kept alive: only the bias add joins the GEMM, the residual add is issued
    base = SequencedOracle()
    w = Window(base)
    kept, okept = [], []
    got = value(w, run(w, "both", kept))
    want = ological(run(oracle, "both", okept))
    assert np.array_equal(got, want) and np.array_equal(value(w, kept[0]), ological(okept[0]))
    assert w.stats["linear"] == 1 and w.stats["issued"] == 1
