"""The deferred-evaluation window below the C ABI (nxh_set_deferred): the frontend
issues its primitives one by one through the plain backend, the library records
them and replaces the runs that spell softmax (frontend.ml:4242-4252), layer
norm (kaun/lib/layer_norm.ml:43-68), GELU (fn.ml:31-38), the attention core
(attention.ml:67-110) and linear + residual (linear.ml:50-52, gpt2.ml:165-176)
by the fused entry points.

What is checked: the fused call really ran (the library's counters), its result
is bit for bit what the fused entry point gives when called directly, it agrees
with the eager op-by-op result as closely as the fused tests promise, an
intermediate that is still alive is written exactly as the eager path writes it,
and nothing the record touches is handed out again before the record has run."""

import math

import numpy as np
import pytest

from helpers import TOL, close, decode, encode, logical, pair, same_bits
from raven_amd import dtype as dt
from raven_amd.kaun_gpt2 import Config, Gpt2, LayerNorm, Linear, host_params, upload
from raven_amd.nx_frontend import Nx

pytestmark = pytest.mark.gpu


class deferred:
    """The mode is switched off again even when the body raises (the context is shared)."""

    def __init__(self, hip):
        self.hip = hip

    def __enter__(self):
        self.hip.set_deferred(True)
        self.before = self.hip.deferred_stats()
        return self

    def delta(self):
        now = self.hip.deferred_stats()
        return {k: now[k] - self.before[k] for k in now}

    def __exit__(self, *exc):
        try:
            self.hip.set_deferred(False)
        except Exception:
            if exc[0] is None:
                raise
        return False


def tensor(hip, a, d):
    return hip.reshape(hip.from_host(np.ascontiguousarray(a), d), a.shape)


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_softmax_layer_norm_and_gelu_runs_fuse(hip, oracle, d):
    rng = np.random.default_rng(300 + d.tag)
    nx = Nx(hip)
    model = Gpt2(nx, Config())
    x = tensor(hip, encode(rng.standard_normal((6, 40, 96)) * 2, d, oracle), d)
    gamma = tensor(hip, encode(1 + 0.1 * rng.standard_normal(96), d, oracle), d)
    beta = tensor(hip, encode(0.1 * rng.standard_normal(96), d, oracle), d)
    eager = [logical(nx.softmax(x)), logical(model.layer_norm(LayerNorm(gamma, beta), x, 1e-5)), logical(model.gelu_approx(x))]
    direct = [logical(hip.softmax_rows(x)), logical(hip.layer_norm_rows(x, gamma, beta, 1e-5)), logical(hip.gelu_tanh(x))]
    with deferred(hip) as win:
        got = [nx.softmax(x), model.layer_norm(LayerNorm(gamma, beta), x, 1e-5), model.gelu_approx(x)]
        got = [logical(t) for t in got]
        s = win.delta()
    assert (s["softmax_rows"], s["layer_norm_rows"], s["gelu_tanh"], s["fallbacks"]) == (1, 1, 1, 0), s
    assert s["issued"] == 0 and s["recorded"] >= 5 + 14 + 9
    for g, dr, e, name in zip(got, direct, eager, ("softmax", "layer_norm", "gelu")):
        same_bits(g, dr, f"{name}: the recorded run against the fused entry point")
        close(g, e, d, oracle, 4 * TOL[d.name][0] if d is not dt.float32 else 2e-6, 2e-6, f"{name}: against the eager sequence")
    same_bits(got[2], eager[2], "gelu has no sum: equal to the eager sequence bit for bit")


class Holding:
    """A backend whose results all stay referenced, like handles that wait for a garbage
    collector: nothing the frontend drops is given back to the library before `release`."""

    def __init__(self, hip):
        self._hip, self.kept = hip, []

    def __getattr__(self, name):
        attr = getattr(self._hip, name)
        if not callable(attr):
            return attr

        def call(*a, **k):
            r = attr(*a, **k)
            self.kept.append(r)
            return r

        return call

    def release(self):
        self.kept.clear()


def test_an_intermediate_that_is_still_held_is_written_when_it_is_read(hip, oracle):
    rng = np.random.default_rng(31)
    nx = Nx(hip)
    x = tensor(hip, rng.standard_normal((33, 70)).astype(np.float32), dt.float32)
    want_e = logical(nx.exp(nx.sub(x, nx.max(x, [-1], keepdims=True))))
    want = logical(hip.softmax_rows(x))
    with deferred(hip) as win:
        # the same five primitives, with the exponentials kept by the caller
        mx = nx.max(x, [-1], keepdims=True)
        e = nx.exp(nx.sub(x, mx))
        out = nx.div(e, nx.sum(e, [-1], keepdims=True))
        del mx
        got = logical(out)
        s = win.delta()
        # fused all the same; the four entries in front of the division wait for a reader or a free
        assert (s["softmax_rows"], s["issued"], s["postponed"], s["materialised"]) == (1, 0, 4, 0), s
        got_e = logical(e)
        s = win.delta()
        assert (s["issued"], s["materialised"]) == (4, 4), s
    same_bits(got, want, "softmax with a held intermediate")
    same_bits(got_e, want_e, "the held intermediate, written when it was read")


@pytest.mark.parametrize("reader", ["recorded", "entry_point", "mode_off"])
def test_postponed_entries_run_before_whatever_reads_them(hip, oracle, reader):
    rng = np.random.default_rng(35)
    nx = Nx(hip)
    x = tensor(hip, rng.standard_normal((20, 64)).astype(np.float32), dt.float32)
    e_want = logical(nx.exp(nx.sub(x, nx.max(x, [-1], keepdims=True))))
    with deferred(hip) as win:
        e = nx.exp(nx.sub(x, nx.max(x, [-1], keepdims=True)))
        out = nx.div(e, nx.sum(e, [-1], keepdims=True))
        hip.synchronize()  # executes the record; touches no tensor
        assert win.delta()["postponed"] == 4 and win.delta()["materialised"] == 0
        if reader == "recorded":
            got = logical(nx.add(e, e)) / 2
        elif reader == "entry_point":
            got = logical(hip.copy(e))
        else:
            hip.set_deferred(False)
            got = logical(e)
        assert win.delta()["materialised"] == 4
    same_bits(got, e_want, f"a postponed result read by {reader}")
    del out


def test_a_call_that_runs_at_once_reads_what_its_own_flush_postponed(hip, oracle):
    """A recordable primitive whose result cannot be recorded (a matmul result with padded rows
    is no plain block) executes the record and runs at once. Its operand here is the interior of a
    fused run, which that very flush postpones because the caller still holds it: it has to be
    written before the call reads it."""
    rng = np.random.default_rng(37)
    nx = Nx(hip)
    x = tensor(hip, rng.standard_normal((20, 64)).astype(np.float32), dt.float32)
    w = tensor(hip, rng.standard_normal((64, 4099)).astype(np.float32), dt.float32)
    want = logical(hip.matmul(nx.exp(nx.sub(x, nx.max(x, [-1], keepdims=True))), w))
    with deferred(hip) as win:
        e = nx.exp(nx.sub(x, nx.max(x, [-1], keepdims=True)))
        p = nx.div(e, nx.sum(e, [-1], keepdims=True))
        out = hip.matmul(e, w)
        assert tuple(out.strides) == (4128, 1)  # 4099 float32 per row, in whole 128-byte lines
        s = win.delta()
        assert (s["softmax_rows"], s["materialised"]) == (1, 4), s
        got = logical(out)
    same_bits(got, want, "matmul over the interior of a run that its own flush postponed")
    del p


def test_postponed_entries_run_before_their_operand_is_overwritten(hip, oracle):
    rng = np.random.default_rng(36)
    nx = Nx(hip)
    a = rng.standard_normal((20, 64)).astype(np.float32)
    x = tensor(hip, a, dt.float32)
    other = tensor(hip, a + 5.0, dt.float32)
    e_want = np.exp(a - a.max(-1, keepdims=True))
    with deferred(hip) as win:
        e = nx.exp(nx.sub(x, nx.max(x, [-1], keepdims=True)))
        out = nx.div(e, nx.sum(e, [-1], keepdims=True))
        got = logical(out)
        assert win.delta()["postponed"] == 4
        hip.assign(x, other)          # the run's operand changes under it: it is written first
        assert win.delta()["materialised"] == 4
        got_e = logical(e)
    assert np.allclose(got_e, e_want, rtol=2e-6, atol=0)
    assert np.allclose(got.sum(-1), 1.0, atol=1e-5)


def test_handles_that_die_late_fuse_like_handles_that_die_at_once(hip, oracle):
    """Every result stays referenced until after the read (a collector that has not run yet):
    the same fused kernels, nothing issued as recorded, and once the handles go nothing is left."""
    rng = np.random.default_rng(37)
    d = dt.bfloat16
    held = Holding(hip)
    nx, model = Nx(held), Gpt2(Nx(held), Config())
    x = tensor(hip, encode(rng.standard_normal((6, 40, 96)) * 2, d, oracle), d)
    gamma = tensor(hip, encode(1 + 0.1 * rng.standard_normal(96), d, oracle), d)
    beta = tensor(hip, encode(0.1 * rng.standard_normal(96), d, oracle), d)
    direct = [logical(hip.softmax_rows(x)), logical(hip.layer_norm_rows(x, gamma, beta, 1e-5)), logical(hip.gelu_tanh(x))]
    hip.synchronize()
    before = hip.memory_stats()["in_use"]
    with deferred(hip) as win:
        got = [nx.softmax(x), model.layer_norm(LayerNorm(gamma, beta), x, 1e-5), model.gelu_approx(x)]
        got = [logical(t) for t in got]
        s = win.delta()
        assert (s["softmax_rows"], s["layer_norm_rows"], s["gelu_tanh"], s["fallbacks"]) == (1, 1, 1, 0), s
        assert s["issued"] == 0 and s["postponed"] >= 4 + 15 + 8, s
        held.release()
        hip.synchronize()
        s = win.delta()
        assert s["materialised"] == 0 and s["issued"] == 0, s
    for g, dr, name in zip(got, direct, ("softmax", "layer_norm", "gelu")):
        same_bits(g, dr, f"{name}: fused with every handle still held")
    del got
    assert hip.memory_stats()["in_use"] == before


def test_blocks_of_recorded_entries_are_not_handed_out_again(hip):
    """An output is freed while its entry is recorded and a new, equally large output is
    allocated right behind it: the free is held back, so the two never share a block."""
    nx = Nx(hip)
    a = hip.full(dt.float32, (256, 256), 3.0)
    b = hip.full(dt.float32, (256, 256), 4.0)
    with deferred(hip):
        t = nx.add(a, b)          # recorded: 7
        u = nx.mul(t, t)          # recorded: 49, reads t
        del t                     # t's block may not be reused before the record has run
        v = nx.sub(nx.add(a, a), b)  # fresh outputs of the same size: 2
        w = nx.add(u, v)          # 51
        got = logical(w)
    assert np.all(got == 51.0)
    stats = hip.memory_stats()
    hip.synchronize()
    assert hip.memory_stats()["in_use"] <= stats["in_use"]


def test_linear_with_bias_and_residual_fuses(hip, oracle):
    rng = np.random.default_rng(32)
    d = dt.bfloat16
    nx = Nx(hip)
    model = Gpt2(nx, Config())
    x = tensor(hip, encode(rng.standard_normal((4, 128, 256)), d, oracle), d)
    w = tensor(hip, encode(rng.standard_normal((256, 512)) * 0.05, d, oracle), d)
    b = tensor(hip, encode(rng.standard_normal(512), d, oracle), d)
    r = tensor(hip, encode(rng.standard_normal((4, 128, 512)), d, oracle), d)
    eager = logical(nx.add(r, model.linear(Linear(w, b), x)))
    with deferred(hip) as win:
        got = logical(nx.add(r, model.linear(Linear(w, b), x)))
        s = win.delta()
    assert (s["linear"], s["issued"], s["fallbacks"]) == (1, 0, 0), s
    same_bits(got, eager, "linear + bias + residual: the epilogue rounds where the three calls round")


@pytest.mark.parametrize("kind", ["causal", "mask", "none"])
def test_attention_core_fuses(hip, oracle, kind):
    rng = np.random.default_rng(33)
    d = dt.bfloat16
    b, h, s, hd = 2, 3, 96, 64
    nx = Nx(hip)
    model = Gpt2(nx, Config())
    q, k, v = (tensor(hip, encode(rng.standard_normal((b, h, s, hd)), d, oracle), d) for _ in range(3))

    def mask_of():
        if kind == "causal":
            idx = nx.arange(dt.int32, 0, s, 1)
            return nx.less_equal(nx.reshape((1, s), idx), nx.reshape((s, 1), idx))
        if kind == "mask":
            m = (np.random.default_rng(34).random((s, s)) < 0.7).astype(np.uint8)
            m[:, 0] = 1
            return tensor(hip, m, dt.bool_)
        return None

    eager = logical(model.scaled_dot_product_attention(q, k, v, mask_of()))
    with deferred(hip) as win:
        got = logical(model.scaled_dot_product_attention(q, k, v, mask_of()))
        st = win.delta()
    assert (st["attention"], st["fallbacks"], st["softmax_rows"]) == (1, 0, 0), st
    # the causal mask is recognised from its aranges and never computed; a given mask is only read
    assert st["issued"] == 0, st
    direct = logical(hip.attention(q, k, v, 1.0 / math.sqrt(hd),
                                   mask=None if kind != "mask" else hip.expand(hip.reshape(mask_of(), (1, 1, s, s)), (b, h, s, s)),
                                   masked_value=None if kind == "none" else float("-inf"), causal=kind == "causal"))
    same_bits(got, direct, "the recorded run against nxh_attention")
    # the one-pass kernel rounds the exponentials, the sequence the quotients: a few units of bfloat16 apart
    close(got, eager, d, oracle, 2 * 2.0 ** -7, 8e-3, "against the eager sequence")


def test_errors_of_recorded_primitives_surface_when_the_record_runs(hip):
    a = hip.full(dt.float32, (4, 5), 1.0)
    bad = hip.full(dt.float32, (4, 6), 1.0)
    with deferred(hip):
        out = hip.buffer(dt.float32, (4, 5))
        import ctypes as C

        o, x, y = out._desc(), a._desc(), bad._desc()
        rc = hip._lib.nxh_binary(hip._h, 0, C.byref(o), C.byref(x), C.byref(y))
        assert rc == 0  # recorded, not checked yet
        with pytest.raises(ValueError, match="shape mismatch"):
            hip.synchronize()
        hip.synchronize()  # the record is gone
        ok = Nx(hip).add(a, a)
        assert np.all(logical(ok) == 2.0)


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16], ids=lambda d: d.name)
def test_gpt2_forward_with_the_library_window(hip, oracle, d):
    """The frontend's calls straight through the plain backend, recorded and fused below the ABI:
    every sequence is found, and the logits are bit for bit those of the Python window (which
    issues the same fused calls on the same operands)."""
    from nx_window import Window

    cfg = Config(vocab_size=1031, n_positions=128, n_embd=256, n_layer=2, n_head=4, n_inner=1024)
    hp = host_params(cfg, seed=16, stddev=0.05)
    ids = np.random.default_rng(17).integers(0, cfg.vocab_size, (2, 96)).astype(np.int32)
    enc = lambda a, dd: encode(a, dd, oracle)  # noqa: E731

    def run(front):
        nx = Nx(front)
        params = upload(nx, hp, d, enc)
        t_ids = nx.create(dt.int32, ids.shape, ids)
        return Gpt2(nx, cfg).logits(params, t_ids)

    eager = decode(logical(run(hip)), d, oracle)
    win = Window(hip)
    py = logical(win.force(run(win)))
    with deferred(hip) as lib:
        got = logical(run(hip))
        s = lib.delta()
    L = cfg.n_layer
    # 16-bit dtypes: the MLP's first linear layer and its GELU are one GEMM with the GELU in its epilogue
    mlp = L if d is dt.bfloat16 else 0
    assert (s["layer_norm_rows"], s["gelu_tanh"], s["linear"], s["linear_gelu"], s["fallbacks"]) == (2 * L + 1, L - mlp, 6 * L - mlp, mlp, 0), s
    assert (s["attention"], s["softmax_rows"]) == ((L, 0) if d is dt.bfloat16 else (0, L)), s
    assert s["grouped"] == 3 * L, s  # the q, k and v projections of a layer share one launch
    # (the causal mask is still a local of the attention layer when its head merge executes the
    # record: it waits, with its run, and is dropped unwritten when the layer returns)
    assert s["materialised"] == 0
    same_bits(got, py, "library window against the Python window")
    # the same forward with every handle alive until the logits have been read
    held = Holding(hip)
    with deferred(hip) as lib:
        late = logical(run(held))
        s2 = lib.delta()
        held.release()
        hip.synchronize()
        s3 = lib.delta()
    for k in ("layer_norm_rows", "gelu_tanh", "linear", "linear_gelu", "attention", "softmax_rows", "fallbacks", "issued"):
        assert s2[k] == s[k], (k, s2, s)
    assert s2["postponed"] > 0 and s3["materialised"] == 0, (s2, s3)
    same_bits(late, got, "handles that die late against handles that die at once")
    gv = decode(got, d, oracle)
    if d is dt.float32:
        assert np.max(np.abs(gv - eager)) <= 2e-5 * max(1.0, np.max(np.abs(eager)))
    else:
        assert np.all(np.abs(gv - eager) <= 6e-2 + 6e-2 * np.abs(eager))


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float16], ids=lambda d: d.name)
@pytest.mark.parametrize("rows,inputs,outputs", [(256, 128, 384), (200, 128, 384)], ids=["whole_tiles", "ragged_rows"])
def test_linear_then_gelu_is_one_gemm(hip, oracle, d, rows, inputs, outputs):
    """gelu_approx (linear x): with whole 128 x 128 tiles the GELU runs in the GEMM's epilogue,
    otherwise as the fused linear followed by the fused GELU; either way the bits of the eleven
    primitives."""
    rng = np.random.default_rng(38)
    nx = Nx(hip)
    model = Gpt2(nx, Config())
    x = tensor(hip, encode(rng.standard_normal((2, rows, inputs)), d, oracle), d)
    w = tensor(hip, encode(rng.standard_normal((inputs, outputs)) * 0.2, d, oracle), d)
    b = tensor(hip, encode(rng.standard_normal(outputs), d, oracle), d)
    eager = logical(model.gelu_approx(model.linear(Linear(w, b), x)))
    with deferred(hip) as win:
        got = logical(model.gelu_approx(model.linear(Linear(w, b), x)))
        s = win.delta()
    assert (s["linear_gelu"], s["linear"], s["gelu_tanh"], s["issued"], s["fallbacks"]) == (1, 0, 0, 0, 0), s
    same_bits(got, eager, "linear + gelu in one run against the primitives")
    if rows % 128 == 0:
        assert hip.last_path() == "linear_dl_128x192"  # 384 outputs: two 192-column blocks
        direct = logical(hip.linear_gelu_tanh(x, w, b))
        same_bits(got, direct, "against nxh_linear_gelu_tanh called by name")
    else:
        with pytest.raises(RuntimeError):
            hip.linear_gelu_tanh(x, w, b)


@pytest.mark.parametrize("rows,width,path", [(192, 256, "linear_tile_128x64"), (1408, 256, "linear_tile_128x128"),
                                             (1024, 384, "linear_dl_128x192")],
                         ids=["half_blocks", "staged_tiles", "direct_to_lds"])
def test_linear_layers_over_one_input_share_a_launch(hip, oracle, rows, width, path):
    """q, k and v of an attention layer: three linear layers over the same x. Recorded one after the
    other, launched as one GEMM over the three weight matrices, each result the bits of its own call."""
    rng = np.random.default_rng(39)
    d = dt.bfloat16
    nx = Nx(hip)
    model = Gpt2(nx, Config())
    x = tensor(hip, encode(rng.standard_normal((2, rows, 256)), d, oracle), d)
    ws = [tensor(hip, encode(rng.standard_normal((256, width)) * 0.1, d, oracle), d) for _ in range(3)]
    bs = [tensor(hip, encode(rng.standard_normal(width), d, oracle), d) for _ in range(3)]
    other_w = tensor(hip, encode(rng.standard_normal((256, 128)) * 0.1, d, oracle), d)
    other_b = tensor(hip, encode(rng.standard_normal(128), d, oracle), d)
    eager = [logical(model.linear(Linear(w, b), x)) for w, b in zip(ws, bs)] + [logical(model.linear(Linear(other_w, other_b), x))]
    with deferred(hip) as win:
        outs = [model.linear(Linear(w, b), x) for w, b in zip(ws, bs)]
        outs.append(model.linear(Linear(other_w, other_b), x))  # another shape: on its own
        got = [logical(t) for t in outs]
        s = win.delta()
    assert (s["linear"], s["grouped"], s["issued"], s["fallbacks"]) == (4, 3, 0, 0), s
    for i, (g, e) in enumerate(zip(got, eager)):
        same_bits(g, e, f"member {i} of the grouped launch against its own call")
    with deferred(hip) as win:  # the members alone: which kernel the grouped launch took
        outs = [model.linear(Linear(w, b), x) for w, b in zip(ws, bs)]
        same_bits(logical(outs[2]), eager[2], "last member")
        assert hip.last_path() == path, hip.last_path()
        assert win.delta()["grouped"] == 3
    # a member whose result is read before the last member was recorded stays out of the group
    with deferred(hip) as win:
        a = model.linear(Linear(ws[0], bs[0]), x)
        a2 = nx.add(a, a)
        b = model.linear(Linear(ws[1], bs[1]), x)
        got = [logical(t) for t in (a, a2, b)]
        s = win.delta()
    assert s["grouped"] == 0 and s["linear"] == 2, s
    same_bits(got[0], eager[0], "ungrouped member")
    same_bits(got[2], eager[1], "ungrouped member")


def test_small_uploads_wait_in_the_record(hip, oracle):
    """A host upload of up to 64 KiB is recorded with its bytes. It is sent when something needs
    it (a recorded reader, an entry point that reads the block, a host read) and in issue order with
    the other writes of its block; the host array may change right after the call."""
    nx = Nx(hip)
    a = np.arange(24, dtype=np.float32).reshape(4, 6)
    with deferred(hip) as win:
        t = hip.reshape(hip.from_host(a.reshape(-1), dt.float32), a.shape)
        src = a.copy()
        a[:] = -1.0  # the caller's buffer is free again
        doubled = nx.add(t, t)            # a recorded reader
        gathered = hip.gather(t, hip.reshape(hip.from_host(np.array([3, 0], np.int32), dt.int32), (2, 1)), 0)  # an entry point
        s = win.delta()
        assert s["recorded"] >= 3
        assert np.array_equal(logical(doubled), 2 * src)
        assert np.array_equal(logical(gathered)[:, 0], src[[3, 0], 0])
        assert np.array_equal(logical(t), src)
        # a second upload into the same block comes after the first
        hip._check(hip._lib.nxh_memcpy_h2d(hip._h, t.buffer.ptr, (src + 100).ctypes.data, src.nbytes))
        assert np.array_equal(logical(t), src + 100)


def test_attention_writes_the_merged_heads_directly(hip, oracle):
    """attention.ml:218-265: contiguous (swapaxes 1 2 (attention ...)). The copy is recorded; as the
    attention result's only reader it becomes the end of the run, and the kernel writes through the
    copy's output with permuted strides: no copy kernel, same bits."""
    rng = np.random.default_rng(40)
    d = dt.bfloat16
    b, h, s, hd = 2, 3, 80, 64
    nx = Nx(hip)
    model = Gpt2(nx, Config())
    q, k, v = (tensor(hip, encode(rng.standard_normal((b, h, s, hd)), d, oracle), d) for _ in range(3))

    def merged():
        idx = nx.arange(dt.int32, 0, s, 1)
        mask = nx.less_equal(nx.reshape((1, s), idx), nx.reshape((s, 1), idx))
        a = model.scaled_dot_product_attention(q, k, v, mask)
        return nx.reshape((b, s, h * hd), nx.contiguous(nx.swapaxes(1, 2, a)))

    direct = logical(hip.contiguous(hip.permute(hip.attention(q, k, v, 1.0 / math.sqrt(hd), masked_value=float("-inf"), causal=True),
                                                (0, 2, 1, 3)))).reshape(b, s, h * hd)
    with deferred(hip) as win:
        got = logical(merged())
        st = win.delta()
    assert (st["attention"], st["issued"], st["fallbacks"]) == (1, 0, 0), st   # the copy was not issued
    assert hip.last_path() == "attention_fused"
    same_bits(got, direct, "attention into the merged layout against attention followed by the copy")


def test_a_freed_scalar_shared_by_two_runs_is_written_for_a_member_that_stays_behind(hip, oracle):
    """One scalar tensor read by two GELU runs rides along with neither; its handle is dropped
    before the record executes, so it is not filled there. An interior result of one run is
    still held: when it is read afterwards, its entry is issued as recorded and multiplies by
    that scalar, which must have been written by then."""
    rng = np.random.default_rng(77)
    nx = Nx(hip)
    d = dt.float32
    xs = [tensor(hip, rng.standard_normal((48, 96)).astype(np.float32), d) for _ in range(2)]

    def gelu_with(x, c3, keep):
        # fn.ml:31-38 with the 0.044715 scalar handed in, so that two runs can share one tensor
        x3 = nx.mul(x, nx.mul(x, x))
        t = nx.mul(x3, c3)
        keep.append(t)
        inner = nx.mul_s(nx.add(x, t), math.sqrt(2.0 / math.pi))
        return nx.mul_s(nx.mul(x, nx.add_s(nx.tanh(inner), 1.0)), 0.5)

    kept_e = []
    c3 = nx.scalar(d, 0.044715)
    eager = [logical(gelu_with(x, c3, kept_e)) for x in xs]
    eager_t = logical(kept_e[0])
    del c3, kept_e
    # the small blocks the allocator hands out next hold another value: a scalar that is
    # recorded but never filled does not equal 0.044715 by accident
    poison = [hip.full(d, (), 123.0) for _ in range(16)]
    hip.synchronize()
    del poison
    with deferred(hip) as win:
        kept = []
        c3 = nx.scalar(d, 0.044715)
        outs = [gelu_with(x, c3, kept) for x in xs]
        held = kept[0]  # an interior of the first run stays referenced
        del kept, c3     # the shared scalar's handle goes before anything executes
        got = [logical(o) for o in outs]
        s = win.delta()
        assert s["gelu_tanh"] == 2 and s["postponed"] >= 1, s
        got_t = logical(held)  # issued as recorded now: x3 * c3
    for g, e in zip(got, eager):
        same_bits(g, e, "gelu with a shared scalar")
    same_bits(got_t, eager_t, "the held interior result, computed from the shared scalar")
