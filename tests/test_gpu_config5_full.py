"""Config 5 at its stated shape: GPT-2 small (12 layers, d 768, 12 heads, FFN
3072, vocab 50257), batch 8 x seq 1024, bfloat16, weights from seed 16 and
token ids from seed 17 — and the attention call of that forward,
[8,12,1024,64] causal on head-split views.

The CPU oracle cannot run 8192 positions in seconds, but the model is causal:
logits[b, :k] depend only on ids[b, :k]. So the oracle runs batch row 0's first
K positions as a forward of its own and is compared with logits[0, :K, :] of
the full GPU forward, within the reference contract's bfloat16 tolerance
(rel = abs = 6e-2, backend_contract.ml:179-188), with the top-1 agreement
reported. The three GPU routes (eager, one call per primitive; through the
deferred-evaluation window; the windowed forward recorded and replayed as a
graph) are compared with each other over all 8192 positions, and so is the route
a binding gets: the library's own deferred mode (nxh_set_deferred), eagerly
issued and recorded into a graph, bit for bit against the Python window over the
same fused entry points. The compiled host (raven_amd/host_c) runs the same
forward from C at the same shape; its logits for batch row 0's first K
positions are held to the same oracle head."""

import math
import subprocess

import numpy as np
import pytest

from helpers import TOL, close, encode, logical
from raven_amd import _ffi, build
from raven_amd import dtype as dt
from raven_amd.kaun_gpt2 import Config, Gpt2, host_params, upload
from raven_amd.nx_frontend import Nx
from nx_window import Window

pytestmark = pytest.mark.gpu

BATCH, SEQ, K = 8, 1024, 128
REL = ABS = 6e-2


def bf16_values(u16):
    return (np.ascontiguousarray(u16).astype(np.uint32) << 16).view(np.float32)


def compare_logits(got, want, what):
    """Row by row (a [1024, 50257] float32 pair at a time): contract tolerance,
    top-1 agreement, largest absolute difference."""
    assert got.shape == want.shape, (got.shape, want.shape)
    g2, w2 = got.reshape(-1, got.shape[-1]), want.reshape(-1, want.shape[-1])
    agree, worst, rows = 0, 0.0, g2.shape[0]
    for r0 in range(0, rows, 1024):
        g, w = bf16_values(g2[r0:r0 + 1024]), bf16_values(w2[r0:r0 + 1024])
        assert not np.isnan(g).any() and not np.isnan(w).any(), what
        err = np.abs(g - w)
        lim = ABS + REL * np.abs(w)
        assert np.all(err <= lim), (what, r0, float((err - lim).max()))
        worst = max(worst, float(err.max()))
        agree += int(np.sum(g.argmax(-1) == w.argmax(-1)))
    print(f"[config 5] {what}: top-1 agreement {agree}/{rows} = {agree / rows:.4f}, max |diff| {worst:.4f}")
    return agree / rows


def test_attention_at_gpt2_shape_matches_the_sequence(hip, oracle):
    """The benchmarked attention call — 96 (batch, head) pairs, 16 query tiles
    each, late tiles first — against the oracle's primitive sequence on a sample
    of (batch, head) pairs, and against the GPU's own sequence on all of them."""
    rng = np.random.default_rng(1024)
    b, h, s, hd = BATCH, 12, SEQ, 64
    d = dt.bfloat16
    host = [encode(rng.standard_normal((b, s, h * hd)), d, oracle) for _ in range(3)]

    def split(B, t, nb):
        return B.permute(B.reshape(t, (nb, s, h, hd)), (0, 2, 1, 3))

    dev = [hip.reshape(hip.from_host(a, d), a.shape) for a in host]
    hq, hk, hv = (split(hip, t, b) for t in dev)
    scale = 1.0 / math.sqrt(hd)
    got_t = hip.attention(hq, hk, hv, scale, causal=True, masked_value=float("-inf"))
    assert hip.last_path() == "attention_fused"
    got = logical(got_t)
    model = Gpt2(Nx(hip), Config.small())
    idx = Nx(hip).arange(dt.int32, 0, s, 1)
    mask = Nx(hip).less_equal(Nx(hip).reshape((1, s), idx), Nx(hip).reshape((s, 1), idx))
    want_gpu = logical(model.scaled_dot_product_attention(hq, hk, hv, mask))
    # the one-pass kernel rounds the exponentials, the sequence the quotients: a few units of bfloat16 apart
    close(got, want_gpu, d, oracle, 2 * 2.0 ** -7, 8e-3, "vs the GPU's primitive sequence, all 96 heads")
    assert np.mean(got == want_gpu) > 0.4  # identical 16-bit outputs; the rest differ by a unit or two
    # the oracle's sequence on sampled (batch, head) pairs, first and last included
    onx = Nx(oracle)
    omodel = Gpt2(onx, Config.small())
    oidx = onx.arange(dt.int32, 0, s, 1)
    omask = onx.less_equal(onx.reshape((1, s), oidx), onx.reshape((s, 1), oidx))
    for bi, hi in ((0, 0), (3, 7), (7, 11)):
        sl = [np.ascontiguousarray(a[bi:bi + 1, :, hi * hd:(hi + 1) * hd]) for a in host]
        oq, ok, ov = (oracle.reshape(oracle.from_host(a, d), (1, 1, s, hd)) for a in sl)
        want = logical(omodel.scaled_dot_product_attention(oq, ok, ov, omask))
        close(got[bi:bi + 1, hi:hi + 1], want, d, oracle, TOL[d.name][0], TOL[d.name][0],
              f"vs the oracle's sequence, batch {bi} head {hi}")


def test_gpt2_small_forward_at_the_stated_shape(hip, oracle):
    cfg = Config.small()
    hp = host_params(cfg, seed=16)
    ids = np.random.default_rng(17).integers(0, cfg.vocab_size, (BATCH, SEQ)).astype(np.int32)
    enc = lambda a, d: encode(a, d, oracle)  # noqa: E731  the oracle's pinned f32 -> bf16 rule

    def forward(front, warm):
        nx = Nx(front)
        params = upload(nx, hp, dt.bfloat16, enc)
        t_ids = nx.create(dt.int32, ids.shape, ids)
        model = Gpt2(nx, cfg)
        if warm:
            del_me = model.logits(params, t_ids)
            del del_me
        return model, params, t_ids

    # eager: one backend call per primitive
    model, params, t_ids = forward(hip, warm=False)
    eager = logical(model.logits(params, t_ids))
    assert eager.shape == (BATCH, SEQ, cfg.vocab_size)
    del model, params, t_ids
    hip.trim()

    # through the window; then the windowed forward recorded once and replayed
    win = Window(hip)
    model, params, t_ids = forward(win, warm=True)
    windowed = logical(win.force(model.logits(params, t_ids)))
    L = cfg.n_layer
    assert (win.stats["attention"], win.stats["layer_norm_rows"], win.stats["gelu_tanh"]) == (2 * L, 2 * (2 * L + 1), 2 * L)
    assert win.stats["fallbacks"] == 0
    win.synchronize()
    win.capture_begin()
    try:
        out = win.force(model.logits(params, t_ids))
    finally:
        graph = win.capture_end()
    replays = []
    for _ in range(2):
        hip.assign(out, hip.expand(hip.full(dt.bfloat16, (), 0.0), out.shape))  # a replay must write every logit again
        graph.launch()
        hip.synchronize()
        replays.append(logical(out))
    del out
    graph.destroy()
    del model, params, t_ids, win
    hip.trim()

    assert np.array_equal(replays[0], windowed), "replay 1 differs from the windowed forward"
    assert np.array_equal(replays[1], windowed), "replay 2 differs from the windowed forward"

    # what a binding gets: the library's own deferred mode, issued eagerly and recorded into a graph
    model, params, t_ids = forward(hip, warm=False)
    hip.set_deferred(True)
    try:
        before = hip.deferred_stats()
        deferred = logical(model.logits(params, t_ids))
        after = hip.deferred_stats()
        s = {k: after[k] - before[k] for k in after}
        assert (s["attention"], s["layer_norm_rows"], s["linear_gelu"], s["linear"], s["fallbacks"]) == (L, 2 * L + 1, L, 5 * L, 0), s
        hip.synchronize()
        hip.capture_begin()
        try:
            out = model.logits(params, t_ids)
        finally:
            graph = hip.capture_end()
        hip.set_deferred(False)
        hip.assign(out, hip.expand(hip.full(dt.bfloat16, (), 0.0), out.shape))
        graph.launch()
        hip.synchronize()
        deferred_replay = logical(out)
        del out
        graph.destroy()
    finally:
        hip.set_deferred(False)
    del model, params, t_ids
    hip.trim()
    assert np.array_equal(deferred_replay, deferred), "the library's deferred forward: replay differs from the issued one"
    agree = compare_logits(deferred, windowed, "library deferred mode vs the Python window, all 8192 positions")
    assert agree >= 0.999
    assert np.array_equal(deferred, windowed), "the library's deferred mode and the Python window run the same fused calls"
    agree = compare_logits(windowed, eager, "window vs eager, all 8192 positions")
    assert agree >= 0.95

    # the oracle on batch row 0's first K positions (a forward of its own: the model is causal)
    onx = Nx(oracle)
    oparams = upload(onx, hp, dt.bfloat16, enc)
    o_ids = onx.create(dt.int32, (1, K), ids[:1, :K])
    want = logical(Gpt2(onx, cfg).logits(oparams, o_ids))
    assert want.shape == (1, K, cfg.vocab_size)
    for name, got in (("eager", eager), ("window", windowed), ("replay", replays[1]), ("library deferred mode", deferred)):
        agree = compare_logits(got[:1, :K], want, f"{name} vs oracle, batch row 0, first {K} positions")
        assert agree >= 0.90, (name, agree)


def test_the_compiled_host_at_the_stated_shape(hip, oracle, tmp_path):
    """kaun_gpt2_host issues the 12-layer forward at batch 8 x seq 1024 from C with the library's
    deferred mode on; logits[0, :K, :] go to a file and are held to the oracle's head, and are
    bit for bit what the Python mirror gets from the same library calls."""
    from test_gpu_c_host import leaves_in_file_order

    assert build.GPT2_HOST_BIN.exists(), "run __graft_entry__.build() first"
    cfg = Config.small()
    hp = host_params(cfg, seed=16)
    ids = np.random.default_rng(17).integers(0, cfg.vocab_size, (BATCH, SEQ)).astype(np.int32)
    enc = lambda a, d: encode(a, d, oracle)  # noqa: E731
    with open(tmp_path / "params.bin", "wb") as f:
        for a in leaves_in_file_order(hp):
            f.write(np.ascontiguousarray(enc(a, dt.bfloat16)).tobytes())
    ids.tofile(tmp_path / "ids.bin")
    out = tmp_path / "head.bin"
    cmd = [str(build.GPT2_HOST_BIN), str(_ffi.LIB_PATH), "--batch", str(BATCH), "--seq", str(SEQ), "--dtype", "bf16",
           "--params", str(tmp_path / "params.bin"), "--ids", str(tmp_path / "ids.bin"), "--logits", str(out),
           "--logits-bytes", str(K * cfg.vocab_size * 2), "--mode", "deferred"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    got = np.fromfile(out, dtype=np.uint16).reshape(1, K, cfg.vocab_size)
    # the Python mirror through the same library mode
    nx = Nx(hip)
    params = upload(nx, hp, dt.bfloat16, enc)
    t_ids = nx.create(dt.int32, ids.shape, ids)
    hip.set_deferred(True)
    try:
        mirror = logical(hip.contiguous(hip.shrink(Gpt2(nx, cfg).logits(params, t_ids), [(0, 1), (0, K), (0, cfg.vocab_size)])))
    finally:
        hip.set_deferred(False)
    del params, t_ids
    hip.trim()
    assert np.array_equal(got, mirror), "compiled host against the Python mirror, deferred mode"
    onx = Nx(oracle)
    oparams = upload(onx, hp, dt.bfloat16, enc)
    o_ids = onx.create(dt.int32, (1, K), ids[:1, :K])
    want = logical(Gpt2(onx, cfg).logits(oparams, o_ids))
    agree = compare_logits(got, want, f"compiled host (deferred mode) vs oracle, batch row 0, first {K} positions")
    assert agree >= 0.90
