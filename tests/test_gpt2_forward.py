"""GPT-2 forward through the frontend/Kaun mirror.

CPU part: the primitive sequence, driven through the CPU oracle, is checked
against an independent float64 numpy statement of the GPT-2 mathematics (so a
wrong axis, a missing scale or a transposed head fails). GPU part: the same
sequence on the HIP backend against the oracle, f32 (tight) and bf16 (the
reference contract's bf16 tolerance, backend_contract.ml:179-188)."""

import numpy as np
import pytest

from helpers import decode, encode, logical
from raven_amd import dtype as dt
from raven_amd.kaun_gpt2 import Config, Gpt2, host_params, upload
from raven_amd.nx_frontend import Nx

TINY = Config(vocab_size=97, n_positions=16, n_embd=32, n_layer=2, n_head=4, n_inner=64)
SMALL = Config(vocab_size=1031, n_positions=128, n_embd=256, n_layer=2, n_head=4, n_inner=1024)


def numpy_gpt2(cfg, hp, ids):
    """float64 GPT-2 forward straight from the model's definition."""
    f = lambda a: np.asarray(a, np.float64)

    def ln(p, x):
        mu = x.mean(-1, keepdims=True)
        var = ((x - mu) ** 2).mean(-1, keepdims=True)
        return (x - mu) / np.sqrt(var + cfg.layer_norm_eps) * f(p["gamma"]) + f(p["beta"])

    def lin(p, x):
        return x @ f(p["w"]) + f(p["b"])

    b, s = ids.shape
    x = f(hp["wte"])[ids] + f(hp["wpe"])[np.arange(s)][None]
    hd = cfg.n_embd // cfg.n_head
    causal = np.tril(np.ones((s, s), bool))
    for blk in hp["blocks"]:
        h = ln(blk["ln1"], x)
        q, k, v = (lin(blk["attn"][n], h).reshape(b, s, cfg.n_head, hd).transpose(0, 2, 1, 3) for n in "qkv")
        sc = q @ k.transpose(0, 1, 3, 2) / np.sqrt(hd)
        sc = np.where(causal, sc, -np.inf)
        sc = np.exp(sc - sc.max(-1, keepdims=True))
        pr = sc / sc.sum(-1, keepdims=True)
        a = (pr @ v).transpose(0, 2, 1, 3).reshape(b, s, cfg.n_embd)
        x = x + lin(blk["attn"]["out"], a)
        h = lin(blk["fc"], ln(blk["ln2"], x))
        h = 0.5 * h * (1.0 + np.tanh(0.7978845608028654 * (h + 0.044715 * h ** 3)))
        x = x + lin(blk["proj"], h)
    return ln(hp["ln_f"], x) @ f(hp["wte"]).T


def run(backend, oracle, cfg, hp, ids, d):
    nx = Nx(backend)
    params = upload(nx, hp, d, lambda a, dd: encode(a, dd, oracle))
    t_ids = nx.create(dt.int32, ids.shape, ids.astype(np.int32))
    return Gpt2(nx, cfg).logits(params, t_ids)


def test_oracle_sequence_matches_gpt2_mathematics(oracle):
    hp = host_params(TINY, seed=3, stddev=0.2)
    for blk in hp["blocks"]:  # non-trivial affine parameters
        blk["ln1"]["gamma"] += 0.1
        blk["ln2"]["beta"] -= 0.05
    ids = np.random.default_rng(4).integers(0, TINY.vocab_size, (2, 8))
    got = logical(run(oracle, oracle, TINY, hp, ids, dt.float32)).astype(np.float64)
    want = numpy_gpt2(TINY, hp, ids)
    assert got.shape == (2, 8, TINY.vocab_size)
    assert np.max(np.abs(got - want)) <= 2e-4 * max(1.0, np.max(np.abs(want)))
    # causality: a change of the last token leaves earlier positions untouched
    ids2 = ids.copy()
    ids2[:, -1] = (ids2[:, -1] + 1) % TINY.vocab_size
    got2 = logical(run(oracle, oracle, TINY, hp, ids2, dt.float32))
    assert np.array_equal(got2[:, :-1], logical(run(oracle, oracle, TINY, hp, ids, dt.float32))[:, :-1])


def test_sequence_rejects_too_long_input(oracle):
    hp = host_params(TINY, seed=1)
    ids = np.zeros((1, TINY.n_positions + 1), np.int64)
    with pytest.raises(ValueError, match="exceeds n_positions"):
        run(oracle, oracle, TINY, hp, ids, dt.float32)


@pytest.mark.gpu
def test_gpt2_forward_f32_matches_oracle(hip, oracle):
    hp = host_params(SMALL, seed=16, stddev=0.05)
    ids = np.random.default_rng(17).integers(0, SMALL.vocab_size, (2, 96))
    got = logical(run(hip, oracle, SMALL, hp, ids, dt.float32)).astype(np.float64)
    want = logical(run(oracle, oracle, SMALL, hp, ids, dt.float32)).astype(np.float64)
    assert np.max(np.abs(got - want)) <= 1e-4 * max(1.0, np.max(np.abs(want)))
    assert np.mean(got.argmax(-1) == want.argmax(-1)) >= 0.999


@pytest.mark.gpu
def test_gpt2_forward_bf16_matches_oracle(hip, oracle):
    hp = host_params(SMALL, seed=16, stddev=0.05)
    ids = np.random.default_rng(17).integers(0, SMALL.vocab_size, (2, 96))
    got = decode(logical(run(hip, oracle, SMALL, hp, ids, dt.bfloat16)), dt.bfloat16, oracle)
    want = decode(logical(run(oracle, oracle, SMALL, hp, ids, dt.bfloat16)), dt.bfloat16, oracle)
    # bf16 transcendental tolerance of the reference contract: rel = abs = 6e-2
    assert np.all(np.abs(got - want) <= 6e-2 + 6e-2 * np.abs(want))
    assert np.mean(got.argmax(-1) == want.argmax(-1)) >= 0.97


@pytest.mark.gpu
@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16], ids=lambda d: d.name)
def test_gpt2_forward_through_the_window_on_the_gpu(hip, oracle, d):
    """The same frontend calls through the deferred-evaluation window: every
    softmax, layer norm and GELU runs as its fused kernel, and the logits agree
    with the eager GPU forward (a row sum's order is the only difference) and
    with the oracle."""
    from nx_window import Window

    hp = host_params(SMALL, seed=16, stddev=0.05)
    ids = np.random.default_rng(17).integers(0, SMALL.vocab_size, (2, 96))
    win = Window(hip)
    got = decode(logical(win.force(run(win, oracle, SMALL, hp, ids, d))), d, oracle)
    L = SMALL.n_layer
    assert (win.stats["layer_norm_rows"], win.stats["gelu_tanh"]) == (2 * L + 1, L)
    # head dim 64: bfloat16 runs the whole attention core as one kernel, float32 its softmax
    assert (win.stats["attention"], win.stats["softmax_rows"]) == ((L, 0) if d is dt.bfloat16 else (0, L))
    assert win.stats["linear"] == 6 * L   # every bias add, and the two residual adds, ride their GEMM
    assert win.stats["fallbacks"] == 0
    eager = decode(logical(run(hip, oracle, SMALL, hp, ids, d)), d, oracle)
    want = decode(logical(run(oracle, oracle, SMALL, hp, ids, d)), d, oracle)
    if d is dt.float32:
        assert np.max(np.abs(got - eager)) <= 2e-5 * max(1.0, np.max(np.abs(eager)))
        assert np.max(np.abs(got - want)) <= 1e-4 * max(1.0, np.max(np.abs(want)))
        assert np.mean(got.argmax(-1) == want.argmax(-1)) >= 0.999
    else:
        assert np.all(np.abs(got - want) <= 6e-2 + 6e-2 * np.abs(want))
        assert np.all(np.abs(got - eager) <= 6e-2 + 6e-2 * np.abs(eager))
        assert np.mean(got.argmax(-1) == want.argmax(-1)) >= 0.97
