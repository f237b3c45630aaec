"""Kaun's GPT-2 forward issued by the compiled host (raven_amd/host_c/kaun_gpt2_host.c) through
the C ABI, one library call per primitive, no Python in the process: its logits are bit for bit
those of the Python mirror issuing the same sequence, eagerly and with the deferred mode on, with
handles freed at once and with every free held back until the logits have been read."""

import json
import subprocess

import numpy as np
import pytest

from helpers import encode, logical, same_bits
from raven_amd import _ffi, build
from raven_amd import dtype as dt
from raven_amd.kaun_gpt2 import Config, Gpt2, host_params, upload
from raven_amd.nx_frontend import Nx

pytestmark = pytest.mark.gpu


def leaves_in_file_order(hp):
    yield hp["wte"]
    yield hp["wpe"]
    for b in hp["blocks"]:
        yield from (b["ln1"]["gamma"], b["ln1"]["beta"])
        for n in ("q", "k", "v", "out"):
            yield from (b["attn"][n]["w"], b["attn"][n]["b"])
        yield from (b["ln2"]["gamma"], b["ln2"]["beta"], b["fc"]["w"], b["fc"]["b"], b["proj"]["w"], b["proj"]["b"])
    yield from (hp["ln_f"]["gamma"], hp["ln_f"]["beta"])


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float32], ids=lambda d: d.name)
def test_the_compiled_host_matches_the_python_mirror(hip, oracle, tmp_path, d):
    assert build.GPT2_HOST_BIN.exists(), "run __graft_entry__.build() first"
    cfg = Config(vocab_size=1031, n_positions=128, n_embd=256, n_layer=2, n_head=4, n_inner=1024)
    hp = host_params(cfg, seed=26, stddev=0.05)
    rng = np.random.default_rng(27)
    for b in hp["blocks"]:  # layer-norm parameters away from 1 and 0, so that they are seen
        for ln in (b["ln1"], b["ln2"]):
            ln["gamma"] = (1 + 0.1 * rng.standard_normal(cfg.n_embd)).astype(np.float32)
            ln["beta"] = (0.1 * rng.standard_normal(cfg.n_embd)).astype(np.float32)
    ids = rng.integers(0, cfg.vocab_size, (2, 96)).astype(np.int32)
    enc = lambda a, dd: encode(a, dd, oracle)  # noqa: E731
    with open(tmp_path / "params.bin", "wb") as f:
        for a in leaves_in_file_order(hp):
            f.write(np.ascontiguousarray(enc(a, d)).tobytes())
    ids.tofile(tmp_path / "ids.bin")

    counted = ("recorded", "issued", "fallbacks", "softmax_rows", "layer_norm_rows", "gelu_tanh", "attention", "linear", "linear_gelu")

    def python_logits(deferred):
        nx = Nx(hip)
        params = upload(nx, hp, d, enc)
        t_ids = nx.create(dt.int32, ids.shape, ids)
        hip.set_deferred(deferred)
        try:
            before = hip.deferred_stats()
            out = logical(Gpt2(nx, cfg).logits(params, t_ids))
            after = hip.deferred_stats()
            return out, {k: after[k] - before[k] for k in counted}
        finally:
            hip.set_deferred(False)

    want = {"eager": python_logits(False)[0]}
    want["deferred"], mirror_stats = python_logits(True)
    want["late"] = want["deferred"]
    L = cfg.n_layer
    for mode in ("eager", "deferred", "late"):
        out = tmp_path / f"logits_{mode}.bin"
        cmd = [str(build.GPT2_HOST_BIN), str(_ffi.LIB_PATH), "--vocab", str(cfg.vocab_size), "--positions", str(cfg.n_positions),
               "--embd", str(cfg.n_embd), "--layers", str(L), "--heads", str(cfg.n_head), "--inner", str(cfg.n_inner),
               "--batch", "2", "--seq", "96", "--dtype", "bf16" if d is dt.bfloat16 else "f32",
               "--params", str(tmp_path / "params.bin"), "--ids", str(tmp_path / "ids.bin"), "--logits", str(out), "--mode", mode]
        r = subprocess.run(cmd, capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stdout + r.stderr
        s = json.loads(r.stdout.strip().splitlines()[-1])
        got = np.fromfile(out, dtype=want[mode].dtype).reshape(want[mode].shape)
        same_bits(got, want[mode], f"compiled host, {mode}, against the Python mirror")
        if mode == "eager":
            assert s["recorded"] == 0
            continue
        # the same record, the same runs found, the same few primitives issued as recorded
        assert {k: s[k] for k in counted} == mirror_stats, (s, mirror_stats)
        mlp = L if d is dt.bfloat16 else 0  # linear + GELU as one GEMM (16-bit dtypes)
        assert (s["layer_norm_rows"], s["gelu_tanh"], s["linear"], s["linear_gelu"], s["fallbacks"]) == (2 * L + 1, L - mlp, 6 * L - mlp, mlp, 0), s
        if d is dt.bfloat16:  # the sum of the two embeddings and the tied head's matmul, nothing else
            assert s["issued"] == 2, s
        assert (s["attention"], s["softmax_rows"]) == ((L, 0) if d is dt.bfloat16 else (0, L)), s
        assert s["materialised"] == 0, s
        if mode == "late":
            assert s["postponed"] > 50 * L, s
