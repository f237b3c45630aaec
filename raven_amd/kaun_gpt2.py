"""The Kaun GPT-2 forward as the reference issues it, eagerly, one backend call
per primitive: packages/kaun/examples/04-gpt2/gpt2.ml:165-200 (``block_apply``,
``logits``) over packages/kaun/lib/{embedding,linear,layer_norm,attention,fn}.ml.

Parameters are plain records of backend tensors; every ``apply`` is a pure
function of them, as in Kaun. The frontend functions come from
``raven_amd.nx_frontend.Nx`` bound to the backend under test, so the same code
drives the GPU backend and the CPU oracle.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional

import numpy as np

from . import dtype as dt
from .nx_frontend import Nx

LOW_PRECISION = ("float16", "bfloat16", "float8_e4m3", "float8_e5m2")
SQRT_2_OVER_PI = 0.7978845608028654  # fn.ml:29


@dataclass
class Config:
    """gpt2.ml:13-21. ``small()`` is GPT-2 124M."""
    vocab_size: int = 50257
    n_positions: int = 1024
    n_embd: int = 768
    n_layer: int = 12
    n_head: int = 12
    n_inner: int = 3072
    layer_norm_eps: float = 1e-5

    @staticmethod
    def small() -> "Config":
        return Config()


@dataclass
class Linear:
    w: object  # [inputs, outputs]
    b: Optional[object]  # [outputs]


@dataclass
class LayerNorm:
    gamma: object
    beta: object


@dataclass
class Attention:
    q: Linear
    k: Linear
    v: Linear
    out: Linear


@dataclass
class Block:
    ln1: LayerNorm
    attn: Attention
    ln2: LayerNorm
    fc: Linear
    proj: Linear


@dataclass
class Params:
    wte: object  # [vocab, n_embd]
    wpe: object  # [n_positions, n_embd]
    blocks: List[Block]
    ln_f: LayerNorm


def host_params(cfg: Config, seed: int, stddev: float = 0.02) -> dict:
    """Random-init weights on the host as float32, one N(0, stddev) draw per leaf
    in a fixed order from one seeded generator; layer-norm gamma = 1, beta = 0
    (layer_norm.ml:27-30). Biases are drawn too so that the bias adds see data."""
    rng = np.random.default_rng(seed)

    def normal(*shape):
        return (rng.standard_normal(shape) * stddev).astype(np.float32)

    def linear(i, o):
        return {"w": normal(i, o), "b": normal(o)}

    def ln():
        return {"gamma": np.ones(cfg.n_embd, np.float32), "beta": np.zeros(cfg.n_embd, np.float32)}

    d = cfg.n_embd
    return {
        "wte": normal(cfg.vocab_size, d),
        "wpe": normal(cfg.n_positions, d),
        "blocks": [{"ln1": ln(),
                    "attn": {n: linear(d, d) for n in ("q", "k", "v", "out")},
                    "ln2": ln(), "fc": linear(d, cfg.n_inner), "proj": linear(cfg.n_inner, d)}
                   for _ in range(cfg.n_layer)],
        "ln_f": ln(),
    }


def upload(nx: Nx, host: dict, dtype: dt.DType, encode) -> Params:
    """Moves host float32 leaves to the backend in ``dtype``. ``encode(values,
    dtype)`` yields the dtype's storage array (the caller's narrowing rule, so
    both backends receive identical bytes)."""

    def leaf(a):
        return nx.create(dtype, a.shape, encode(a, dtype))

    def lin(p):
        return Linear(leaf(p["w"]), leaf(p["b"]))

    def ln(p):
        return LayerNorm(leaf(p["gamma"]), leaf(p["beta"]))

    return Params(
        wte=leaf(host["wte"]), wpe=leaf(host["wpe"]),
        blocks=[Block(ln(b["ln1"]), Attention(*(lin(b["attn"][n]) for n in ("q", "k", "v", "out"))),
                      ln(b["ln2"]), lin(b["fc"]), lin(b["proj"])) for b in host["blocks"]],
        ln_f=ln(host["ln_f"]))


class Gpt2:
    def __init__(self, nx: Nx, cfg: Config):
        self.nx, self.cfg = nx, cfg

    # embedding.ml:31-36
    def embedding(self, table, indices):
        rows = self.nx.take(table, indices, axis=0)
        return self.nx.reshape(tuple(indices.shape) + (table.shape[1],), rows)

    # linear.ml:50-52
    def linear(self, p: Linear, x):
        y = self.nx.matmul(x, p.w)
        return y if p.b is None else self.nx.add(y, p.b)

    # layer_norm.ml:43-68: statistics in a float32 island for narrow floats
    def _normalize(self, x, eps):
        nx = self.nx
        axes = [len(x.shape) - 1]
        mu = nx.mean(x, axes, keepdims=True)
        xc = nx.sub(x, mu)
        var = nx.mean(nx.mul(xc, xc), axes, keepdims=True)
        return nx.div(xc, nx.sqrt(nx.add_s(var, eps)))

    def layer_norm(self, p: LayerNorm, x, eps):
        nx = self.nx
        if x.dtype.name in LOW_PRECISION:
            normalized = nx.cast(x.dtype, self._normalize(nx.cast(dt.float32, x), eps))
        else:
            normalized = self._normalize(x, eps)
        return nx.add(nx.mul(normalized, p.gamma), p.beta)

    # fn.ml:31-38
    def gelu_approx(self, x):
        nx = self.nx
        x3 = nx.mul(x, nx.mul(x, x))
        inner = nx.mul_s(nx.add(x, nx.mul_s(x3, 0.044715)), SQRT_2_OVER_PI)
        return nx.mul_s(nx.mul(x, nx.add_s(nx.tanh(inner), 1.0)), 0.5)

    # attention.ml:67-110
    def scaled_dot_product_attention(self, q, k, v, mask):
        nx = self.nx
        scale = 1.0 / math.sqrt(float(q.shape[-1]))
        kr = len(k.shape)

        def weights(q, k):
            scores = nx.mul_s(nx.matmul(q, nx.swapaxes(kr - 2, kr - 1, k)), scale)
            if mask is not None:
                scores = nx.where(mask, scores, nx.scalar_like(scores, float("-inf")))
            return nx.softmax(scores)

        if q.dtype.name in LOW_PRECISION:
            probs = nx.cast(q.dtype, weights(nx.cast(dt.float32, q), nx.cast(dt.float32, k)))
        else:
            probs = weights(q, k)
        return nx.matmul(probs, v)

    # attention.ml:218-265
    def attention(self, p: Attention, x, num_heads, causal=True):
        nx = self.nx
        shape = tuple(x.shape)
        rank = len(shape)
        embed = p.q.w.shape[0]
        head_dim = embed // num_heads
        seq = shape[rank - 2]

        def split(t):
            return nx.swapaxes(rank - 2, rank - 1, nx.reshape(shape[:rank - 1] + (num_heads, head_dim), t))

        def merge(t):
            return nx.reshape(shape, nx.contiguous(nx.swapaxes(rank - 2, rank - 1, t)))

        q, k, v = split(self.linear(p.q, x)), split(self.linear(p.k, x)), split(self.linear(p.v, x))
        mask = None
        if causal:
            idx = nx.arange(dt.int32, 0, seq, 1)
            mask = nx.less_equal(nx.reshape((1, seq), idx), nx.reshape((seq, 1), idx))
        return self.linear(p.out, merge(self.scaled_dot_product_attention(q, k, v, mask)))

    # gpt2.ml:165-176
    def block(self, b: Block, x):
        nx, eps = self.nx, self.cfg.layer_norm_eps
        x = nx.add(x, self.attention(b.attn, self.layer_norm(b.ln1, x, eps), self.cfg.n_head, causal=True))
        return nx.add(x, self.linear(b.proj, self.gelu_approx(self.linear(b.fc, self.layer_norm(b.ln2, x, eps)))))

    # gpt2.ml:178-200
    def logits(self, p: Params, ids):
        nx = self.nx
        seq = ids.shape[1]
        if seq > self.cfg.n_positions:
            raise ValueError(f"Gpt2.logits: seq {seq} exceeds n_positions {self.cfg.n_positions}")
        pos = nx.reshape((1, seq), nx.arange(dt.int32, 0, seq, 1))
        x = nx.add(self.embedding(p.wte, ids), self.embedding(p.wpe, pos))
        for b in p.blocks:
            x = self.block(b, x)
        h = self.layer_norm(p.ln_f, x, self.cfg.layer_norm_eps)
        return nx.matmul(h, nx.transpose(p.wte))  # tied head: h @ wte^T, a strided B operand
