"""The fused row kernels (softmax_rows, layer_norm_rows, gelu_tanh) through the
C ABI against the op-by-op sequences they stand for.

Two references per case: the sequence of primitives on the CPU oracle (the
reference's lowering, frontend.ml:4242-4252, kaun/lib/{layer_norm,fn,attention}.ml)
and the same sequence on the GPU backend. Elementwise steps are the same
expressions with the same rounding points, so against the GPU sequence only the
order of a row's sum can differ: a few ulp of the result dtype. gelu has no sum
and must equal the GPU sequence bit for bit."""

import numpy as np
import pytest

from helpers import TOL, close, decode, encode, logical, pair, same_bits
from raven_amd import dtype as dt
from raven_amd.kaun_gpt2 import Config, Gpt2, LayerNorm
from raven_amd.nx_frontend import Nx

pytestmark = pytest.mark.gpu

ULP = {"float64": 2.0 ** -52, "float32": 2.0 ** -23, "float16": 2.0 ** -10, "bfloat16": 2.0 ** -7}
FLOATS = [dt.float32, dt.bfloat16, dt.float16, dt.float64]


def within_ulps(got, want, d, oracle, n, what=""):
    """|got - want| <= n ulp of dtype d at the magnitude of want (+ the smallest
    normal as absolute slack for results that round to zero)."""
    close(got, want, d, oracle, n * ULP[d.name], 1e-37 if d is not dt.float16 else 1e-7, what)


def softmax_sequence(B, x, scale, mask, out_dtype):
    """attention.ml:93-108: scale, mask against -inf, softmax, cast."""
    nx = Nx(B)
    t = x
    if scale is not None:
        t = nx.mul_s(t, scale)
    if mask is not None:
        t = nx.where(mask, t, nx.scalar_like(t, float("-inf")))
    t = nx.softmax(t)
    return nx.cast(out_dtype, t) if out_dtype is not None else t


@pytest.mark.parametrize("d", FLOATS, ids=lambda d: d.name)
@pytest.mark.parametrize("shape", [(2, 3, 64, 64), (5, 770), (3, 2050), (2, 4100), (1, 8192), (4, 1), (3, 8196), (2, 50257)],
                         ids=lambda s: "x".join(map(str, s)))
def test_softmax_rows_matches_the_sequence(hip, oracle, d, shape):
    rng = np.random.default_rng(sum(shape) + d.tag)
    x = encode(rng.standard_normal(shape) * 4, d, oracle)
    hx, ox = pair(x, d, hip, oracle)
    for scale, masked, cast in ((None, False, None), (0.125, True, None),
                                (0.125, True, dt.bfloat16 if d is dt.float32 else None),
                                (None, False, dt.float16 if d is dt.float32 else None)):
        hm = om = None
        if masked:
            n = shape[-1]
            tri = np.tril(np.ones((shape[-2], n), np.uint8), k=max(0, n - shape[-2]))
            hm, om = (B.expand(B.reshape(B.from_host(tri, dt.bool_), (1,) * (len(shape) - 2) + tri.shape), shape)
                      for B in (hip, oracle))
        got = hip.softmax_rows(hx, scale, hm, float("-inf") if masked else None, cast)
        assert hip.last_path() == ("softmax_rows_long" if shape[-1] > 8192 else "softmax_rows")
        od = cast or d
        want_cpu = logical(softmax_sequence(oracle, ox, scale, om, cast))
        want_gpu = logical(softmax_sequence(hip, hx, scale, hm, cast))
        what = f"{d.name} {shape} scale={scale} mask={masked} cast={cast and cast.name}"
        within_ulps(logical(got), want_gpu, od, oracle, 4 if od.itemsize == 2 else 16, what + " vs GPU sequence")
        close(logical(got), want_cpu, od, oracle, TOL[od.name][1], 1e-30, what + " vs oracle sequence")
        rows = decode(logical(got), od, oracle).sum(-1)
        assert np.all(np.abs(rows - 1) <= 8 * shape[-1] ** 0.5 * ULP[od.name] + 1e-6)


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16], ids=lambda d: d.name)
@pytest.mark.parametrize("start, width", [(0, 8201), (1, 8199), (2, 8205), (3, 9000), (1, 8193), (4, 8203), (0, 9011)])
def test_long_rows_off_their_vector_boundaries(hip, oracle, d, start, width):
    """Rows of a window [3, start:start+width] of a [3, 9011] matrix start off a 4-element boundary by
    a different amount each (9011 is odd). Where the fresh result's rows are off by the same amounts
    (start = 4, width = 8203: both row pitches are 3 modulo 4) the long-row kernels move vectors and
    take head and tail one element to a lane; the other windows move single elements. Both must
    agree with the result on a contiguous copy of the window within the reassociation of a row's
    sum."""
    rng = np.random.default_rng(start * 10007 + width + d.tag)
    wide = encode(rng.standard_normal((3, 9011)) * 2, d, oracle)
    gamma = encode(rng.standard_normal(width) * 0.5 + 1, d, oracle)
    beta = encode(rng.standard_normal(width) * 0.1, d, oracle)
    hw = hip.reshape(hip.from_host(wide, d), (3, 9011))
    view = hip.shrink(hw, [(0, 3), (start, start + width)])
    flat = hip.reshape(hip.from_host(np.ascontiguousarray(wide[:, start:start + width]), d), (3, width))
    got, want = hip.softmax_rows(view), hip.softmax_rows(flat)
    assert hip.last_path() == "softmax_rows_long"
    within_ulps(logical(got), logical(want), d, oracle, 4 if d.itemsize == 2 else 16, f"softmax {d.name} {start}+{width}")
    hg, hb = hip.from_host(gamma, d), hip.from_host(beta, d)
    got, want = hip.layer_norm_rows(view, hg, hb, 1e-5), hip.layer_norm_rows(flat, hg, hb, 1e-5)
    assert hip.last_path() == "layer_norm_rows_long"
    step = ULP[d.name] * float(np.abs(decode(beta, d, oracle)).max())
    close(logical(got), logical(want), d, oracle, 2 * ULP[d.name] + 1e-5, 1e-5 + step, f"layer norm {d.name} {start}+{width}")


def test_softmax_rows_special_values_and_errors(hip, oracle):
    x = np.zeros((6, 8), np.float32)
    x[0] = np.arange(8)
    x[1, 3] = np.nan              # a NaN poisons its row (max keeps NaN)
    x[2] = -np.inf                # exp(-inf - -inf) = NaN
    x[3, 2] = np.inf              # inf - inf = NaN at that element, 0 elsewhere
    x[4] = 1e30
    mask = np.ones((6, 8), np.uint8)
    mask[5] = 0                   # fully masked row: -inf everywhere
    hx, ox = pair(x, dt.float32, hip, oracle)
    hm, om = pair(mask, dt.bool_, hip, oracle)
    got = logical(hip.softmax_rows(hx, None, hm, float("-inf")))
    want = logical(softmax_sequence(oracle, ox, None, om, None))
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.allclose(got[~np.isnan(got)], want[~np.isnan(want)], rtol=1e-6)
    assert np.isnan(got[1]).all() and np.isnan(got[2]).all() and np.isnan(got[5]).all()
    # the 16-bit outputs take the short exponential, quotient and hardware maximum: same NaN rows
    for od in (dt.bfloat16, dt.float16):
        got16 = decode(logical(hip.softmax_rows(hx, None, hm, float("-inf"), od)), od, oracle)
        want16 = decode(logical(softmax_sequence(oracle, ox, None, om, od)), od, oracle)
        assert np.array_equal(np.isnan(got16), np.isnan(want16)), od.name
        assert np.allclose(got16[~np.isnan(got16)], want16[~np.isnan(want16)], rtol=2 * ULP[od.name], atol=1e-30)
    # a masked value other than -inf, taken as given
    got = logical(hip.softmax_rows(hx, 2.0, hm, -1e4))
    nx = Nx(oracle)
    want = logical(nx.softmax(nx.where(om, nx.mul_s(ox, 2.0), nx.scalar_like(ox, -1e4))))
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.allclose(got[~np.isnan(got)], want[~np.isnan(want)], rtol=1e-6)
    # a row that no block holds in registers: walked three times, same result
    long_ = logical(hip.softmax_rows(hip.full(dt.float32, (2, 8200), 0.0)))
    assert hip.last_path() == "softmax_rows_long" and np.array_equal(long_, np.full((2, 8200), np.float32(1) / np.float32(8200)))
    with pytest.raises(RuntimeError, match="contiguous"):
        hip.softmax_rows(hip.permute(hx, (1, 0)))
    with pytest.raises(RuntimeError):
        hip.softmax_rows(hip.full(dt.int32, (2, 8), 1))
    with pytest.raises(ValueError):
        hip.softmax_rows(hx, None, hip.full(dt.bool_, (6, 4), 1), 0.0)
    # strided rows (a column slice of a wider tensor) and an empty tensor
    wide = np.random.default_rng(5).standard_normal((9, 40)).astype(np.float32)
    hw, ow = pair(wide, dt.float32, hip, oracle, lambda B, t: B.shrink(t, [(0, 9), (3, 35)]))
    within_ulps(logical(hip.softmax_rows(hw)), logical(Nx(oracle).softmax(ow)), dt.float32, oracle, 16)
    assert logical(hip.softmax_rows(hip.full(dt.float32, (0, 8), 0.0))).shape == (0, 8)


@pytest.mark.parametrize("d", FLOATS, ids=lambda d: d.name)
@pytest.mark.parametrize("shape", [(4, 33, 768), (7, 770), (3, 4100), (5, 1), (3, 8196), (2, 50257)], ids=lambda s: "x".join(map(str, s)))
def test_layer_norm_rows_matches_the_sequence(hip, oracle, d, shape):
    rng = np.random.default_rng(sum(shape) + 7 * d.tag)
    n = shape[-1]
    x = encode(rng.standard_normal(shape) * 2 + 3, d, oracle)
    gamma = encode(rng.standard_normal(n) * 0.5 + 1, d, oracle)
    beta = encode(rng.standard_normal(n) * 0.1, d, oracle)
    hx, ox = pair(x, d, hip, oracle)
    hg, og = pair(gamma, d, hip, oracle)
    hb, ob = pair(beta, d, hip, oracle)
    eps = 1e-5
    got = hip.layer_norm_rows(hx, hg, hb, eps)
    assert hip.last_path() == ("layer_norm_rows_long" if n > 8192 else "layer_norm_rows")
    cfg = Config()
    want_cpu = logical(Gpt2(Nx(oracle), cfg).layer_norm(LayerNorm(og, ob), ox, eps))
    want_gpu = logical(Gpt2(Nx(hip), cfg).layer_norm(LayerNorm(hg, hb), hx, eps))
    what = f"{d.name} {shape}"
    # the mean and variance carry the sum-order difference into every element:
    # a few ulp of float32 in the statistics, at most one rounding step of d
    # (where y * gamma and beta nearly cancel, the one rounding step is one of y * gamma's size)
    step = ULP[d.name] * float(np.abs(decode(beta, d, oracle)).max())
    close(logical(got), want_gpu, d, oracle, 2 * ULP[d.name] + 1e-5, 1e-5 + step, what + " vs GPU sequence")
    close(logical(got), want_cpu, d, oracle, TOL[d.name][0], TOL[d.name][0], what + " vs oracle sequence")
    if d in (dt.bfloat16, dt.float16) and n > 1:
        frac = np.mean(logical(got) == want_gpu)
        assert frac > 0.98, (what, frac)
    # without the affine step: the normalisation alone (layer_norm.ml:43-49)
    got = logical(hip.layer_norm_rows(hx, None, None, eps))
    ones, zeros = (encode(np.full(n, v), d, oracle) for v in (1.0, 0.0))
    og1, ob0 = pair(ones, d, oracle, oracle)[0], pair(zeros, d, oracle, oracle)[0]
    want = logical(Gpt2(Nx(oracle), cfg).layer_norm(LayerNorm(og1, ob0), ox, eps))
    close(got, want, d, oracle, TOL[d.name][0], TOL[d.name][0], what + " plain")


def test_layer_norm_rows_errors(hip):
    x = hip.full(dt.float32, (4, 8), 1.0)
    with pytest.raises(ValueError):
        hip.layer_norm_rows(x, hip.full(dt.float32, (7,), 1.0), None, 1e-5)
    with pytest.raises(ValueError, match="eps"):
        hip.layer_norm_rows(x, None, None, -1.0)
    with pytest.raises(RuntimeError):
        hip.layer_norm_rows(x, hip.full(dt.float64, (8,), 1.0), None, 1e-5)
    assert np.array_equal(logical(hip.layer_norm_rows(hip.full(dt.float32, (1, 9000), 1.0), None, None, 1e-5)),
                          np.zeros((1, 9000), np.float32))
    assert hip.last_path() == "layer_norm_rows_long"
    # a constant row has zero variance: 0 / sqrt(eps) = 0
    assert np.array_equal(logical(hip.layer_norm_rows(x, None, None, 1e-5)), np.zeros((4, 8), np.float32))


@pytest.mark.parametrize("d", FLOATS, ids=lambda d: d.name)
def test_gelu_tanh_equals_the_sequence(hip, oracle, d):
    rng = np.random.default_rng(300 + d.tag)
    for shape in ((8, 3072), (1001,), (3, 5, 7)):
        v = rng.standard_normal(shape) * 3
        v.reshape(-1)[:6] = [0.0, -0.0, np.inf, -np.inf, np.nan, 60.0]
        x = encode(v, d, oracle)
        hx, ox = pair(x, d, hip, oracle)
        got = logical(hip.gelu_tanh(hx))
        assert hip.last_path() == "gelu_tanh"
        cfg = Config()
        want_gpu = logical(Gpt2(Nx(hip), cfg).gelu_approx(hx))
        nan = np.isnan(decode(want_gpu, d, oracle))
        assert np.array_equal(np.isnan(decode(got, d, oracle)), nan)
        same_bits(np.where(nan, np.zeros_like(got), got), np.where(nan, np.zeros_like(got), want_gpu),
                  f"{d.name} {shape}")
        want_cpu = logical(Gpt2(Nx(oracle), cfg).gelu_approx(ox))
        close(got, want_cpu, d, oracle, TOL[d.name][1], TOL[d.name][1], f"{d.name} {shape} vs oracle sequence")
    with pytest.raises(RuntimeError, match="contiguous"):
        hip.gelu_tanh(hip.permute(hip.full(d, (3, 4), 1.0), (1, 0)))


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_gelu_tanh_by_table_holds_the_arithmetic_bits_of_every_input(hip, d):
    """Four million elements or more of a 16-bit dtype go through a table of all 65 536 results:
    every entry must hold the bits the arithmetic kernel gives (NaN payloads included), for the
    default constants and for others (the table is made again), and in a captured graph."""
    rng = np.random.default_rng(310 + d.tag)
    pats = np.arange(65536, dtype=np.uint16)
    idx = rng.integers(0, 65536, 1 << 22).astype(np.int64)
    idx[:65536] = pats  # every input at least once
    small = hip.reshape(hip.from_host(pats, d), (65536,))
    big = hip.reshape(hip.from_host(pats[idx], d), (2048, 2048))
    for consts in ((0.044715, 0.7978845608028654, 1.0, 0.5), (0.05, 0.75, 1.0, 0.5), (0.044715, 0.7978845608028654, 1.0, 0.5)):
        want = logical(hip.gelu_tanh(small, consts))
        assert hip.last_path() == "gelu_tanh"
        got = logical(hip.gelu_tanh(big, consts))
        assert hip.last_path() == "gelu_tanh_table"
        assert np.array_equal(got.reshape(-1).view(np.uint16), want.view(np.uint16)[idx]), consts
    # a shape the table form leaves alone: not whole vectors
    odd = hip.reshape(hip.from_host(np.concatenate([pats[idx], pats[:3]]), d), ((1 << 22) + 3,))
    hip.gelu_tanh(odd)
    assert hip.last_path() == "gelu_tanh"
    hip.capture_begin()
    try:
        out = hip.gelu_tanh(big)
        path = hip.last_path()
    finally:
        graph = hip.capture_end()
    assert path == "gelu_tanh_table"
    for _ in range(2):
        graph.launch()
        hip.synchronize()
        assert np.array_equal(logical(out).reshape(-1).view(np.uint16), want.view(np.uint16)[idx])
    graph.destroy()
    # other constants inside a capture: the table cannot be refilled there, the arithmetic runs;
    # the table of the constants used last outside stays what it was
    other = (0.03, 0.7, 1.0, 0.5)
    want_other = logical(hip.gelu_tanh(small, other))
    hip.gelu_tanh(big)  # (the table holds the default constants again)
    assert hip.last_path() == "gelu_tanh_table"
    hip.capture_begin()
    try:
        out = hip.gelu_tanh(big, other)
        path = hip.last_path()
    finally:
        graph = hip.capture_end()
    assert path == "gelu_tanh"
    graph.launch()
    hip.synchronize()
    assert np.array_equal(logical(out).reshape(-1).view(np.uint16), want_other.view(np.uint16)[idx])
    got = logical(hip.gelu_tanh(big))
    assert hip.last_path() == "gelu_tanh_table"
    assert np.array_equal(got.reshape(-1).view(np.uint16), want.view(np.uint16)[idx])
    graph.destroy()


def test_a_recorded_gelu_keeps_its_table_when_other_constants_come_later(hip):
    """A recorded graph reads the table that was there when it was captured. A later eager call with
    other constants must not refill that table (it takes the arithmetic while the graph lives): the
    graph's next replay still gives the results of its own constants. Once the graph is destroyed
    the table takes the other constants again. The same for the table of the linear + GELU epilogue."""
    d = dt.bfloat16
    rng = np.random.default_rng(77)
    pats = np.arange(65536, dtype=np.uint16)
    idx = rng.integers(0, 65536, 1 << 22).astype(np.int64)
    small = hip.reshape(hip.from_host(pats, d), (65536,))
    big = hip.reshape(hip.from_host(pats[idx], d), (2048, 2048))
    mine, other = (0.044715, 0.7978845608028654, 1.0, 0.5), (0.06, 0.7, 1.0, 0.5)
    want = {c: logical(hip.gelu_tanh(small, c)).view(np.uint16)[idx] for c in (mine, other)}
    n = 4 * 192
    x = hip.reshape(hip.from_host(np.zeros(128 * 64, np.uint16), d), (128, 64))
    w = hip.reshape(hip.from_host(np.zeros(64 * n, np.uint16), d), (64, n))
    b = hip.reshape(hip.from_host(pats[idx[:n]], d), (n,))
    want_lin = {c: logical(hip.gelu_tanh(hip.contiguous(hip.shrink(hip.linear(x, w, b), [(0, 1), (0, n)])), c)).view(np.uint16)
                for c in (mine, other)}
    hip.gelu_tanh(big, mine)  # the tables exist, made for `mine`
    hip.linear_gelu_tanh(x, w, b, mine)
    hip.capture_begin()
    try:
        out = hip.gelu_tanh(big, mine)
        path = hip.last_path()
        lin = hip.linear_gelu_tanh(x, w, b, mine)
    finally:
        graph = hip.capture_end()
    assert path == "gelu_tanh_table"
    try:
        got = logical(hip.gelu_tanh(big, other))
        assert hip.last_path() == "gelu_tanh"  # not by table: the graph's table stays
        assert np.array_equal(got.reshape(-1).view(np.uint16), want[other])
        got = logical(hip.linear_gelu_tanh(x, w, b, other)).view(np.uint16)
        assert np.array_equal(got, np.broadcast_to(want_lin[other], got.shape))
        for _ in range(2):
            graph.launch()
            hip.synchronize()
            assert np.array_equal(logical(out).reshape(-1).view(np.uint16), want[mine])
            assert np.array_equal(logical(lin).view(np.uint16), np.broadcast_to(want_lin[mine], got.shape))
    finally:
        graph.destroy()
    got = logical(hip.gelu_tanh(big, other))
    assert hip.last_path() == "gelu_tanh_table"
    assert np.array_equal(got.reshape(-1).view(np.uint16), want[other])
    got = logical(hip.linear_gelu_tanh(x, w, b, other)).view(np.uint16)
    assert np.array_equal(got, np.broadcast_to(want_lin[other], got.shape))
