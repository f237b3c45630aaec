"""The memory-side cache policy (nxh_set_cache_policy): which accesses of the elementwise
kernels go past the cache is a per-call decision that may change when bytes reach HBM and
never what they are. Checked three ways: every map operation of the layout matrix with
every access forced to stream (mode 7) against the CPU oracle, bit for bit; benchmark
config 2's step repeated until the policy streams by itself, against the oracle and
against the same step with the policy off; and that a working set that fits the cache
streams nothing."""

import numpy as np
import pytest

from helpers import INT_DTYPES, layouts, logical, pair, same_bits
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu

SHAPE = (5, 33, 70)


@pytest.fixture()
def streaming(hip):
    hip.set_cache_policy(7)
    yield hip
    hip.set_cache_policy(3)


@pytest.mark.parametrize("d", [dt.int8, dt.uint16, dt.int32, dt.int64, dt.float32, dt.float64, dt.complex128],
                         ids=lambda d: d.name)
def test_forced_streaming_is_bit_exact(streaming, oracle, d):
    hip = streaming
    rng = np.random.default_rng(700 + d.tag)
    before = hip.cache_policy_stats()
    for lname, src_shape, build in layouts(SHAPE):
        if d.is_complex:
            x = (rng.standard_normal(src_shape) + 1j * rng.standard_normal(src_shape)).astype(d.np_storage)
            y = (rng.standard_normal(SHAPE) + 1j * rng.standard_normal(SHAPE)).astype(d.np_storage)
        elif d in INT_DTYPES:
            info = np.iinfo(d.np_storage)
            x = rng.integers(info.min, info.max, src_shape, dtype=d.np_storage, endpoint=True)
            y = rng.integers(info.min, info.max, SHAPE, dtype=d.np_storage, endpoint=True)
        else:
            x, y = rng.standard_normal(src_shape).astype(d.np_storage), rng.standard_normal(SHAPE).astype(d.np_storage)
        hx, ox = pair(x, d, hip, oracle, build)
        hy, oy = pair(y, d, hip, oracle)
        for op in ("add", "mul"):
            same_bits(logical(hip.binary(op, hx, hy)), logical(oracle.binary(op, ox, oy)), f"{op}/{lname}")
        same_bits(logical(hip.unary("neg", hx)), logical(oracle.unary("neg", ox)), f"neg/{lname}")
        same_bits(logical(hip.contiguous(hx)), logical(oracle.contiguous(ox)), f"copy/{lname}")
        if not d.is_complex:
            hm, om = hip.compare("cmplt", hx, hy), oracle.compare("cmplt", ox, oy)
            same_bits(logical(hm), logical(om), f"cmplt/{lname}")
            same_bits(logical(hip.where(hm, hx, hy)), logical(oracle.where(om, ox, oy)), f"where/{lname}")
            for to in (dt.float16, dt.uint8, dt.int64):
                same_bits(logical(hip.cast(hx, to)), logical(oracle.cast(ox, to)), f"cast {to.name}/{lname}")
    after = hip.cache_policy_stats()
    assert after["streaming_out"] > before["streaming_out"] and after["streaming_in"] > before["streaming_in"]


@pytest.mark.parametrize("n", [1, 3, 4, 255, 1024 + 7, 100003])
def test_forced_streaming_ragged_lengths(streaming, oracle, n):
    hip = streaming
    rng = np.random.default_rng(n)
    for d in (dt.float32, dt.int16, dt.uint8):
        x = rng.integers(-100, 100, n).astype(d.np_storage)
        y = rng.integers(-100, 100, n).astype(d.np_storage)
        (hx, ox), (hy, oy) = pair(x, d, hip, oracle), pair(y, d, hip, oracle)
        same_bits(logical(hip.binary("add", hx, hy)), logical(oracle.binary("add", ox, oy)), f"add {d.name} n={n}")
        same_bits(logical(hip.cast(hx, dt.int8)), logical(oracle.cast(ox, dt.int8)), f"cast {d.name} n={n}")


def config2_step(B, a, b, ai, bi, shp):
    ap, aip = B.permute(a, (0, 2, 1)), B.permute(ai, (0, 2, 1))
    bx, bix = B.expand(b, shp), B.expand(bi, shp)
    half = B.expand(B.full(dt.float32, (), np.array([0.5], np.float32)), shp)
    v = B.cast(B.binary("mul", B.binary("add", ap, bx), half), dt.float16)
    s, p = B.binary("add", aip, bix), B.binary("mul", aip, bix)
    w = B.where(B.compare("cmplt", bix, aip), aip, bix)
    return v, s, p, w


def test_config2_step_streams_by_itself_and_keeps_its_bits(hip, oracle):
    """[64,512,512] f32 + int32 chains (496 MiB of tensors per step): after a few steps the
    results nothing reads back are written past the cache and the operands read once per
    step are read past it. Every step's results equal the oracle's."""
    shp = (64, 512, 512)
    rng = [np.random.default_rng(s) for s in (4, 5, 6, 7)]
    host = [rng[0].standard_normal(shp).astype(np.float32), rng[1].standard_normal((1, 512, 1)).astype(np.float32),
            rng[2].integers(-1000, 1001, shp).astype(np.int32), rng[3].integers(-1000, 1001, (1, 512, 1)).astype(np.int32)]
    dts = [dt.float32, dt.float32, dt.int32, dt.int32]
    want = [logical(t) for t in config2_step(oracle, *[pair(h, d, hip, oracle)[1] for h, d in zip(host, dts)], shp)]
    dev = [pair(h, d, hip, oracle)[0] for h, d in zip(host, dts)]
    hip.trim()
    hip.set_cache_policy(3)
    before = hip.cache_policy_stats()
    for step in range(6):
        got = config2_step(hip, *dev, shp)
        if step in (0, 5):
            for g, w, name in zip(got, want, ("v", "add", "mul", "where")):
                same_bits(logical(g), w, f"step {step}: {name}")
        del got
    after = hip.cache_policy_stats()
    assert after["streaming_out"] - before["streaming_out"] >= 4, (before, after)
    assert after["streaming_in"] - before["streaming_in"] >= 1, (before, after)
    hip.set_cache_policy(0)
    try:
        off = hip.cache_policy_stats()
        got = config2_step(hip, *dev, shp)
        for g, w, name in zip(got, want, ("v", "add", "mul", "where")):
            same_bits(logical(g), w, f"policy off: {name}")
        assert hip.cache_policy_stats() == off
    finally:
        hip.set_cache_policy(3)


def test_a_working_set_that_fits_streams_nothing(hip):
    """Three 32 MiB tensors in a loop: everything stays cached, nothing streams."""
    n = 8 << 20
    rng = np.random.default_rng(1)
    x = hip.reshape(hip.from_host(rng.standard_normal(n).astype(np.float32), dt.float32), (n,))
    y = hip.reshape(hip.from_host(rng.standard_normal(n).astype(np.float32), dt.float32), (n,))
    hip.trim()
    hip.set_cache_policy(3)
    before = hip.cache_policy_stats()
    for _ in range(8):
        z = hip.binary("mul", x, y)
        del z
    assert hip.cache_policy_stats() == before


def test_mode_is_validated(hip):
    with pytest.raises(ValueError):
        hip.set_cache_policy(8)


def test_forced_streaming_in_unfold_fold_and_the_column_scan(streaming, oracle):
    """The other kernels that take the policy's decision: unfold's stores and the one-pass column
    scan's stores (fold is in the loop as unfold's inverse). Forced to stream, their results are the oracle's."""
    hip = streaming
    rng = np.random.default_rng(720)
    for d in (dt.float32, dt.int16, dt.uint8, dt.float64):
        x = rng.integers(-50, 50, (2, 3, 16, 20)).astype(d.np_storage)
        (hx, ox) = pair(x, d, hip, oracle)
        args = ((3, 3), (1, 1), (1, 1), ((1, 1), (1, 1)))
        hu, ou = hip.unfold(hx, *args), oracle.unfold(ox, *args)
        same_bits(logical(hu), logical(ou), f"unfold {d.name}")
        same_bits(logical(hip.fold(hu, (16, 20), *args)), logical(oracle.fold(ou, (16, 20), *args)), f"fold {d.name}")
        args = ((3, 2), (2, 1), (1, 2), ((0, 1), (2, 0)))
        hu, ou = hip.unfold(hx, *args), oracle.unfold(ox, *args)
        same_bits(logical(hu), logical(ou), f"unfold strided {d.name}")
    y = rng.integers(-9, 9, (700, 260)).astype(np.int32)
    hy, oy = pair(y, dt.int32, hip, oracle)
    same_bits(logical(hip.associative_scan(0, "sum", hy)), logical(oracle.associative_scan(0, "sum", oy)), "column scan")
    assert hip.last_path() == "scan_cols"


def test_a_loop_of_large_unfolds_streams_by_itself(hip):
    """[8,64,128,128] f32 unfolded 3 x 3 (302 MB of windows nothing reads back): after a few calls
    the windows are written past the cache; the interior taps still equal the shifted input."""
    rng = np.random.default_rng(730)
    x = rng.standard_normal((8, 64, 128, 128)).astype(np.float32)
    hx = hip.reshape(hip.from_host(x, dt.float32), x.shape)
    hip.trim()
    hip.set_cache_policy(3)
    before = hip.cache_policy_stats()
    for _ in range(5):
        u = hip.unfold(hx, (3, 3), (1, 1), (1, 1), ((1, 1), (1, 1)))
        last = u
    after = hip.cache_policy_stats()
    assert after["streaming_out"] > before["streaming_out"], (before, after)
    got = logical(last).reshape(8, 64, 9, 128, 128)
    assert np.array_equal(got[:, :, 4], x)                       # the centre tap
    assert np.array_equal(got[:, :, 0, 1:, 1:], x[:, :, :-1, :-1])  # the top-left tap
    assert np.all(got[:, :, 0, 0, :] == 0)                       # its padding row


def test_forced_streaming_in_pad_and_cat(streaming, oracle):
    """pad and cat as one kernel take the policy's decision for their stores: forced to stream,
    vectors and single elements alike, the results are the oracle's."""
    hip = streaming
    rng = np.random.default_rng(740)
    for d in (dt.float32, dt.int16, dt.uint8, dt.float64, dt.complex128):
        for shape, padding in (((6, 40), ((1, 2), (4, 4))), ((3, 5, 7), ((0, 1), (2, 0), (3, 1)))):
            x = rng.integers(0, 100, shape).astype(d.np_storage)
            hx, ox = pair(x, d, hip, oracle)
            fill = np.array([7]).astype(d.np_storage)
            same_bits(logical(hip.pad(hx, padding, fill)), logical(oracle.pad(ox, padding, fill)), f"pad {d.name} {shape}")
            assert hip.last_path() == "pad_fused"
        parts = [rng.integers(0, 100, (4, n, 8)).astype(d.np_storage) for n in (3, 8, 1)]
        hs, os_ = zip(*(pair(p_, d, hip, oracle) for p_ in parts))
        for axis in (0, 1, 2):
            members = parts if axis == 1 else parts[:1] * 3
            hm, om = (hs, os_) if axis == 1 else (hs[:1] * 3, os_[:1] * 3)
            same_bits(logical(hip.cat(list(hm), axis)), logical(oracle.cat(list(om), axis)), f"cat {d.name} axis {axis}")
            assert hip.last_path() == "cat_fused"
            assert logical(hip.cat(list(hm), axis)).shape[axis] == sum(m.shape[axis] for m in members)


def test_a_loop_of_large_cats_streams_by_itself(hip):
    """4 x 64 MiB joined into 256 MiB that nothing reads back: after a few calls the result is
    written past the cache; its values stay the members'."""
    rng = np.random.default_rng(750)
    parts = [rng.integers(-1000, 1000, (2048, 8192)).astype(np.int32) for _ in range(4)]
    hs = [hip.reshape(hip.from_host(p_, dt.int32), p_.shape) for p_ in parts]
    hip.trim()
    hip.set_cache_policy(3)
    before = hip.cache_policy_stats()
    for _ in range(5):
        last = hip.cat(hs, 0)
    after = hip.cache_policy_stats()
    assert hip.last_path() == "cat_fused"
    assert after["streaming_out"] > before["streaming_out"], (before, after)
    got = logical(last)
    for i, p_ in enumerate(parts):
        assert np.array_equal(got[2048 * i:2048 * (i + 1)], p_)


def test_forced_streaming_in_softmax_rows(streaming, oracle):
    """The fused softmax reads its scores and writes its probabilities past the cache when the
    policy says so: forced, the result is what the kernel gives with plain accesses."""
    hip = streaming
    rng = np.random.default_rng(760)
    for shape, out_d in (((7, 300), dt.float32), ((3, 5, 1024), dt.bfloat16), ((9, 70), dt.float32)):
        x = rng.standard_normal(shape).astype(np.float32) * 3
        hx = hip.reshape(hip.from_host(x, dt.float32), shape)
        got = logical(hip.softmax_rows(hx, 0.125, None, None, out_d))
        hip.set_cache_policy(0)
        want = logical(hip.softmax_rows(hx, 0.125, None, None, out_d))
        hip.set_cache_policy(7)
        same_bits(got, want, f"softmax {shape} -> {out_d.name}")
    e = np.exp(x * 0.125 - (x * 0.125).max(-1, keepdims=True))
    assert np.allclose(got, e / e.sum(-1, keepdims=True), rtol=1e-5, atol=1e-7)


def test_a_loop_of_large_softmaxes_streams_by_itself(hip):
    """[24576,4096] float32 scores (402 MB) to bfloat16 probabilities nobody reads back."""
    rng = np.random.default_rng(770)
    x = rng.standard_normal((24576, 4096)).astype(np.float32)
    hx = hip.reshape(hip.from_host(x, dt.float32), x.shape)
    hip.trim()
    hip.set_cache_policy(3)
    before = hip.cache_policy_stats()
    for _ in range(5):
        last = hip.softmax_rows(hx, None, None, None, dt.bfloat16)
    after = hip.cache_policy_stats()
    assert after["streaming_out"] > before["streaming_out"] or after["streaming_in"] > before["streaming_in"], (before, after)
    got = (logical(last)[:64].astype(np.uint32) << 16).view(np.float32)
    e = np.exp(x[:64] - x[:64].max(-1, keepdims=True))
    assert np.allclose(got, e / e.sum(-1, keepdims=True), rtol=2 ** -7, atol=1e-7)
