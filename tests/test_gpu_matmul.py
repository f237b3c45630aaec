"""GPU parity of matmul against the CPU oracle and an f64 reference.

Tolerances are the reference GEMM suite's (packages/nx/lib/backend_c/test/
matmul_test.ml:831-974): f32 1e-3, f64 1e-9, f16 2e-2, bf16 6e-2 (relative to
the f64 product of the QUANTISED inputs, plus the same absolute term); integer
products are exact modulo 2^w."""

import numpy as np
import pytest

from helpers import TOL, close, decode, encode, logical, pair, same_bits
from raven_amd import dtype as dt

pytestmark = pytest.mark.gpu

MM_TOL = {"float32": 1e-3, "float64": 1e-9, "float16": 2e-2, "bfloat16": 6e-2,
          "float8_e4m3": 0.3, "float8_e5m2": 0.4, "complex64": 1e-3, "complex128": 1e-9}


def ref_f64(a, b, d, oracle):
    return np.matmul(decode(a, d, oracle), decode(b, d, oracle))


def check(hip, oracle, d, ha, hb, a_log, b_log, what):
    got = decode(logical(hip.matmul(ha, hb)), d, oracle)
    want = ref_f64(a_log, b_log, d, oracle)
    tol = MM_TOL[d.name]
    scale = np.sqrt(a_log.shape[-1])  # typical magnitude of a k-term sum of unit-variance products
    err = np.abs(got - want)
    lim = tol * (np.abs(want) + scale)
    assert got.shape == want.shape, what
    assert np.all(err <= lim), (what, float(err.max()), float(lim.min()))


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.float16, dt.float64, dt.float8_e4m3],
                         ids=lambda d: d.name)
def test_matmul_layouts(hip, oracle, d):
    rng = np.random.default_rng(1100 + d.tag)
    sizes = [(1, 1, 1), (3, 5, 7), (33, 70, 41), (128, 128, 128), (130, 257, 200), (257, 64, 129), (64, 300, 8)]
    for (m, k, n) in sizes:
        a = encode(rng.standard_normal((m, k)), d, oracle)
        b = encode(rng.standard_normal((k, n)), d, oracle)
        for ta in (False, True):
            for tb in (False, True):
                ha, _ = pair(np.ascontiguousarray(a.T) if ta else a, d, hip, oracle,
                             (lambda B, t: B.permute(t, (1, 0))) if ta else None)
                hb, _ = pair(np.ascontiguousarray(b.T) if tb else b, d, hip, oracle,
                             (lambda B, t: B.permute(t, (1, 0))) if tb else None)
                check(hip, oracle, d, ha, hb, a, b, f"{m}x{k}x{n} ta={ta} tb={tb}")
    # offset views and row-strided (every other row / column) operands
    a = encode(rng.standard_normal((70, 90)), d, oracle)
    b = encode(rng.standard_normal((100, 80)), d, oracle)
    ha, _ = pair(a, d, hip, oracle, lambda B, t: B.shrink(t, [(3, 67), (5, 85)]))
    hb, _ = pair(b, d, hip, oracle, lambda B, t: B.shrink(t, [(7, 87), (1, 78)]))
    check(hip, oracle, d, ha, hb, a[3:67, 5:85], b[7:87, 1:78], "offset")
    ha, _ = pair(a, d, hip, oracle,
                 lambda B, t: B.permute(B.shrink(B.reshape(t, (35, 2, 90)), [(0, 35), (0, 1), (0, 90)]), (0, 2, 1)))
    ha = hip.reshape(ha, (35, 90))
    check(hip, oracle, d, ha, hip.shrink(hb, [(0, 80), (0, 77)]) if False else
          pair(b[:90], d, hip, oracle)[0], a[::2], b[:90], "strided rows")


def test_matmul_batched_and_broadcast(hip, oracle):
    rng = np.random.default_rng(12)
    for d in (dt.float32, dt.bfloat16):
        a = encode(rng.standard_normal((2, 3, 40, 50)), d, oracle)
        b = encode(rng.standard_normal((2, 3, 50, 60)), d, oracle)
        ha, hb = pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0]
        check(hip, oracle, d, ha, hb, a, b, "batched 4-D")
        # [2,1,m,k] x [3,k,n] -> [2,3,m,n]
        a1, b1 = a[:, :1], b[0]
        ha, hb = pair(a1, d, hip, oracle)[0], pair(b1, d, hip, oracle)[0]
        check(hip, oracle, d, ha, hb, a1, b1, "broadcast")
        # rank-2 weight broadcast over a rank-3 batch, and a transposed K^T-style view
        w = encode(rng.standard_normal((50, 30)), d, oracle)
        x3 = a[0]
        check(hip, oracle, d, pair(x3, d, hip, oracle)[0], pair(w, d, hip, oracle)[0], x3, w, "x @ W")
        q = encode(rng.standard_normal((2, 3, 40, 16)), d, oracle)
        kt = encode(rng.standard_normal((2, 3, 40, 16)), d, oracle)
        hq = pair(q, d, hip, oracle)[0]
        hk = pair(kt, d, hip, oracle, lambda B, t: B.permute(t, (0, 1, 3, 2)))[0]
        check(hip, oracle, d, hq, hk, q, np.swapaxes(kt, -1, -2), "q @ k^T")


def test_matmul_vs_oracle_small(hip, oracle):
    """Same inputs through the oracle's k-ordered f32 accumulation: the two
    agree to within the tolerance, and exactly on small-integer data where
    every partial sum is representable (backend_contract.ml:2012-2021)."""
    rng = np.random.default_rng(13)
    for d in (dt.float32, dt.bfloat16, dt.float16):
        a = encode(rng.integers(-4, 5, (65, 96)).astype(np.float64), d, oracle)
        b = encode(rng.integers(-4, 5, (96, 130)).astype(np.float64), d, oracle)
        (ha, oa), (hb, ob) = pair(a, d, hip, oracle), pair(b, d, hip, oracle)
        got, want = logical(hip.matmul(ha, hb)), logical(oracle.matmul(oa, ob))
        if d is dt.float32:
            same_bits(got, want)
        else:
            assert np.max(np.abs(decode(got, d, oracle) - decode(want, d, oracle))) <= \
                MM_TOL[d.name] * np.max(np.abs(decode(want, d, oracle)))


@pytest.mark.parametrize("d", [dt.int8, dt.uint8, dt.int16, dt.int32, dt.uint32, dt.int64, dt.uint64],
                         ids=lambda d: d.name)
def test_matmul_int_exact(hip, oracle, d):
    rng = np.random.default_rng(1200 + d.tag)
    info = np.iinfo(d.np_storage)
    a = rng.integers(info.min, info.max, (19, 37), endpoint=True, dtype=d.np_storage)
    b = rng.integers(info.min, info.max, (37, 23), endpoint=True, dtype=d.np_storage)
    (ha, oa), (hb, ob) = pair(a, d, hip, oracle), pair(b, d, hip, oracle)
    same_bits(logical(hip.matmul(ha, hb)), logical(oracle.matmul(oa, ob)))
    hat, oat = (B.permute(t, (1, 0)) for B, t in ((hip, pair(a.T.copy(), d, hip, oracle)[0]),
                                                  (oracle, pair(a.T.copy(), d, hip, oracle)[1])))
    same_bits(logical(hip.matmul(hat, hb)), logical(oracle.matmul(oat, ob)))


def test_matmul_complex_and_edges(hip, oracle):
    rng = np.random.default_rng(14)
    for d in (dt.complex64, dt.complex128):
        a = (rng.standard_normal((9, 21)) + 1j * rng.standard_normal((9, 21))).astype(d.np_storage)
        b = (rng.standard_normal((21, 13)) + 1j * rng.standard_normal((21, 13))).astype(d.np_storage)
        got = logical(hip.matmul(pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0])).astype(np.complex128)
        want = a.astype(np.complex128) @ b.astype(np.complex128)
        assert np.allclose(got, want, rtol=MM_TOL[d.name], atol=MM_TOL[d.name])
    # k == 0 stores zeros; m == 0 / n == 0 are no-ops
    z = logical(hip.matmul(hip.buffer(dt.float32, (3, 0)), hip.buffer(dt.float32, (0, 2))))
    assert z.tolist() == [[0, 0], [0, 0], [0, 0]]
    assert logical(hip.matmul(hip.buffer(dt.float32, (0, 4)), hip.buffer(dt.float32, (4, 2)))).shape == (0, 2)
    with pytest.raises(ValueError):
        hip.matmul(hip.buffer(dt.float32, (3, 4)), hip.buffer(dt.float32, (5, 2)))
    with pytest.raises(RuntimeError):
        hip.matmul(hip.buffer(dt.bool_, (3, 4)), hip.buffer(dt.bool_, (4, 2)))


def test_matmul_cancellation_witness(hip, oracle):
    """matmul_test.ml:182-230: +a on the first k/2 columns, -a on the rest, B all
    b; the exact product is 0, which only an f32 accumulator rounded once
    reproduces (|C| <= 0.1 is the reference's bound)."""
    for d, (m, k, n) in [(dt.float16, (16, 4096, 24)), (dt.bfloat16, (16, 4096, 24)),
                         (dt.float16, (128, 4096, 128)), (dt.bfloat16, (200, 2304, 130))]:
        av = np.full((m, k), 1.3)
        av[:, k // 2:] *= -1
        a, b = encode(av, d, oracle), encode(np.full((k, n), 1.5), d, oracle)
        got = decode(logical(hip.matmul(pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0])), d, oracle)
        assert np.max(np.abs(got)) <= 0.1, (d.name, m, k, n, float(np.max(np.abs(got))))


def test_matmul_skinny_decode_shape(hip, oracle):
    rng = np.random.default_rng(15)
    for d in (dt.bfloat16, dt.float32):
        for m in (1, 8, 13):
            a = encode(rng.standard_normal((m, 1024)) * 0.5, d, oracle)
            b = encode(rng.standard_normal((1024, 2048)) * 0.5, d, oracle)
            ha, hb = pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0]
            check(hip, oracle, d, ha, hb, a, b, f"skinny m={m}")
            assert hip.last_path().startswith("gemm_skinny")
    # ragged shapes: K not a multiple of the row-group unroll, N ending inside a
    # lane's 16-byte vector (a column slice of a wider, aligned B), m = 16
    for d in (dt.float16, dt.float32):
        a = encode(rng.standard_normal((16, 1003)) * 0.5, d, oracle)
        bw = encode(rng.standard_normal((1003, 2056)) * 0.5, d, oracle)
        ha = pair(a, d, hip, oracle)[0]
        hb = pair(bw, d, hip, oracle, lambda B, t: B.shrink(t, [(0, 1003), (0, 2051)]))[0]
        check(hip, oracle, d, ha, hb, a, np.ascontiguousarray(bw[:, :2051]), "skinny ragged")
        assert hip.last_path().startswith("gemm_skinny")
        # whole 8-column vectors but a ragged K and a column count that ends inside a wave's tile
        hb = pair(bw, d, hip, oracle, lambda B, t: B.shrink(t, [(0, 1003), (8, 2048)]))[0]
        check(hip, oracle, d, ha, hb, a, np.ascontiguousarray(bw[:, 8:2048]), "skinny ragged K")
        assert hip.last_path().startswith("gemm_skinny_mfma" if d is dt.float16 else "gemm_skinny")
    # an Inf in B next to the K tail must not leak through zero padding
    a = encode(rng.standard_normal((4, 300)) * 0.5, dt.bfloat16, oracle)
    b = encode(rng.standard_normal((300, 1024)) * 0.5, dt.bfloat16, oracle)
    b[299, 5] = 0x7F80  # +inf in bf16 storage
    ha, hb = pair(a, dt.bfloat16, hip, oracle)[0], pair(b, dt.bfloat16, hip, oracle)[0]
    got = decode(logical(hip.matmul(ha, hb)), dt.bfloat16, oracle)
    assert hip.last_path().startswith("gemm_skinny_mfma")
    assert np.all(np.isinf(got[:, 5]) | np.isnan(got[:, 5])) and np.all(np.isfinite(np.delete(got, 5, axis=1)))


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float16], ids=lambda d: d.name)
@pytest.mark.parametrize("m,k,n", [(8, 1024, 16384), (1, 520, 16392), (16, 4096, 16384), (13, 768, 17000)],
                         ids=lambda v: str(v))
def test_matmul_skinny_wide_output(hip, oracle, d, m, k, n):
    """Decode-like products whose N alone fills the chip: K is split over the eight waves of a block
    and folded in LDS (one launch, no partials in memory). Ragged K (a multiple of 8, not of the
    waves' 32-row steps), N ending inside a block's 64 columns, m = 1 and m = 16."""
    rng = np.random.default_rng(m + k + n + d.tag)
    a = encode(rng.standard_normal((m, k)) * 0.5, d, oracle)
    b = encode(rng.standard_normal((k, n)) * 0.5, d, oracle)
    ha, hb = pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0]
    check(hip, oracle, d, ha, hb, a, b, f"skinny wide m={m} k={k} n={n}")
    assert hip.last_path() == "gemm_skinny_mfma_k8"
    # the same product twice: the fold order is fixed, so the bits repeat
    assert np.array_equal(logical(hip.matmul(ha, hb)), logical(hip.matmul(ha, hb)))


@pytest.mark.parametrize("m,k,n", [(8, 1024, 16384), (1, 515, 16388), (16, 4096, 16384), (13, 770, 17000)],
                         ids=lambda v: str(v))
def test_matmul_skinny_wide_output_f32(hip, oracle, m, k, n):
    """The float32 form: B rows go from registers straight into v_mfma_f32_16x16x4_f32, the eight
    waves of a block split K. Ragged K (not a multiple of the 4-row steps), N ending inside a
    block's 64 columns, a transposed A (its elements are read one by one)."""
    rng = np.random.default_rng(m + k + n)
    d = dt.float32
    a = encode(rng.standard_normal((m, k)) * 0.5, d, oracle)
    b = encode(rng.standard_normal((k, n)) * 0.5, d, oracle)
    ha, hb = pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0]
    check(hip, oracle, d, ha, hb, a, b, f"skinny wide f32 m={m} k={k} n={n}")
    assert hip.last_path() == "gemm_skinny_f32_k8"
    assert np.array_equal(logical(hip.matmul(ha, hb)), logical(hip.matmul(ha, hb)))
    at = np.ascontiguousarray(a.T)
    hat = pair(at, d, hip, oracle, lambda B, t: B.permute(t, (1, 0)))[0]
    same = logical(hip.matmul(hat, hb))
    assert hip.last_path() == "gemm_skinny_f32_k8"
    assert np.array_equal(same, logical(hip.matmul(ha, hb)))


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float16, dt.float32], ids=lambda d: d.name)
def test_matmul_big_tile_kernel(hip, oracle, d):
    """The LDS-tiled kernel family: every block shape, whole and ragged tiles,
    all four operand orientations, batched and batch-broadcast."""
    rng = np.random.default_rng(1400 + d.tag)
    # (blocks of 128 x 128 up to half the compute units become 128 x 64, and for f32 64 x 64; one
    # f32 product with a long K is cut along K on top of that)
    small = "gemm_tile_64x64" if d is dt.float32 else "gemm_tile_128x64"
    cases = [
        # whole tiles
        (256, 64, 256, small), (512, 192, 768, small),
        (768, 320, 256, small), (512, 128, 64, small),
        (2048, 64, 2048, "gemm_tile_128x128"), (65536, 64, 64, "gemm_tile_256x64"),
        (4096, 64, 4096, "gemm_tile_256x256"),
        # ragged in M and N (multiples of 8, so M/N-contiguous operands qualify too)
        (200, 64, 136, small), (264, 128, 40, small),
        (2040, 64, 2040, "gemm_tile_128x128"), (65528, 128, 40, "gemm_tile_256x64"),
        (4000, 64, 4088, "gemm_tile_256x256"),
    ]
    for (m, k, n, path) in cases:
        a = encode(rng.standard_normal((m, k)), d, oracle)
        b = encode(rng.standard_normal((k, n)), d, oracle)
        for ta in (False, True):
            for tb in (False, True):
                if m * n > 4_000_000 and (ta, tb) not in ((False, False), (True, True)):
                    continue  # keep the float64 reference products of the large cases to two
                ha, _ = pair(np.ascontiguousarray(a.T) if ta else a, d, hip, oracle,
                             (lambda B, t: B.permute(t, (1, 0))) if ta else None)
                hb, _ = pair(np.ascontiguousarray(b.T) if tb else b, d, hip, oracle,
                             (lambda B, t: B.permute(t, (1, 0))) if tb else None)
                check(hip, oracle, d, ha, hb, a, b, f"tile {m}x{k}x{n} ta={ta} tb={tb}")
                # whole 256-tiles of 16-bit operands take the direct-to-LDS form
                want_path = "gemm_dl_256x256" if (path, m % 256, n % 256) == ("gemm_tile_256x256", 0, 0) and d is not dt.float32 else path
                assert hip.last_path() == want_path, (m, k, n, ta, tb, hip.last_path())
    # odd M and N: only K-contiguous operands (A row-major, B given as its transpose) qualify
    a = encode(rng.standard_normal((203, 128)), d, oracle)
    b = encode(rng.standard_normal((128, 157)), d, oracle)
    hb, _ = pair(np.ascontiguousarray(b.T), d, hip, oracle, lambda B, t: B.permute(t, (1, 0)))
    check(hip, oracle, d, pair(a, d, hip, oracle)[0], hb, a, b, "tile odd edges")
    assert hip.last_path() == small
    check(hip, oracle, d, pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0], a, b, "odd N, row-major B")
    assert hip.last_path() == "gemm_mfma"
    # odd N on every block shape: the rows of C start at every 2-byte alignment, and 16-bit
    # results leave as 16-byte stores at the aligned addresses plus single elements at the ends
    for (m, k, n, path) in [(4000, 64, 4087, "gemm_tile_256x256"), (264, 128, 57, small),
                            (203, 192, 1031, small), (131, 64, 9, small),
                            (2041, 64, 2039, "gemm_tile_128x128"), (65529, 64, 57, "gemm_tile_256x64")]:
        a = encode(rng.standard_normal((m, k)), d, oracle)
        b = encode(rng.standard_normal((k, n)), d, oracle)
        hb, _ = pair(np.ascontiguousarray(b.T), d, hip, oracle, lambda B, t: B.permute(t, (1, 0)))
        check(hip, oracle, d, pair(a, d, hip, oracle)[0], hb, a, b, f"odd N {m}x{k}x{n}")
        assert hip.last_path() == path, (m, k, n, hip.last_path())
    a = encode(rng.standard_normal((3, 2, 256, 128)), d, oracle)
    b = encode(rng.standard_normal((128, 512)), d, oracle)
    check(hip, oracle, d, pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0], a, b, "big batched x broadcast W")
    assert hip.last_path().startswith("gemm_tile")
    b4 = encode(rng.standard_normal((3, 1, 128, 256)), d, oracle)
    check(hip, oracle, d, pair(a, d, hip, oracle)[0], pair(b4, d, hip, oracle)[0], a, b4, "big batch broadcast")
    # a sliced (offset, larger row stride) operand still qualifies when rows stay 16-byte aligned
    wide = encode(rng.standard_normal((256, 256 + 64)), d, oracle)
    hw, _ = pair(wide, d, hip, oracle, lambda B, t: B.shrink(t, [(0, 256), (32, 288)]))
    hb2, _ = pair(b4[0, 0][:, :256].copy(), d, hip, oracle)
    check(hip, oracle, d, hip.shrink(hw, [(0, 256), (0, 128)]), hb2, wide[:, 32:160], b4[0, 0][:, :256], "big sliced A")


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_matmul_padded_copies(hip, oracle, d):
    """Large products whose operands are not whole 16-byte vectors of whole K-slabs (the
    [C k k, 14 x 14] matrices of unfolded windows, their transposes, a ragged K) run the
    tiled kernels over zero-padded copies; the inputs are left as they were."""
    rng = np.random.default_rng(1450 + d.tag)
    # weights broadcast over a batch of window matrices: [co, ckk] x [n, ckk, L]
    for (n, co, ckk, L) in [(8, 256, 576, 196), (32, 128, 1152, 49)]:
        w = encode(rng.standard_normal((1, co, ckk)), d, oracle)
        cols = encode(rng.standard_normal((n, ckk, L)), d, oracle)
        hw, _ = pair(w, d, hip, oracle, lambda B, t: B.expand(t, (n, co, ckk)))
        hc, oc = pair(cols, d, hip, oracle)
        check(hip, oracle, d, hw, hc, np.broadcast_to(w, (n, co, ckk)), cols, f"conv {co}x{ckk}x{L}")
        # (rows of 196 floats are whole vectors already)
        vec_rows = d is dt.float32 and L % 4 == 0
        assert hip.last_path() == ("gemm_tile_64x64" if vec_rows else "gemm_tile_padded"), hip.last_path()
        same_bits(logical(hc), cols, "input untouched")
        # the weight gradient's shape: K is the ragged dim of both operands
        dy = encode(rng.standard_normal((n, co, L)), d, oracle)
        hd = pair(dy, d, hip, oracle)[0]
        hct = pair(cols, d, hip, oracle, lambda B, t: B.permute(t, (0, 2, 1)))[0]
        check(hip, oracle, d, hd, hct, dy, np.swapaxes(cols, 1, 2), f"ragged K {co}x{L}x{ckk}")
        assert hip.last_path() == "gemm_tile_padded", hip.last_path()
        # the input gradient's shape: A is the transposed weight (contiguous along M)
        hwt = pair(w[0], d, hip, oracle, lambda B, t: B.permute(t, (1, 0)))[0]
        check(hip, oracle, d, hwt, hd, w[0].T, dy, f"transposed A {ckk}x{co}x{L}")
        assert hip.last_path() == ("gemm_tile_128x64" if vec_rows else "gemm_tile_padded"), hip.last_path()
    # an odd row pitch of a k-contiguous A and an odd M of an M-contiguous A
    a = encode(rng.standard_normal((515, 517)), d, oracle)
    b = encode(rng.standard_normal((512, 519)), d, oracle)
    ha = pair(a, d, hip, oracle, lambda B, t: B.shrink(t, [(0, 515), (1, 513)]))[0]
    check(hip, oracle, d, ha, pair(b, d, hip, oracle)[0], a[:, 1:513], b, "odd pitches")
    assert hip.last_path() == "gemm_tile_padded", hip.last_path()
    at = np.ascontiguousarray(a[:, 1:513].T)
    hat = pair(at, d, hip, oracle, lambda B, t: B.permute(t, (1, 0)))[0]
    check(hip, oracle, d, hat, pair(b, d, hip, oracle)[0], a[:, 1:513], b, "odd M, M-contiguous A")
    assert hip.last_path() == "gemm_tile_padded", hip.last_path()
    # a NaN or an infinity next to the padding stays where it is and reaches no other element
    a = encode(rng.standard_normal((256, 196)), d, oracle)
    b = encode(rng.standard_normal((196, 3000)), d, oracle)
    af, bf_ = decode(a, d, oracle).copy(), decode(b, d, oracle).copy()
    af[7, 195] = np.inf
    bf_[195, 2999] = np.nan
    a, b = encode(af, d, oracle), encode(bf_, d, oracle)
    got = decode(logical(hip.matmul(pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0])), d, oracle)
    assert hip.last_path() == "gemm_tile_padded", hip.last_path()
    want = ref_f64(a, b, d, oracle)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want))


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.float16, dt.float64], ids=lambda d: d.name)
def test_matmul_seeded_shape_sweep(hip, oracle, d):
    """Eighty seeded shapes per dtype across the dispatch's thresholds (block shapes, the cut along
    K, padded copies, the general kernel): extents drawn around multiples of the tile sizes, every
    orientation, with and without a batch, against the float64 product of the stored values."""
    rng = np.random.default_rng(4200 + d.tag)
    T = lambda B, t: B.permute(t, tuple(range(len(t.shape) - 2)) + (len(t.shape) - 1, len(t.shape) - 2))  # noqa: E731
    seen = set()
    for case in range(80):
        def extent(bases):
            return max(1, int(rng.choice(bases)) + int(rng.integers(-9, 10)) * int(rng.integers(0, 4) == 0))
        m = extent([8, 64, 128, 200, 256, 512, 1024, 2048])
        n = extent([8, 64, 128, 196, 256, 768, 1536, 2048])
        k = extent([32, 64, 128, 256, 576, 2048])
        batch = () if rng.integers(0, 2) else (int(rng.integers(1, 5)),)
        if m * n * k * int(np.prod(batch, dtype=np.int64)) > 1e9:
            k = max(32, k // 8)
        ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        share_b = bool(batch) and bool(rng.integers(0, 2))  # one B for the whole batch
        a = encode(rng.standard_normal(batch + (m, k)), d, oracle)
        b = encode(rng.standard_normal((() if share_b else batch) + (k, n)), d, oracle)
        ha, _ = pair(np.ascontiguousarray(np.swapaxes(a, -1, -2)) if ta else a, d, hip, oracle, T if ta else None)
        hb, _ = pair(np.ascontiguousarray(np.swapaxes(b, -1, -2)) if tb else b, d, hip, oracle, T if tb else None)
        check(hip, oracle, d, ha, hb, a, b, f"case {case}: {batch} {m}x{k}x{n} ta={ta} tb={tb} shared B={share_b}")
        seen.add(hip.last_path())
    # the sweep is only worth its time if it crosses the dispatch: at least three kernels per dtype
    assert len(seen) >= 3, seen


def test_matmul_f64_matrix_kernel(hip, oracle):
    """float64 on the f64 matrix instruction: the three block shapes, every orientation, ragged M / N / K,
    batches with a broadcast operand, operands with no unit stride; products of doubles summed in
    double, so 1e-9 of the float64 reference is loose by orders of magnitude."""
    d = dt.float64
    rng = np.random.default_rng(1470)
    T = lambda B, t: B.permute(t, (1, 0))  # noqa: E731
    for (m, k, n, path) in [(512, 300, 700, "gemm_f64_32x32"), (1024, 40, 1024, "gemm_f64_64x64"),
                            (1000, 100, 1001, "gemm_f64_64x64"), (2048, 64, 2048, "gemm_f64_128x128"),
                            (2041, 37, 2039, "gemm_f64_128x128"), (1, 5, 1, "gemm_f64_32x32"), (130, 1, 3, "gemm_f64_32x32")]:
        a = rng.standard_normal((m, k))
        b = rng.standard_normal((k, n))
        for ta in (False, True):
            for tb in (False, True):
                ha, _ = pair(np.ascontiguousarray(a.T) if ta else a, d, hip, oracle, T if ta else None)
                hb, _ = pair(np.ascontiguousarray(b.T) if tb else b, d, hip, oracle, T if tb else None)
                got = logical(hip.matmul(ha, hb))
                assert hip.last_path() == path, (m, k, n, hip.last_path())
                want = a @ b
                assert np.all(np.abs(got - want) <= 1e-12 * (np.abs(want) + np.sqrt(k))), (m, k, n, ta, tb)
    a = rng.standard_normal((3, 1, 70, 50))
    b = rng.standard_normal((1, 4, 50, 90))
    got = logical(hip.matmul(pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0]))
    assert hip.last_path() == "gemm_f64_32x32" and np.allclose(got, a @ b, rtol=1e-12, atol=1e-12)
    # every other row and column of both operands: no unit stride anywhere
    a = rng.standard_normal((200, 160))
    b = rng.standard_normal((160, 120))
    every_other = lambda B, t: B.shrink(B.reshape(t, (t.shape[0] // 2, 2, t.shape[1] // 2, 2)),  # noqa: E731
                                        [(0, t.shape[0] // 2), (0, 1), (0, t.shape[1] // 2), (0, 1)])
    ha = pair(a, d, hip, oracle, every_other)[0]
    hb = pair(b, d, hip, oracle, every_other)[0]
    ha, hb = hip.reshape(ha, (100, 80)), hip.reshape(hb, (80, 60))
    got = logical(hip.matmul(ha, hb))
    assert hip.last_path() == "gemm_f64_32x32" and np.allclose(got, a[::2, ::2] @ b[::2, ::2], rtol=1e-12, atol=1e-12)
    # flipped operands (negative strides)
    fl = lambda B, t: B.flip(t, (True, True))  # noqa: E731
    got = logical(hip.matmul(pair(a, d, hip, oracle, fl)[0], pair(b, d, hip, oracle, fl)[0]))
    assert hip.last_path() == "gemm_f64_32x32" and np.allclose(got, a[::-1, ::-1] @ b[::-1, ::-1], rtol=1e-12, atol=1e-12)
    # k == 0 stores zeros
    z = logical(hip.matmul(hip.buffer(d, (70, 0)), hip.buffer(d, (0, 40))))
    assert z.shape == (70, 40) and not z.any()
    # non-finite values stay where the arithmetic puts them
    a = rng.standard_normal((64, 33))
    b = rng.standard_normal((33, 64))
    a[3, 32] = np.inf
    b[32, 63] = np.nan
    got = logical(hip.matmul(pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0]))
    with np.errstate(invalid="ignore"):
        want = a @ b
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(np.isinf(got), np.isinf(want))


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_matmul_few_blocks_cut_along_k(hip, oracle, d):
    """One product with few output blocks and a long K (a weight gradient) is cut along K; the f32
    partial sums are added in a fixed order and rounded once: within the matmul tolerance, and the
    same bits every call."""
    rng = np.random.default_rng(1460 + d.tag)
    T = lambda B, t: B.permute(t, (1, 0))  # noqa: E731
    f32 = d is dt.float32
    cut = "gemm_tile_64x64_splitk" if f32 else "gemm_tile_128x64_splitk"
    for (m, k, n, path) in [(128, 4096, 64, cut), (256, 2048, 256, cut), (200, 1024, 72, cut if f32 else "gemm_tile_128x64"),
                            (768, 8192, 768, "gemm_tile_64x64" if f32 else cut),
                            (64, 128, 64, "gemm_tile_64x64" if f32 else "gemm_tile_128x64")]:
        a = encode(rng.standard_normal((m, k)), d, oracle)
        b = encode(rng.standard_normal((k, n)), d, oracle)
        for ta in (False, True):
            for tb in (False, True):
                ha, _ = pair(np.ascontiguousarray(a.T) if ta else a, d, hip, oracle, T if ta else None)
                hb, _ = pair(np.ascontiguousarray(b.T) if tb else b, d, hip, oracle, T if tb else None)
                check(hip, oracle, d, ha, hb, a, b, f"{m}x{k}x{n} ta={ta} tb={tb}")
                assert hip.last_path() == path, (m, k, n, ta, tb, hip.last_path())
                first = logical(hip.matmul(ha, hb))
                same_bits(logical(hip.matmul(ha, hb)), first, "same bits on every call")
                if not f32:  # one rounding of the f32 sum: within one unit of the f64 product rounded
                    got, want = decode(first, d, oracle), ref_f64(a, b, d, oracle)
                    ulp = 2.0 ** (-8 if d is dt.bfloat16 else -11)
                    assert np.all(np.abs(got - want) <= ulp * 2 * np.abs(want) + np.sqrt(k) * 4e-6), (m, k, n, ta, tb)
    # into a strided output: a column slice of a wider result
    a = encode(rng.standard_normal((128, 2048)), d, oracle)
    b = encode(rng.standard_normal((2048, 64)), d, oracle)
    ha, hb = pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0]
    dense = logical(hip.matmul(ha, hb))
    wide = hip.reshape(hip.from_host(np.zeros(128 * 80, dense.dtype), d), (128, 80))
    import ctypes as C
    view = hip.shrink(wide, [(0, 128), (8, 72)])
    hip._check(hip._lib.nxh_matmul(hip._h, C.byref(view._desc()), C.byref(ha._desc()), C.byref(hb._desc())))
    assert hip.last_path() == cut
    w = logical(wide)
    same_bits(np.ascontiguousarray(w[:, 8:72]), dense, "strided output")
    assert not w[:, :8].any() and not w[:, 72:].any()


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_matmul_streamed_weights_cut_along_k(hip, oracle, d):
    """A decode step of 8 to 128 sequences against a weight matrix of 16 MiB or more with fewer
    128-column blocks than compute units: 128 x 128 blocks cut along K, f32 partial sums added in a
    fixed order. Both layouts of the weights ([K, N] and the transposed view of [N, K])."""
    rng = np.random.default_rng(1480 + d.tag)
    T = lambda B, t: B.permute(t, (1, 0))  # noqa: E731
    for (m, k, n) in [(32, 4096, 4096), (8, 2048, 8192), (100, 4096, 2176)]:
        a = encode(rng.standard_normal((m, k)), d, oracle)
        b = encode(rng.standard_normal((k, n)) * 0.1, d, oracle)
        want = ref_f64(a, b, d, oracle)
        ha = pair(a, d, hip, oracle)[0]
        for tb in (False, True):
            hb = pair(np.ascontiguousarray(b.T) if tb else b, d, hip, oracle, T if tb else None)[0]
            first = logical(hip.matmul(ha, hb))
            assert hip.last_path() == "gemm_tile_128x128_splitk", (m, k, n, tb, hip.last_path())
            got = decode(first, d, oracle)
            ulp = 2.0 ** (-8 if d is dt.bfloat16 else -11)
            assert np.all(np.abs(got - want) <= ulp * 2 * np.abs(want) + np.sqrt(k) * 4e-6), (m, k, n, tb)
            same_bits(logical(hip.matmul(ha, hb)), first, "same bits on every call")
    # below 16 MiB of weights the strips keep the call
    a = encode(rng.standard_normal((8, 1024)), d, oracle)
    b = encode(rng.standard_normal((1024, 4096)), d, oracle)
    check(hip, oracle, d, pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0], a, b, "small weights")
    assert hip.last_path().startswith("gemm_skinny"), hip.last_path()
    # a short K leaves nothing to cut (576 = nine slabs): 16 rows stay on the strips instead of
    # filling one eighth of a whole-K 128-row tile
    a = encode(rng.standard_normal((16, 576)), d, oracle)
    b = encode(rng.standard_normal((576, 16000)) * 0.1, d, oracle)
    check(hip, oracle, d, pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0], a, b, "short K")
    assert hip.last_path().startswith("gemm_skinny_mfma"), hip.last_path()


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_matmul_direct_to_lds_kernel(hip, oracle, d):
    """The large-product form (operands straight from global memory into swizzled LDS
    tiles, 16x16x32 MFMA): every operand orientation, one to seven K-slabs, batches
    with a broadcast operand, a sliced operand with a larger row stride."""
    rng = np.random.default_rng(1500 + d.tag)
    T = lambda B, t: B.permute(t, (1, 0))  # noqa: E731
    for k in (64, 128, 192, 448):
        a = encode(rng.standard_normal((4096, k)), d, oracle)
        b = encode(rng.standard_normal((k, 4096)), d, oracle)
        want = ref_f64(a, b, d, oracle)
        for ta in (False, True):
            for tb in (False, True):
                if k != 192 and ta != tb:
                    continue
                ha, _ = pair(np.ascontiguousarray(a.T) if ta else a, d, hip, oracle, T if ta else None)
                hb, _ = pair(np.ascontiguousarray(b.T) if tb else b, d, hip, oracle, T if tb else None)
                got = decode(logical(hip.matmul(ha, hb)), d, oracle)
                assert hip.last_path() == "gemm_dl_256x256", (k, ta, tb, hip.last_path())
                lim = MM_TOL[d.name] * (np.abs(want) + np.sqrt(k))
                assert np.all(np.abs(got - want) <= lim), (k, ta, tb, float(np.abs(got - want).max()))
                # a 16-bit result is the f32 sum rounded once: within one unit of the f64 product rounded
                ulp = 2.0 ** (-8 if d is dt.bfloat16 else -11)
                assert np.all(np.abs(got - want) <= ulp * 2 * np.abs(want) + np.sqrt(k) * 2e-6), (k, ta, tb)
    # batches: [4, 2048, 128] x [128, 2048] (one B for all), [4,1,..] x [1,2,..] (both broadcast)
    a = encode(rng.standard_normal((4, 2048, 128)), d, oracle)
    b = encode(rng.standard_normal((128, 2048)), d, oracle)
    check(hip, oracle, d, pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0], a, b, "dl batched x one B")
    assert hip.last_path() == "gemm_dl_256x256"
    a4 = encode(rng.standard_normal((4, 1, 1024, 64)), d, oracle)
    b4 = encode(rng.standard_normal((1, 4, 64, 1024)), d, oracle)
    check(hip, oracle, d, pair(a4, d, hip, oracle)[0], pair(b4, d, hip, oracle)[0], a4, b4, "dl both batch-broadcast")
    assert hip.last_path() == "gemm_dl_256x256"
    # a column slice of a wider matrix (row stride 4096 + 64, offset 32 elements: still 16-byte aligned)
    wide = encode(rng.standard_normal((4096, 128 + 64)), d, oracle)
    hw, _ = pair(wide, d, hip, oracle, lambda B, t: B.shrink(t, [(0, 4096), (32, 160)]))
    b = encode(rng.standard_normal((128, 4096)), d, oracle)
    check(hip, oracle, d, hw, pair(b, d, hip, oracle)[0], wide[:, 32:160], b, "dl sliced A")
    assert hip.last_path() == "gemm_dl_256x256"


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_matmul_and_linear_on_128x192_blocks(hip, oracle, d):
    """The 128 x 192 direct-to-LDS shape (N = 768-like widths): both orientations of B, one to
    fifty K-slabs, batches; then the fused linear on it (bias, residual, both, tanh GELU), bit for
    bit the sequence of primitives, whose matmul takes the same kernel."""
    rng = np.random.default_rng(1700 + d.tag)
    T = lambda B, t: B.permute(t, (1, 0))  # noqa: E731
    for m, k, n in ((3072, 64, 768), (3072, 192, 768), (8448, 448, 192), (5632, 3200, 384)):
        a = encode(rng.standard_normal((m, k)) * 0.5, d, oracle)
        b = encode(rng.standard_normal((k, n)) * 0.5, d, oracle)
        want = ref_f64(a, b, d, oracle)
        ha, _ = pair(a, d, hip, oracle)
        for tb in (False, True):
            hb, _ = pair(np.ascontiguousarray(b.T) if tb else b, d, hip, oracle, T if tb else None)
            got = decode(logical(hip.matmul(ha, hb)), d, oracle)
            assert hip.last_path() == "gemm_dl_128x192", (m, k, n, tb, hip.last_path())
            ulp = 2.0 ** (-8 if d is dt.bfloat16 else -11)
            assert np.all(np.abs(got - want) <= ulp * 2 * np.abs(want) + np.sqrt(k) * 2e-6), (m, k, n, tb, float(np.abs(got - want).max()))
    a = encode(rng.standard_normal((3, 2304, 128)), d, oracle)
    b = encode(rng.standard_normal((128, 576)), d, oracle)
    check(hip, oracle, d, pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0], a, b, "128x192 batched x one B")
    assert hip.last_path() == "gemm_dl_128x192"
    a4 = encode(rng.standard_normal((2, 1, 1536, 64)), d, oracle)
    b4 = encode(rng.standard_normal((1, 3, 64, 768)), d, oracle)
    check(hip, oracle, d, pair(a4, d, hip, oracle)[0], pair(b4, d, hip, oracle)[0], a4, b4, "128x192 both batch-broadcast")
    assert hip.last_path() == "gemm_dl_128x192"
    # the fused linear
    for xs, ws in (((4, 1152, 256), (256, 768)), ((8448, 1024), (1024, 192))):
        x = encode(rng.standard_normal(xs) * 0.5, d, oracle)
        w = encode(rng.standard_normal(ws) * 0.1, d, oracle)
        bias = encode(rng.standard_normal(ws[-1]), d, oracle)
        r = encode(rng.standard_normal(xs[:-1] + (ws[-1],)), d, oracle)
        hx, hw, hb, hr = (pair(v, d, hip, oracle)[0] for v in (x, w, bias, r))
        bshape = (1,) * (len(xs) - 1) + (ws[-1],)
        for use_b, use_r in ((True, True), (True, False), (False, True)):
            got = logical(hip.linear(hx, hw, hb if use_b else None, hr if use_r else None))
            assert hip.last_path() == "linear_dl_128x192", hip.last_path()
            y = hip.matmul(hx, hw)
            assert hip.last_path() == "gemm_dl_128x192"
            if use_b:
                y = hip.binary("add", y, hip.expand(hip.reshape(hb, bshape), y.shape))
            if use_r:
                y = hip.binary("add", hr, y)
            same_bits(got, logical(y), f"{d.name} {xs}x{ws} bias={use_b} residual={use_r}")
        # a residual that is a column slice of a wider tensor, the weight given transposed
        wide = encode(rng.standard_normal(xs[:-1] + (ws[-1] + 8,)), d, oracle)
        hwide = hip.shrink(pair(wide, d, hip, oracle)[0], [(0, s) for s in xs[:-1]] + [(8, ws[-1] + 8)])
        hwt = hip.permute(pair(np.ascontiguousarray(np.swapaxes(w, 0, 1)), d, hip, oracle)[0], (1, 0))
        got = logical(hip.linear(hx, hwt, hb, hwide))
        assert hip.last_path() == "linear_dl_128x192", hip.last_path()
        y = hip.binary("add", hip.matmul(hx, hwt), hip.expand(hip.reshape(hb, bshape), got.shape))
        same_bits(got, logical(hip.binary("add", hwide, y)), f"{d.name} strided residual, transposed weight")
        # the tanh GELU in the epilogue against the fused linear followed by the GELU kernel
        got = logical(hip.linear_gelu_tanh(hx, hw, hb))
        assert hip.last_path() == "linear_dl_128x192", hip.last_path()
        same_bits(got, logical(hip.gelu_tanh(hip.linear(hx, hw, hb))), f"{d.name} linear + gelu")


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float16, dt.float32], ids=lambda d: d.name)
def test_linear_epilogue_equals_the_sequence(hip, oracle, d):
    """nxh_linear = matmul, + bias, + residual with the primitives' rounding
    points: bit-identical to the three GPU calls, and within the matmul
    tolerance of the oracle's sequence."""
    rng = np.random.default_rng(900 + d.tag)
    for xs, ws in (((8, 128, 768), (768, 768)), ((4, 100, 256), (256, 200)), ((512, 128), (128, 1024)),
                   ((2, 3, 64, 64), (64, 72))):
        x = encode(rng.standard_normal(xs) * 0.5, d, oracle)
        w = encode(rng.standard_normal(ws) * 0.1, d, oracle)
        b = encode(rng.standard_normal(ws[-1]), d, oracle)
        r = encode(rng.standard_normal(xs[:-1] + (ws[-1],)), d, oracle)
        (hx, ox), (hw, ow), (hb, ob), (hr, orr) = (pair(a, d, hip, oracle) for a in (x, w, b, r))
        bshape = (1,) * (len(xs) - 1) + (ws[-1],)

        def sequence(B, tx, tw, tb, tr):
            y = B.matmul(tx, tw)
            if tb is not None:
                y = B.binary("add", y, B.expand(B.reshape(tb, bshape), y.shape))
            if tr is not None:
                y = B.binary("add", tr, y)
            return y

        for use_b, use_r in ((True, True), (True, False), (False, True)):
            got = logical(hip.linear(hx, hw, hb if use_b else None, hr if use_r else None))
            assert hip.last_path().startswith(("linear_tile", "linear_dl")), hip.last_path()
            want_gpu = logical(sequence(hip, hx, hw, hb if use_b else None, hr if use_r else None))
            same_bits(got, want_gpu, f"{d.name} {xs}x{ws} bias={use_b} residual={use_r}")
            want_cpu = logical(sequence(oracle, ox, ow, ob if use_b else None, orr if use_r else None))
            k = xs[-1]
            close(got, want_cpu, d, oracle, TOL[d.name][0], TOL[d.name][0] * (1 + k ** 0.5 * 0.05), f"{d.name} vs oracle")
        # a strided residual (a column slice of a wider tensor) and the weight given transposed
        wide = encode(rng.standard_normal(xs[:-1] + (ws[-1] + 8,)), d, oracle)
        hwide = hip.shrink(pair(wide, d, hip, oracle)[0], [(0, s) for s in xs[:-1]] + [(8, ws[-1] + 8)])
        hwt = hip.permute(pair(np.ascontiguousarray(np.swapaxes(w, 0, 1)), d, hip, oracle)[0], (1, 0))
        got = logical(hip.linear(hx, hwt, hb, hwide))
        want = logical(sequence(hip, hx, hwt, hb, hwide))
        same_bits(got, want, f"{d.name} strided residual")
    with pytest.raises(RuntimeError, match="tiled GEMM"):
        hip.linear(hip.full(d, (4, 30), 1.0), hip.full(d, (30, 8), 1.0), hip.full(d, (8,), 1.0))
    with pytest.raises(ValueError):
        hip.linear(hip.full(d, (64, 64), 1.0), hip.full(d, (64, 64), 1.0), hip.full(d, (32,), 1.0))
    with pytest.raises(RuntimeError):
        hip.linear(hip.full(dt.int32, (64, 64), 1), hip.full(dt.int32, (64, 64), 1), hip.full(dt.int32, (64,), 1))


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_matmul_wide_product_with_a_ragged_last_column_block(hip, oracle, d):
    """N = 16 x 256 + 81 (the shape class of GPT-2's tied head, [8192,768] x [768,50257]): the whole
    256-column blocks go through the direct-to-LDS kernel, whose stores take C's odd row pitch as
    it is, the last 81 columns through a launch of their own. Both layouts of B; every element is
    one k-ordered f32 sum rounded once, so the bits equal the unsplit kernels' bits on each side."""
    rng = np.random.default_rng(1700 + d.tag)
    T = lambda B, t: B.permute(t, (1, 0))  # noqa: E731
    m, k, n = 4096, 192, 16 * 256 + 81
    a = encode(rng.standard_normal((m, k)), d, oracle)
    b = encode(rng.standard_normal((k, n)), d, oracle)
    want = ref_f64(a, b, d, oracle)
    ha = pair(a, d, hip, oracle)[0]
    for tb in (False, True):
        if not tb and n % 8:
            continue  # rows of an N-contiguous B must be whole 16-byte vectors for the tiled kernels
        hb = pair(np.ascontiguousarray(b.T) if tb else b, d, hip, oracle, T if tb else None)[0]
        got_bits = logical(hip.matmul(ha, hb))
        assert hip.last_path() == "gemm_dl_256x256", hip.last_path()
        got = decode(got_bits, d, oracle)
        ulp = 2.0 ** (-8 if d is dt.bfloat16 else -11)
        assert np.all(np.abs(got - want) <= ulp * 2 * np.abs(want) + np.sqrt(k) * 2e-6), float(np.abs(got - want).max())
        # the left part against the same columns computed alone (aligned C, no split)
        left = hip.matmul(ha, hip.shrink(hb, [(0, k), (0, 16 * 256)]))
        same_bits(got_bits[:, :16 * 256], logical(left), "whole blocks: the same bits as the product of those columns alone")


def test_linear_gelu_by_table_for_every_bfloat16_input(hip):
    """The bfloat16 linear + GELU epilogue looks its results up in a table held in LDS. A zero
    product plus a bias that runs through all 65 536 bit patterns (NaNs with their payloads,
    infinities, subnormals, the last finite binade included) must give, in every row, the bits
    of the arithmetic GELU kernel on that bias; the same for other constants (another table)
    and inside a captured graph."""
    n = 342 * 192  # whole 128 x 192 blocks, >= 65 536
    pats = np.arange(n, dtype=np.uint32).astype(np.uint16)  # (wraps: the first 128 patterns twice)
    x = hip.reshape(hip.from_host(np.zeros(128 * 64, np.uint16), dt.bfloat16), (128, 64))
    w = hip.reshape(hip.from_host(np.zeros(64 * n, np.uint16), dt.bfloat16), (64, n))
    b = hip.reshape(hip.from_host(pats, dt.bfloat16), (n,))
    pre = hip.linear(x, w, b)  # 0 + bias: the bias itself, -0 turned into +0
    row = hip.shrink(pre, [(0, 1), (0, n)])
    for consts in ((0.044715, 0.7978845608028654, 1.0, 0.5), (0.05, 0.75, 1.0, 0.5)):
        want = logical(hip.gelu_tanh(hip.contiguous(row), consts)).view(np.uint16)
        assert hip.last_path() == "gelu_tanh"  # the arithmetic kernel (a small tensor)
        got = logical(hip.linear_gelu_tanh(x, w, b, consts)).view(np.uint16)
        assert hip.last_path() == "linear_dl_128x192", hip.last_path()
        assert np.array_equal(got, np.broadcast_to(want, got.shape)), consts
    hip.capture_begin()
    try:
        out = hip.linear_gelu_tanh(x, w, b, (0.05, 0.75, 1.0, 0.5))
    finally:
        graph = hip.capture_end()
    for _ in range(2):
        graph.launch()
        hip.synchronize()
        assert np.array_equal(logical(out).view(np.uint16), np.broadcast_to(want, got.shape))
    graph.destroy()


@pytest.mark.parametrize("d", [dt.bfloat16, dt.float32, dt.int32], ids=lambda d: d.name)
def test_long_ragged_rows_get_whole_memory_lines(hip, oracle, d):
    """The binding gives a matmul result whose rows are long and no whole number of 128-byte
    lines a padded row pitch and returns the [..., n] view of it (the reference allocates
    C-contiguous, nx_backend.ml:485-500; GPT-2's tied head writes 50257 logits per token). The
    view has the product's values, reshapes where its dims merge, and feeds further calls."""
    rng = np.random.default_rng(1700 + d.tag)
    line = 128 // d.itemsize
    for (batch, m, k, n) in (((), 64, 64, 4099), ((2, 3), 16, 32, 4100), ((), 8, 128, 50257)):
        a = encode(rng.integers(-4, 5, batch + (m, k)).astype(np.float64), d, oracle)
        b = encode(rng.integers(-4, 5, (k, n)).astype(np.float64), d, oracle)
        (ha, oa), (hb, ob) = pair(a, d, hip, oracle), pair(b, d, hip, oracle)
        got = hip.matmul(ha, hb)
        pitch = (n + line - 1) // line * line
        assert tuple(got.shape) == batch + (m, n) and tuple(got.strides)[-2:] == (pitch, 1), (got.shape, got.strides)
        want = logical(oracle.matmul(oa, ob))
        same_bits(logical(got), want, f"{d.name} {batch} {m}x{k}x{n}")  # small integers: every sum is exact
        flat = hip.reshape(got, (int(np.prod(batch, dtype=np.int64)) * m, n))  # the leading dims merge: still a view
        same_bits(logical(flat), want.reshape(-1, n))
        same_bits(logical(hip.contiguous(got)), want)
        same_bits(logical(hip.reduce("max", [len(batch) + 1], got)), logical(oracle.reduce("max", [len(batch) + 1], oracle.matmul(oa, ob))))
    # whole lines, or short rows: the plain block
    for n in (4096, 4160, 1000):
        got = hip.matmul(hip.full(d, (4, 8), 1), hip.full(d, (8, n), 1))
        assert tuple(got.strides) == (n, 1)


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_matrix_times_vector(hip, oracle, d):
    """A matrix whose rows run along K times one to four columns takes a wave per row
    (gemm_rowdot): whole and ragged K, rows that are no whole vectors (element loads), a window of a
    wider matrix, two to four columns of a strided B, a batch with a shared vector, against the
    float64 product of the stored values."""
    rng = np.random.default_rng(5200 + d.tag)
    for m, k, n in ((4096, 4096, 1), (300, 1000, 1), (257, 67, 1), (512, 2051, 2), (1000, 768, 3), (256, 4096, 4)):
        a = encode(rng.standard_normal((m, k)), d, oracle)
        b = encode(rng.standard_normal((k, n)), d, oracle)
        ha, hb = pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0]
        check(hip, oracle, d, ha, hb, a, b, f"{m}x{k}x{n}")
        assert hip.last_path() == "gemm_rowdot", hip.last_path()
    # a window of a wider matrix (row pitch 1003, first column 1: no aligned pieces) and B as a column of a wider one
    wide = encode(rng.standard_normal((700, 1003)), d, oracle)
    bw = encode(rng.standard_normal((1000, 5)), d, oracle)
    ha = pair(wide, d, hip, oracle, lambda B, t: B.shrink(t, [(0, 700), (1, 1001)]))[0]
    hb = pair(bw, d, hip, oracle, lambda B, t: B.shrink(t, [(0, 1000), (2, 3)]))[0]
    check(hip, oracle, d, ha, hb, wide[:, 1:1001], bw[:, 2:3], "windows")
    assert hip.last_path() == "gemm_rowdot", hip.last_path()
    # a batch of matrices, one vector for all
    a = encode(rng.standard_normal((6, 128, 320)), d, oracle)
    v = encode(rng.standard_normal((320, 1)), d, oracle)
    check(hip, oracle, d, pair(a, d, hip, oracle)[0], pair(v, d, hip, oracle)[0], a, v, "batch, shared vector")
    assert hip.last_path() == "gemm_rowdot", hip.last_path()


@pytest.mark.parametrize("d", [dt.float32, dt.bfloat16, dt.float16], ids=lambda d: d.name)
def test_many_products_of_tiny_matrices(hip, oracle, d):
    """Batches of matrices of a few elements each take a lane per output over the whole batch
    (gemm_tiny): square and ragged shapes, a shared right operand, a batch of two dims, transposed
    operands, against the float64 product of the stored values."""
    rng = np.random.default_rng(5300 + d.tag)
    T = lambda B, t: B.permute(t, tuple(range(len(t.shape) - 2)) + (len(t.shape) - 1, len(t.shape) - 2))  # noqa: E731
    for batch, m, k, n in (((5000,), 4, 4, 4), ((300,), 3, 7, 5), ((16, 40), 2, 3, 2), ((1000,), 16, 16, 16), ((257,), 1, 64, 9)):
        a = encode(rng.standard_normal(batch + (m, k)), d, oracle)
        b = encode(rng.standard_normal(batch + (k, n)), d, oracle)
        check(hip, oracle, d, pair(a, d, hip, oracle)[0], pair(b, d, hip, oracle)[0], a, b, f"{batch} {m}x{k}x{n}")
        assert hip.last_path() == "gemm_tiny", hip.last_path()
        shared = encode(rng.standard_normal((k, n)), d, oracle)
        check(hip, oracle, d, pair(a, d, hip, oracle)[0], pair(shared, d, hip, oracle)[0], a, shared, "shared B")
        assert hip.last_path() == "gemm_tiny", hip.last_path()
        at = np.ascontiguousarray(np.swapaxes(a, -1, -2))
        check(hip, oracle, d, pair(at, d, hip, oracle, T)[0], pair(b, d, hip, oracle)[0], a, b, "transposed A")
        assert hip.last_path() == "gemm_tiny", hip.last_path()
