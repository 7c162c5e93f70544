"""GPU parity: fp32 GEMM family (fp32 MFMA) and bf16 projections (bf16 MFMA, fp32 accumulate)."""
import ctypes

import numpy as np
import pytest

from parity import BF16_TOL, assert_bits_equal, assert_close

pytestmark = pytest.mark.gpu
f32 = np.float32


def r(rng, *s, scale=1.0):
    return (rng.standard_normal(s) * scale).astype(f32)


SHAPES = [(1, 1, 1), (2, 2, 2), (5, 7, 3), (33, 65, 17), (64, 64, 64), (128, 16, 128), (130, 200, 70), (512, 128, 256),
          (257, 512, 129), (1024, 96, 1536)]


def test_matmul_reference_literal(hip):
    """tests/backend/cpu/ops_tests.cpp:36-46 and, through bf16, tests/backend/cuda/ops_tests.cu:85-103."""
    D, ops = hip.DeviceTensor, hip.ops
    a, b = D.fromHost(np.array([[1, 2], [3, 4]], f32)), D.fromHost(np.array([[5, 6], [7, 8]], f32))
    np.testing.assert_array_equal(ops.matmul(a, b).toHost().ravel(), [19, 22, 43, 50])
    np.testing.assert_array_equal(ops.matmulBf16(a, b).toHost().ravel(), [19, 22, 43, 50])
    with pytest.raises(ValueError):
        ops.matmul(D.zeros((2, 3)), D.zeros((2, 2)))
    with pytest.raises(ValueError):
        ops.matmulBf16(D.zeros((2, 3)), D.zeros((2, 2)))
    with pytest.raises(ValueError):
        ops.matmulBackward(D.zeros((2, 3)), D.zeros((3, 2)), D.zeros((2, 3)))


@pytest.mark.parametrize("m,k,n", SHAPES)
def test_fp32_gemm_family(hip, oracle, rng, m, k, n):
    D, ops = hip.DeviceTensor, hip.ops
    a, b, bt, g = r(rng, m, k), r(rng, k, n), r(rng, n, k), r(rng, m, n)
    da, db, dbt, dg = map(D.fromHost, (a, b, bt, g))
    assert_close(ops.matmul(da, db).toHost(), oracle.matmul(a, b), what="matmul")
    assert_close(ops.matmulTransposeB(da, dbt).toHost(), oracle.matmulTransposeB(a, bt), what="matmulTransposeB")
    for got, exp, nm in zip(ops.matmulBackward(da, db, dg), oracle.matmulBackward(a, b, g), ("dA", "dB")):
        assert_close(got.toHost(), exp, what="matmulBackward." + nm)
    for got, exp, nm in zip(ops.matmulTransposeBBackward(da, dbt, dg), oracle.matmulTransposeBBackward(a, bt, g), ("dA", "dB")):
        assert_close(got.toHost(), exp, what="matmulTransposeBBackward." + nm)
    bias = r(rng, n)
    assert_close(ops.linear(da, db, D.fromHost(bias)).toHost(), oracle.linear(a, b, bias), what="linear")


@pytest.mark.parametrize("m,k,n", [(1, 768, 768), (1, 3072, 768), (1, 768, 32003), (2, 72, 9000), (3, 520, 41), (5, 1032, 8200), (8, 768, 2304),
                                   (7, 8, 1), (1, 4100, 16), (4, 44, 300), (8, 30000, 64), (2, 1, 5)])
def test_fp32_products_of_a_few_rows(hip, oracle, rng, m, k, n):
    """matmul / linear (ops.hpp:14,30) with at most eight rows, the shape of a step of incremental decoding (model.cpp:169):
    served by a walk over the weights with the contraction cut into slices.  Widths that take 16-byte loads and widths that
    do not, one slice and many, rows of A too long for the walk's LDS (the tile kernels serve), adds in the store and after
    the slices are summed, accumulation in place."""
    D, ops, call = hip.DeviceTensor, hip.ops, hip.capi.call
    a, b, bias, res = r(rng, m, k), r(rng, k, n), r(rng, n), r(rng, m, n)
    da, db, dbias, dres = map(D.fromHost, (a, b, bias, res))
    expected = (a.astype(np.float64) @ b.astype(np.float64)).astype(f32)
    if m * k * n <= 5_000_000:
        assert_close(oracle.matmul(a, b), expected, tol=1e-5, what="oracle vs float64")
    product = ops.matmul(da, db)
    assert_close(product.toHost(), expected, tol=1e-5, what="few-row product")
    assert_bits_equal(ops.matmul(da, db).toHost(), product.toHost(), "the same product twice")
    out = D((m, n))
    call("bf_hip_gemm_f32_adds", 0, 0, da.ptr, db.ptr, dbias.ptr, dres.ptr, out.ptr, m, n, k, None)
    assert_bits_equal(out.toHost(), ops.addBiasResidual(product, dbias, dres).toHost(), "product + bias + residual")
    acc = D.fromHost(res)
    call("bf_hip_gemm_f32_adds", 0, 0, da.ptr, db.ptr, None, acc.ptr, acc.ptr, m, n, k, None)
    assert_bits_equal(acc.toHost(), ops.add(product, dres).toHost(), "residual += product")


def test_fp32_gemm_large_tile_path(hip, rng):
    """Big enough for the 128x128-tile kernel; checked against float64 numpy on a sample of rows."""
    D, ops = hip.DeviceTensor, hip.ops
    m, k, n = 2048, 300, 4224
    a, b = r(rng, m, k), r(rng, k, n)
    c = ops.matmul(D.fromHost(a), D.fromHost(b)).toHost()
    rows = [0, 1, 127, 128, 1000, 2047]
    assert_close(c[rows], a[rows].astype(np.float64) @ b.astype(np.float64), what="matmul 128-tile")


@pytest.mark.parametrize("m,k,n", [(70, 4100, 90), (130, 2500, 64), (128, 2047, 128)])
def test_fp32_gemm_long_contraction(hip, rng, m, k, n):
    """Few tiles and a contraction of 2048 or more: K is cut into slices that a second kernel adds in order (and one
    just under the limit, which stays whole).  Against float64."""
    D, ops = hip.DeviceTensor, hip.ops
    a, b, g = r(rng, m, k), r(rng, k, n), r(rng, m, n)
    da, db, dg = map(D.fromHost, (a, b, g))
    assert_close(ops.matmul(da, db).toHost(), (a.astype(np.float64) @ b.astype(np.float64)).astype(f32), what="matmul", scale=float(np.sqrt(k)))
    # a weight gradient: dB = X^T G over k rows of tokens
    x, w, gy = r(rng, k, m), r(rng, m, n), r(rng, k, n)
    dX, dW = ops.matmulBackward(D.fromHost(x), D.fromHost(w), D.fromHost(gy))
    assert_close(dW.toHost(), (x.astype(np.float64).T @ gy.astype(np.float64)).astype(f32), what="dW", scale=float(np.sqrt(k)))
    assert_close(dX.toHost(), (gy.astype(np.float64) @ w.astype(np.float64).T).astype(f32), what="dX", scale=float(np.sqrt(n)))


def test_linear_rank3_and_identity(hip, oracle):
    """tests/backend/cpu/ops_tests.cpp:54-63,173-184."""
    D, ops = hip.DeviceTensor, hip.ops
    out = ops.linear(D.fromHost(np.array([[3, 4]], f32)), D.fromHost(np.eye(2, dtype=f32)), D.fromHost(np.array([10, 20], f32)))
    np.testing.assert_array_equal(out.toHost().ravel(), [13, 24])
    x = np.array([1, 1, 2, 2, 3, 3, 4, 4, 5, 5, 6, 6], f32).reshape(2, 3, 2)
    out = ops.linear(D.fromHost(x), D.fromHost(np.ones((2, 1), f32)), D.zeros((1,)))
    assert out.shape == (2, 3, 1)
    np.testing.assert_array_equal(out.toHost().ravel(), x.sum(-1).ravel())


def test_bf16_conversion_is_round_to_nearest_even(hip, oracle, rng):
    import ctypes
    D = hip.DeviceTensor
    x = np.concatenate([r(rng, 1003, scale=100), np.array([1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, np.inf, -np.inf, 0.0, -0.0], f32)])
    dx = D.fromHost(x)
    out = D((x.size,), itemsize=2)
    hip.capi.call("bf_hip_cvt_f32_bf16", dx.ptr, out.ptr, x.size, None)
    bits = out.toHost().astype(np.uint32) << 16
    assert_bits_equal(bits.view(f32), oracle.roundToBf16(x))
    # transposing variant
    m = r(rng, 37, 50)
    outT, dm = D((50, 37), itemsize=2), D.fromHost(m)
    hip.capi.call("bf_hip_cvt_f32_bf16_transpose", dm.ptr, outT.ptr, 37, 50, None)
    assert_bits_equal((outT.toHost().astype(np.uint32) << 16).view(f32), oracle.roundToBf16(m).T)


@pytest.mark.parametrize("m,k,n", SHAPES + [(256, 1024, 768)])
@pytest.mark.parametrize("cached", [False, True])
def test_bf16_projection_and_gradients(hip, oracle, rng, m, k, n, cached):
    """c = bf16(a) bf16(b) with fp32 accumulation: against the fp32 oracle on bf16-rounded operands
    (tight: only the summation order differs) and against the unrounded fp32 product (2e-2)."""
    D, ops = hip.DeviceTensor, hip.ops
    a, b, g = r(rng, m, k), r(rng, k, n, scale=0.1), r(rng, m, n)
    da, db, dg = map(D.fromHost, (a, b, g))
    ar, br, gr = oracle.roundToBf16(a), oracle.roundToBf16(b), oracle.roundToBf16(g)
    fwd = ops.matmulBf16CachedWeight if cached else ops.matmulBf16
    bwd = ops.matmulBf16BackwardCachedWeight if cached else ops.matmulBf16Backward
    ops.invalidateBf16WeightCache()
    c = fwd(da, db).toHost()
    assert_close(c, oracle.matmul(ar, br), tol=1e-4, what="bf16 fwd vs rounded operands")
    assert_close(c, oracle.matmul(a, b), tol=BF16_TOL, what="bf16 fwd vs fp32")
    dA, dB = bwd(da, db, dg)
    eA, eB = oracle.matmulBackward(ar, br, gr)
    assert_close(dA.toHost(), eA, tol=1e-4, what="bf16 dA vs rounded operands")
    assert_close(dB.toHost(), eB, tol=1e-4, what="bf16 dB vs rounded operands")
    fA, fB = oracle.matmulBackward(a, b, g)
    assert_close(dA.toHost(), fA, tol=BF16_TOL, what="bf16 dA vs fp32")
    assert_close(dB.toHost(), fB, tol=BF16_TOL, what="bf16 dB vs fp32")


@pytest.mark.parametrize("m,k,n", [(4100, 129, 71), (2050, 72, 130)])
def test_bf16_gradients_with_long_contraction(hip, oracle, rng, m, k, n):
    """dB contracts over m: long enough that K is cut into slices summed in a fixed order; odd output counts."""
    D, ops = hip.DeviceTensor, hip.ops
    a, b, g = r(rng, m, k), r(rng, k, n, scale=0.1), r(rng, m, n)
    ar, br, gr = oracle.roundToBf16(a), oracle.roundToBf16(b), oracle.roundToBf16(g)
    dA, dB = ops.matmulBf16Backward(*map(D.fromHost, (a, b, g)))
    eA, eB = oracle.matmulBackward(ar, br, gr)
    assert_close(dA.toHost(), eA, tol=1e-4, what="bf16 dA vs rounded operands")
    assert_close(dB.toHost(), eB, tol=1e-4, what="bf16 dB vs rounded operands")
    again = ops.matmulBf16Backward(*map(D.fromHost, (a, b, g)))[1]
    assert_bits_equal(again.toHost(), dB.toHost(), "sliced contraction must be deterministic")


@pytest.mark.parametrize("m,k,n", [(8192, 520, 776), (6001, 300, 1100), (16384, 264, 520)])
def test_bf16_weight_gradient_transposed_in_lds(hip, oracle, rng, m, k, n):
    """Token counts long enough, and weight shapes wide enough, that dB = a^T g runs on the kernel that contracts over
    the ROWS of both operands (fragments transposed on their way out of LDS, K cut into slices): against float64 on
    the bf16-rounded operands, ragged in every dimension, and bit-reproducible."""
    D, ops = hip.DeviceTensor, hip.ops
    a, b, g = r(rng, m, k), r(rng, k, n, scale=0.1), r(rng, m, n)
    ar, br, gr = (oracle.roundToBf16(t).astype(np.float64) for t in (a, b, g))
    dA, dB = ops.matmulBf16Backward(*map(D.fromHost, (a, b, g)))
    assert_close(dA.toHost(), (gr @ br.T).astype(f32), tol=1e-4, what="bf16 dA vs rounded operands")
    assert_close(dB.toHost(), (ar.T @ gr).astype(f32), tol=1e-4, what="bf16 dB vs rounded operands")
    da_, db_, dg_, only = D.fromHost(a), D.fromHost(b), D.fromHost(g), D((k, n))
    hip.capi.call("bf_hip_matmul_bf16_backward", da_.ptr, db_.ptr, dg_.ptr, None, only.ptr, m, k, n, 0, None)
    assert_bits_equal(only.toHost(), dB.toHost(), "dB must not depend on whether dA is requested, and must be deterministic")


@pytest.mark.parametrize("m,n,k", [(768, 768, 8192), (1000, 520, 4100), (264, 3080, 9000), (40, 24, 100), (8, 8, 3)])
def test_bf16_gemm_tn_entry(hip, rng, m, n, k):
    """bf_hip_gemm_bf16_tn: C = A^T B for bf16 A[K,M], B[K,N]: sliced large tiles, a K tail, and the small-product form."""
    D = hip.DeviceTensor
    def bf16(x):
        bits = (x.view(np.uint32) >> 16).astype(np.uint16)
        return bits, (bits.astype(np.uint32) << 16).view(f32)
    (abits, a), (bbits, b) = bf16(r(rng, k, m)), bf16(r(rng, k, n))
    da, db, c = D((k, m), itemsize=2), D((k, n), itemsize=2), D((m, n))
    hip.capi.call("bf_hip_memcpy_h2d", da.ptr, abits.ctypes.data, abits.nbytes)
    hip.capi.call("bf_hip_memcpy_h2d", db.ptr, bbits.ctypes.data, bbits.nbytes)
    hip.capi.call("bf_hip_gemm_bf16_tn", da.ptr, db.ptr, c.ptr, m, n, k, None)
    assert_close(c.toHost(), (a.astype(np.float64).T @ b.astype(np.float64)).astype(f32), tol=1e-5, what="gemm_bf16_tn")


@pytest.mark.parametrize("m,k,n", [(3500, 200, 3700), (4000, 136, 4090), (8192, 64, 2048), (8192, 200, 768), (8100, 136, 700),
                                   (6200, 72, 1500)])
def test_bf16_projection_large_tile_kernel(hip, oracle, rng, m, k, n):
    """Shapes with enough 256x256 tiles for the large-product kernel (ragged edges, a K tail, and a tile grid
    that is dealt to the XCDs in blocks), and tall narrow ones that take the 128-row tiles of the sixteen-wavefront kernel
    (with a K tail and ragged edges too).  Expected value: float64 product of the bf16-rounded operands, which the oracle's
    fp32 matmul matches to 1e-6 on the sampled rows below."""
    D, ops = hip.DeviceTensor, hip.ops
    a, b = r(rng, m, k), r(rng, k, n, scale=0.1)
    ar, br = oracle.roundToBf16(a), oracle.roundToBf16(b)
    c = ops.matmulBf16(D.fromHost(a), D.fromHost(b)).toHost()
    expected = (ar.astype(np.float64) @ br.astype(np.float64)).astype(f32)
    rows = np.r_[0:3, m // 2:m // 2 + 3, m - 3:m]
    assert_close(oracle.matmul(ar[rows], br), expected[rows], tol=1e-5, what="oracle vs float64 on sampled rows")
    assert_close(c, expected, tol=1e-4, what="bf16 fwd (large tiles) vs rounded operands")


ROUTES = {"ping-pong 256": 1, "ping-pong 128": 2, "sixteen wavefronts, 128 x 256": 3, "twelve wavefronts, 128 x 192": 4,
          "sixteen wavefronts, one workgroup per CU walking tiles": 5, "twelve wavefronts, walking tiles": 6,
          "ping-pong 256, walking tiles": 7, "ping-pong 128, walking tiles": 8}


@pytest.mark.parametrize("m,k,n", [(8192, 768, 768), (8192, 200, 2304), (700, 136, 1000), (1, 8, 1), (130, 72, 193), (4100, 64, 4093), (257, 1032, 385),
                                   (4100, 1032, 4096), (9000, 520, 2500)])
def test_bf16_gemm_every_tile_form_on_the_same_operands(hip, oracle, rng, m, k, n):
    """Each large-tile kernel named through bf_hip_gemm_bf16_set_route, whatever the cost estimate would pick: float64 of
    the rounded operands to 1e-4 for one of them, and the same bits from all (an output element is accumulated over k
    in the same order by every form).  Shapes: whole rounds of tiles for the 192-wide form, ragged edges in both
    directions, a K tail, single tiles, one element; for the forms that walk a list of tiles per workgroup, products of
    more tiles than compute units with contractions shorter and longer than the eight K steps over which a finished tile
    is stored, and a ragged last tile in both directions."""
    D, call = hip.DeviceTensor, hip.capi.call
    a, b = oracle.roundToBf16(r(rng, m, k)), oracle.roundToBf16(r(rng, n, k, scale=0.1))
    ai, bi = D((m, k), itemsize=2), D((n, k), itemsize=2)
    call("bf_hip_cvt_f32_bf16", D.fromHost(a).ptr, ai.ptr, m * k, None)
    call("bf_hip_cvt_f32_bf16", D.fromHost(b).ptr, bi.ptr, n * k, None)
    expected = (a.astype(np.float64) @ b.astype(np.float64).T).astype(f32)
    first = None
    try:
        for name, route in ROUTES.items():
            call("bf_hip_gemm_bf16_set_route", route)
            guard = D.fromHost(np.full((m + 2, n), 7.0, f32))   # a row of sevens on either side of the output
            out_ptr = ctypes.c_void_p(guard.ptr.value + 4 * n)
            call("bf_hip_gemm_bf16_nt", ai.ptr, bi.ptr, out_ptr, m, n, k, None)
            got = guard.toHost()
            assert (got[0] == 7).all() and (got[-1] == 7).all(), name + ": wrote outside the output"
            if first is None:
                first = got[1:-1]
                assert_close(first, expected, tol=1e-4, what=name)
            else:
                assert_bits_equal(got[1:-1], first, name + " vs " + next(iter(ROUTES)))
    finally:
        call("bf_hip_gemm_bf16_set_route", 0)
    with pytest.raises(ValueError):
        call("bf_hip_gemm_bf16_set_route", 17)


def test_bf16_shared_input_projections_on_192_wide_tiles(hip, rng):
    """Three projections of width 768 in one product of width 2304 with split outputs: 768 = 4 x 192, so the twelve-wavefront
    form may serve it (and does for 8192 rows); the same bits as the sixteen-wavefront form and as three separate products."""
    D, ops, call = hip.DeviceTensor, hip.ops, hip.capi.call
    m, k, n = 8192, 264, 768
    da = D.fromHost(r(rng, m, k))
    dws = [D.fromHost(r(rng, k, n, scale=0.1)) for _ in range(3)]
    results = {}
    try:
        for route in (0, 3, 4):
            call("bf_hip_gemm_bf16_set_route", route)
            results[route] = [t.toHost() for t in ops.matmulBf16SharedInput(da, dws)]
    finally:
        call("bf_hip_gemm_bf16_set_route", 0)
    singles = [ops.matmulBf16(da, w).toHost() for w in dws]
    for route, outs in results.items():
        for got, single in zip(outs, singles):
            assert_bits_equal(got, single, f"route {route}: split output vs its own product")


@pytest.mark.parametrize("route", [5, 6, 7, 8])
@pytest.mark.parametrize("m,k,n,with_bias,with_residual", [(4100, 72, 4096, True, True), (8192, 648, 2304, True, False), (5000, 1100, 3072, False, True),
                                                           (4100, 136, 4093, True, True)])
def test_bf16_linear_with_adds_on_the_tile_walking_forms(hip, rng, route, m, k, n, with_bias, with_residual):
    """bias and residual added in the store of the kernels that walk a list of tiles (the sixteen- and twelve-wavefront
    forms fetch an eighth of a tile's bias and residual values a K step ahead of storing it): the same bits as the
    one-tile-per-workgroup form of the same tile shape, on products of more tiles than compute units, with contractions of
    2, 11 and 18 K steps, and a width that is no multiple of four (which the wide forms leave to the plain kernel)."""
    D, call = hip.DeviceTensor, hip.capi.call
    a, w = r(rng, m, k), r(rng, k, n, scale=0.1)
    bias, res = r(rng, n), r(rng, m, n)
    da, dw = D.fromHost(a), D.fromHost(w)
    db, dr = (D.fromHost(bias) if with_bias else None), (D.fromHost(res) if with_residual else None)
    outs = {}
    try:
        for rt in (route, {5: 3, 6: 4, 7: 1, 8: 2}[route]):
            call("bf_hip_gemm_bf16_set_route", rt)
            out = D.fromHost(np.full((m, n), 7.0, f32))
            call("bf_hip_linear_bf16", da.ptr, dw.ptr, db.ptr if db else None, dr.ptr if dr else None, out.ptr, m, k, n, 0, None)
            outs[rt] = out.toHost()
    finally:
        call("bf_hip_gemm_bf16_set_route", 0)
    (r1, o1), (r2, o2) = outs.items()
    assert_bits_equal(o1, o2, f"route {r1} vs route {r2}")
    plain = a.astype(np.float64)  # float64 of rounded operands on a sample of rows, to 2e-2 of the bf16 contract
    rows = rng.integers(0, m, 16)
    ref = plain[rows] @ w.astype(np.float64) + (bias if with_bias else 0) + (res[rows] if with_residual else 0)
    assert_close(o1[rows], ref.astype(f32), tol=2e-2, what="sampled rows against float64")


@pytest.mark.parametrize("m,k,n", [(33, 40, 24), (300, 72, 520), (2100, 136, 3000), (70, 4100, 90), (6200, 72, 1501), (4100, 136, 4093),
                                   (4100, 72, 4096)])
@pytest.mark.parametrize("with_bias,with_residual", [(True, False), (False, True), (True, True), (False, False)])
def test_bf16_linear_with_adds_in_the_store(hip, oracle, rng, m, k, n, with_bias, with_residual):
    """bf_hip_linear_bf16 = matmulBf16 followed by addBias / addBiasResidual / add (ops.hpp:14,30,8), through every
    GEMM path: small tiles, 128-row tiles on sixteen wavefronts, 256-row tiles, and a contraction cut into slices; widths
    that are multiples of four (16-byte stores after the transposition inside lane quads) and widths that are not
    (the same stores from 4-byte boundaries, the last group of a row element by element)."""
    D, ops = hip.DeviceTensor, hip.ops
    a, w, bias, res = r(rng, m, k), r(rng, k, n, scale=0.1), r(rng, n), r(rng, m, n)
    got = ops.linearBf16Fused(D.fromHost(a), D.fromHost(w), D.fromHost(bias) if with_bias else None,
                              D.fromHost(res) if with_residual else None).toHost()
    expected = (oracle.roundToBf16(a).astype(np.float64) @ oracle.roundToBf16(w).astype(np.float64)).astype(f32)
    if m * k * n <= 5_000_000:   # small enough for the oracle's own loop
        assert_close(oracle.matmul(oracle.roundToBf16(a), oracle.roundToBf16(w)), expected, tol=1e-5, what="oracle vs float64")
    if with_bias: expected = oracle.addBias(expected, bias)
    if with_residual: expected = oracle.add(expected, res)
    assert_close(got, expected, tol=1e-4, what="fused linear")


@pytest.mark.parametrize("m,k,n", [(1, 768, 768), (1, 3072, 768), (1, 768, 32003), (2, 72, 9000), (3, 520, 41), (5, 1032, 8200), (8, 768, 2304),
                                   (7, 8, 1), (1, 4100, 16), (4, 44, 300), (4, 3072, 768),
                                   (16, 3072, 768), (33, 2504, 40), (64, 768, 2304), (9, 72, 100), (40, 4104, 96), (32, 776, 33), (6, 20000, 8), (128, 768, 768),
                                   (100, 3080, 136)])
@pytest.mark.parametrize("with_bias,with_residual", [(True, True), (False, False)])
def test_bf16_products_of_a_few_rows(hip, oracle, rng, m, k, n, with_bias, with_residual):
    """matmulBf16 / linearBf16 (ops.hpp:14,30,8) with a few rows, the shape of a step of incremental decoding (model.cpp:169,
    one new token per sequence).  Up to four rows are served by a walk over the weights instead of MFMA tiles: widths on
    both sides of the switch from one to four columns a wavefront, odd widths, a contraction of several steps a lane, and
    one that is not a multiple of eight (which stays on the tiles).  Five to 128 rows take 32 x 32 MFMA tiles whose
    wavefronts share out the contraction: one and two row tiles, ragged tiles, contractions that end in half a step, that go
    round the load loop again, and that are cut into slices over several workgroups."""
    D, ops = hip.DeviceTensor, hip.ops
    a, w, bias, res = r(rng, m, k), r(rng, k, n, scale=0.1), r(rng, n), r(rng, m, n)
    expected = (oracle.roundToBf16(a).astype(np.float64) @ oracle.roundToBf16(w).astype(np.float64)).astype(f32)
    if m * k * n <= 5_000_000:
        assert_close(oracle.matmul(oracle.roundToBf16(a), oracle.roundToBf16(w)), expected, tol=1e-5, what="oracle vs float64")
    plain = ops.matmulBf16(D.fromHost(a), D.fromHost(w)).toHost()
    assert_close(plain, expected, tol=1e-4, what="few-row product")
    again = ops.matmulBf16(D.fromHost(a), D.fromHost(w)).toHost()
    assert_bits_equal(again, plain, "the same product twice")
    got = ops.linearBf16Fused(D.fromHost(a), D.fromHost(w), D.fromHost(bias) if with_bias else None,
                              D.fromHost(res) if with_residual else None).toHost()
    if with_bias: expected = oracle.addBias(expected, bias)
    if with_residual: expected = oracle.add(expected, res)
    assert_close(got, expected, tol=1e-4, what="few-row product with the adds in its store")
    if n % 256 == 0 or n <= 300:   # three projections of one input: one product with split outputs when the width allows
        ws = [w, r(rng, k, n, scale=0.1), r(rng, k, n, scale=0.1)]
        outs = ops.matmulBf16SharedInput(D.fromHost(a), [D.fromHost(x) for x in ws])
        for i in range(3):
            e = (oracle.roundToBf16(a).astype(np.float64) @ oracle.roundToBf16(ws[i]).astype(np.float64)).astype(f32)
            assert_close(outs[i].toHost(), e, tol=1e-4, what=f"shared-input product {i}")


@pytest.mark.parametrize("m,k,n,count", [(50, 40, 24, 3), (300, 136, 256, 3), (4096, 64, 1024, 3), (4100, 256, 256, 3), (260, 72, 512, 2),
                                         (64, 32, 48, 1), (8192, 520, 256, 3), (8200, 300, 512, 2)])
@pytest.mark.parametrize("cached", [False, True])
def test_bf16_projections_of_a_shared_input(hip, oracle, rng, m, k, n, count, cached):
    """Q/K/V-style projections of one input and their gradients (ops_transformer.cu:217-257, autodiff.cu:756-798) against
    the same products computed one by one: widths that fuse into one GEMM with split outputs (multiples of 256), widths
    that do not, and a token count long enough that the weight-gradient contraction is cut into slices."""
    D, ops = hip.DeviceTensor, hip.ops
    a = r(rng, m, k)
    ws = [r(rng, k, n, scale=0.1) for _ in range(count)]
    gs = [r(rng, m, n) for _ in range(count)]
    da, dws, dgs = D.fromHost(a), [D.fromHost(w) for w in ws], [D.fromHost(g) for g in gs]
    ops.invalidateBf16WeightCache()
    ar = oracle.roundToBf16(a).astype(np.float64)
    outs = ops.matmulBf16SharedInput(da, dws, cached=cached)
    for i in range(count):
        assert_close(outs[i].toHost(), (ar @ oracle.roundToBf16(ws[i]).astype(np.float64)).astype(f32), tol=1e-4, what=f"product {i}")
    dA, dBs = ops.matmulBf16SharedInputBackward(da, dws, dgs, cached=cached)
    eA = sum(oracle.roundToBf16(gs[i]).astype(np.float64) @ oracle.roundToBf16(ws[i]).astype(np.float64).T for i in range(count))
    assert_close(dA.toHost(), eA.astype(f32), tol=1e-4, what="dA")
    for i in range(count):
        eB = ar.T @ oracle.roundToBf16(gs[i]).astype(np.float64)
        assert_close(dBs[i].toHost(), eB.astype(f32), tol=1e-4, what=f"dB {i}")
    # agreement with the one-by-one operators (same rounding, different summation split): tight
    single = ops.matmulBf16(da, dws[0]).toHost()
    assert_close(outs[0].toHost(), single, tol=1e-5, what="shared-input product vs matmulBf16")
    # partial requests: only the input gradient, only one weight gradient
    onlyA, none = ops.matmulBf16SharedInputBackward(da, dws, dgs, cached=cached, want_dB=(False, False, False))
    assert_bits_equal(onlyA.toHost(), dA.toHost(), "dA must not depend on which weight gradients are requested")
    _, some = ops.matmulBf16SharedInputBackward(da, dws, dgs, cached=cached, want_dA=False, want_dB=(True,) + (False,) * 2)
    assert_close(some[0].toHost(), dBs[0].toHost(), tol=1e-5, what="single requested weight gradient")


def test_bf16_weight_cache_semantics(hip, oracle, rng):
    """A cached weight image is reused until invalidateBf16WeightCache() (ops_tensorcore.cu:98-131,448)."""
    D, ops = hip.DeviceTensor, hip.ops
    a, b = r(rng, 16, 32), r(rng, 32, 24)
    da, db = D.fromHost(a), D.fromHost(b)
    ops.invalidateBf16WeightCache()
    first = ops.matmulBf16CachedWeight(da, db).toHost()
    b2 = r(rng, 32, 24)
    hip.capi.call("bf_hip_memcpy_h2d", db.ptr, b2.ctypes.data, b2.nbytes)   # weights change in place
    stale = ops.matmulBf16CachedWeight(da, db).toHost()
    assert_bits_equal(stale, first, "cached image must be reused")
    ops.invalidateBf16WeightCache()
    fresh = ops.matmulBf16CachedWeight(da, db).toHost()
    assert_close(fresh, oracle.matmul(oracle.roundToBf16(a), oracle.roundToBf16(b2)), tol=1e-4)
    lin = ops.linearBf16(da, db, D.fromHost(np.ones(24, f32))).toHost()
    assert_close(lin, oracle.matmul(oracle.roundToBf16(a), oracle.roundToBf16(b2)) + 1, tol=1e-4)


def bf16_bits_to_f32(raw, rows, cols):
    """Reads a bf16 image kept as raw storage in a float32 tensor of half the width."""
    bits = np.ascontiguousarray(raw).view(np.uint16).reshape(rows, cols)
    return (bits.astype(np.uint32) << 16).view(np.float32)


@pytest.mark.parametrize("m,d,hidden,act", [(64, 32, 128, 0), (64, 32, 128, 1), (64, 32, 128, 2), (300, 72, 264, 0), (300, 72, 264, 1),
                                            (1000, 64, 2048, 2), (4096, 256, 1024, 0), (4096, 256, 1024, 1), (8192, 768, 3072, 0),
                                            (2048, 8, 8, 0), (513, 512, 512, 1), (256, 4096, 256, 1), (256, 4096, 256, 2),
                                            (1, 768, 3072, 1), (3, 72, 264, 0), (8, 1032, 520, 2), (1, 8, 8, 1), (8, 8200, 64, 0)])
def test_feed_forward_with_the_elementwise_steps_in_the_gemm_stores(hip, oracle, rng, m, d, hidden, act):
    """bf_hip_feedforward_bf16[_backward] (feedForwardForwardCached / feedForwardBackwardCached in the bf16 mode,
    ops_transformer.cu:182-215, autodiff.cu:719-750) against the same block built from the separate operators, which are
    themselves checked against the oracle: same roundings, so the agreement is tight.  Shapes cover the small-tile GEMM with
    the transposed-image weight gradients, ragged row counts, the large-tile kernels with fragments transposed in LDS, and
    blocks of at most eight rows (a step of incremental decoding: products as walks over the weights, the activation in the
    first one's store; the last case's rows are too long for that walk's LDS); act 0/1/2 = silu/gelu/relu."""
    D, ops = hip.DeviceTensor, hip.ops
    x, w1, b1 = r(rng, m, d), r(rng, d, hidden, scale=0.1), r(rng, hidden, scale=0.5)
    w2, b2, res, g = r(rng, hidden, d, scale=0.1), r(rng, d), r(rng, m, d), r(rng, m, d)
    dx, dw1, db1, dw2, db2, dres, dg = map(D.fromHost, (x, w1, b1, w2, b2, res, g))
    ops.invalidateBf16WeightCache()
    out, z, hImage, xImage = ops.feedForwardBf16Fused(dx, dw1, db1, dw2, db2, dres, act)
    # the separate operators
    gemm1 = ops.matmulBf16(dx, dw1)
    hiddenT = ops.addBiasAct(gemm1, db1, act)
    expectedOut = ops.linearBf16Fused(hiddenT, dw2, db2, dres)
    assert_close(z.toHost(), ops.addBias(gemm1, db1).toHost(), tol=1e-6, what="pre-activation")
    assert_bits_equal(bf16_bits_to_f32(hImage.toHost(), m, hidden), oracle.roundToBf16(ops._act(z, act).toHost()), "hidden image")
    assert_bits_equal(bf16_bits_to_f32(xImage.toHost(), m, d), oracle.roundToBf16(x), "input image")
    assert_close(out.toHost(), expectedOut.toHost(), tol=1e-5, what="block output")
    if m * d * hidden <= 20_000_000:   # and against float64 arithmetic on the rounded operands
        zr = oracle.roundToBf16(x).astype(np.float64) @ oracle.roundToBf16(w1).astype(np.float64) + b1
        assert_close(z.toHost(), zr.astype(f32), tol=1e-4, what="pre-activation vs float64")
    # gradients
    dX, dW1, dB1, dW2, dB2 = ops.feedForwardBf16FusedBackward(dx, None, dw1, dw2, z, hImage, dg, act)
    eHidden, eW2 = ops.matmulBf16Backward(hiddenT, dw2, dg)
    eGemm1, eB1 = ops.addBiasActBackward(gemm1, db1, eHidden, act)
    eX, eW1 = ops.matmulBf16Backward(dx, dw1, eGemm1)
    for got, exp, name in ((dX, eX, "dX"), (dW1, eW1, "dW1"), (dB1, eB1, "dB1"), (dW2, eW2, "dW2"), (dB2, ops.biasGradientOnly(dg), "dB2")):
        assert_close(got.toHost(), exp.toHost(), tol=2e-5, what=name)
    # the same gradients from the input image alone
    again = ops.feedForwardBf16FusedBackward(None, xImage, dw1, dw2, z, hImage, dg, act)
    for got, exp, name in zip(again, (dX, dW1, dB1, dW2, dB2), ("dX", "dW1", "dB1", "dW2", "dB2")):
        assert_bits_equal(got.toHost(), exp.toHost(), name + " from the input image")


def test_feed_forward_fused_rejects_widths_that_are_not_multiples_of_eight(hip):
    D, ops = hip.DeviceTensor, hip.ops
    with pytest.raises(ValueError):
        ops.feedForwardBf16Fused(D.zeros((4, 12)), D.zeros((12, 16)), D.zeros((16,)), D.zeros((16, 12)), D.zeros((12,)))


@pytest.mark.parametrize("m,k,n", [(512, 128, 256), (70, 300, 33), (257, 4100, 129), (2048, 300, 4224), (64, 64, 64)])
def test_fp32_gemm_with_adds_in_the_store(hip, rng, m, k, n):
    """bf_hip_gemm_f32_adds: the product with bias and residual added where it is stored is bit-identical to the product
    followed by the separate add kernels, in every tile form (32 x 32, 64 x 64, 128 x 128, K slices), and the residual
    may be the output itself (accumulation in place)."""
    D, ops, call = hip.DeviceTensor, hip.ops, hip.capi.call
    a, b, bias, res = r(rng, m, k), r(rng, k, n), r(rng, n), r(rng, m, n)
    da, db, dbias, dres = map(D.fromHost, (a, b, bias, res))
    product = ops.matmul(da, db)
    out = D((m, n))
    call("bf_hip_gemm_f32_adds", 0, 0, da.ptr, db.ptr, dbias.ptr, dres.ptr, out.ptr, m, n, k, None)
    assert_bits_equal(out.toHost(), ops.addBiasResidual(product, dbias, dres).toHost(), "product + bias + residual")
    call("bf_hip_gemm_f32_adds", 0, 0, da.ptr, db.ptr, dbias.ptr, None, out.ptr, m, n, k, None)
    assert_bits_equal(out.toHost(), ops.addBias(product, dbias).toHost(), "product + bias")
    acc = D.fromHost(res)
    call("bf_hip_gemm_f32_adds", 0, 0, da.ptr, db.ptr, None, acc.ptr, acc.ptr, m, n, k, None)
    assert_bits_equal(acc.toHost(), ops.add(product, dres).toHost(), "residual += product")
    # transposed operands take the same store: dA += g b^T
    g = r(rng, m, n)
    dg = D.fromHost(g)
    dA, _ = ops.matmulBackward(da, db, dg)
    acc = D.fromHost(a)
    call("bf_hip_gemm_f32_adds", 0, 1, dg.ptr, db.ptr, None, acc.ptr, acc.ptr, m, k, n, None)
    assert_bits_equal(acc.toHost(), ops.add(dA, da).toHost(), "a += g b^T")


def test_fp32_gemm_group_matches_single_products(hip, rng):
    """bf_hip_gemm_f32_group: products of different shapes and orientations in one call (one launch when they are small)
    give the bits of the same products launched one by one, adds included; a member too large for the shared launch
    sends the whole group down the one-by-one road with the same results."""
    D, call = hip.DeviceTensor, hip.capi.call
    Problem = hip.capi.GemmF32Problem

    def run(specs):
        # specs: (transA, transB, M, N, K, with_bias, accumulate)
        problems, singles, tensors = [], [], []
        for ta, tb, m, n, k, with_bias, accumulate in specs:
            a = D.fromHost(r(rng, *((k, m) if ta else (m, k))))
            b = D.fromHost(r(rng, *((n, k) if tb else (k, n))))
            bias = D.fromHost(r(rng, n)) if with_bias else None
            start = r(rng, m, n)
            c_group, c_single = D.fromHost(start), D.fromHost(start)
            tensors += [a, b, bias, c_group, c_single]
            problems.append(Problem(a.ptr, b.ptr, c_group.ptr, bias.ptr if bias else None, c_group.ptr if accumulate else None, m, n, k, ta, tb))
            call("bf_hip_gemm_f32_adds", ta, tb, a.ptr, b.ptr, bias.ptr if bias else None, c_single.ptr if accumulate else None, c_single.ptr,
                 m, n, k, None)
            singles.append((c_group, c_single))
        array = (Problem * len(problems))(*problems)
        call("bf_hip_gemm_f32_group", array, len(problems), None)
        for i, (got, want) in enumerate(singles):
            assert_bits_equal(got.toHost(), want.toHost(), f"member {i} of {specs}")

    run([(0, 1, 512, 128, 256, False, False), (1, 0, 128, 256, 512, False, False)])                    # a projection's two gradients
    run([(0, 0, 512, 128, 128, False, False)] * 3)                                                      # Q, K and V of one input
    run([(0, 1, 70, 33, 45, True, False), (1, 1, 5, 7, 300, False, True), (1, 0, 130, 64, 513, True, True), (0, 0, 1, 1, 1, False, False)])
    run([(0, 0, 64, 64, 64, False, False), (0, 0, 2048, 4224, 300, True, False)])                       # one member needs the large tiles
    run([(0, 1, 96, 96, 4100, False, False), (1, 0, 96, 96, 96, False, False)])                         # one member needs K slices
    run([(0, 0, 1, 768, 768, False, False)] * 3)                                                        # Q, K and V of one decoded token: one walk
    run([(0, 0, 5, 300, 3000, True, True), (0, 0, 5, 300, 3000, False, False)])                         # few rows, adds after the slice sums
    run([(0, 0, 3, 41, 20, True, False)] * 2 + [(0, 0, 3, 41, 20, False, True)])                        # few rows, one slice, odd width
    run([(0, 0, 2, 64, 64, False, False), (0, 0, 2, 64, 72, False, False)])                             # few rows of different shapes: one by one
