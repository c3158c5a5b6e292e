"""GPU parity of the matrix products (GEMV, MFMA GEMM) against the CPU oracle, through the C ABI."""
import numpy as np
import pytest

from conftest import TOL

pytestmark = pytest.mark.gpu


def test_device_fill_matches_host_generator(moon, O, ctx):
    for n, seed, stream, std in [(1000, 0, 0, 1.0), (4099, 7, 3, 0.02), (1 << 20, 1, 11, 0.02)]:
        buf = ctx.alloc(n * 2)
        buf.fill_normal(n, seed, stream, std)
        got = buf.to_host((n,))
        want = O.fill_normal_f16((n,), seed, stream, std)
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    ids = ctx.alloc(4 * 1000)
    ids.fill_uniform_u32(1000, 0, 50, 51200)
    assert np.array_equal(ids.to_host((1000,), np.uint32), O.fill_uniform_u32(1000, 0, 50, 51200))


# config 1 of the baseline and the other decoder projections (text_model.zig:193,296,310,317,339)
@pytest.mark.parametrize("N,K", [(8192, 2048), (6144, 2048), (2048, 2048), (2048, 8192), (51200, 2048), (1000, 520), (7, 24), (33, 30)])
def test_gemv_nt(moon, O, ctx, N, K):
    x = O.fill_normal_f16((1, K), 0, 0, 1.0)
    w = O.fill_normal_f16((N, K), 0, 1, 0.02)
    y = moon.hgemm_trans.matmul(x, w, ctx=ctx)
    ref = O.hgemm_trans(x, w)
    assert y.shape == (1, N)
    assert O.rel_frobenius(y, ref) <= TOL
    # information: agreement with the f64-accumulated result is as good as the f32 oracle's own
    assert O.rel_frobenius(y, O.hgemm_trans(x, w, f64=True)) <= TOL


@pytest.mark.parametrize("epi", ["bias", "bias_gelu"])
def test_gemv_fused_epilogues(moon, O, ctx, epi):
    N, K = 8192, 2048
    x = O.fill_normal_f16((1, K), 0, 0, 1.0)
    w = O.fill_normal_f16((N, K), 0, 1, 0.02)
    b = O.fill_normal_f16((N,), 0, 2, 0.02)
    c = np.empty((1, N), dtype=np.float16)
    L = moon._lib
    code = L.EPI_BIAS if epi == "bias" else L.EPI_BIAS_GELU
    ctx.check(ctx.lib.moon_linear(ctx.handle, x.ctypes.data, 1, K, w.ctypes.data, N, L.B_NK, b.ctypes.data, code, c.ctypes.data))
    ref = O.bias_add(O.hgemm_trans(x, w), b)
    if epi == "bias_gelu":
        ref = O.gelu(ref)
    assert O.rel_frobenius(c, ref) <= TOL


# config 2 (vision fc1 / fc2, B[K,N]) and the other encoder shapes, M = 729 and the reference's own 1458
@pytest.mark.parametrize("M,K,N", [(729, 1152, 4304), (729, 4304, 1152), (729, 1152, 3456), (729, 1152, 1152), (1458, 1152, 4304)])
def test_hgemm_vision_shapes(moon, O, ctx, M, K, N):
    a = O.fill_normal_f16((M, K), 0, 0, 1.0)
    b = O.fill_normal_f16((K, N), 0, 1, 0.02)
    c = moon.hgemm.matmul(a, b, ctx=ctx)
    assert O.rel_frobenius(c, O.hgemm(a, b)) <= TOL
    assert O.rel_frobenius(c, O.hgemm(a, b, f64=True)) <= TOL


# prefill shapes (B_t[N,K]) -- hgemm_trans tiled path (hgemm_trans.zig:457-487)
@pytest.mark.parametrize("M,K,N", [(768, 2048, 6144), (768, 2048, 2048), (768, 2048, 8192), (768, 8192, 2048), (2, 2048, 512), (5, 64, 40)])
def test_hgemm_trans_prefill_shapes(moon, O, ctx, M, K, N):
    a = O.fill_normal_f16((M, K), 0, 0, 1.0)
    bt = O.fill_normal_f16((N, K), 0, 1, 0.02)
    c = moon.hgemm_trans.matmul(a, bt, ctx=ctx)
    assert O.rel_frobenius(c, O.hgemm_trans(a, bt)) <= TOL


# more 128 x 128 tiles than CUs: the 256 x 128 and 192 x 128 tile kernels, with ragged last tiles in m and n, one and two k-tiles
@pytest.mark.parametrize("M,K,N,epi", [(1000, 128, 6000, "bias"), (2000, 64, 3000, "bias_gelu"), (257, 192, 33000, "none"),
                                       (1458, 1152, 4304, "bias_gelu"), (700, 128, 8000, "bias_gelu"), (768, 64, 8192, "bias")])
def test_linear_many_tiles(moon, O, ctx, M, K, N, epi):
    a = O.fill_normal_f16((M, K), 3, 0, 1.0)
    bt = O.fill_normal_f16((N, K), 3, 1, 0.05)
    bias = O.fill_normal_f16((N,), 3, 2, 0.5)
    c = np.empty((M, N), dtype=np.float16)
    L = moon._lib
    code = {"none": L.EPI_NONE, "bias": L.EPI_BIAS, "bias_gelu": L.EPI_BIAS_GELU}[epi]
    ctx.check(ctx.lib.moon_linear(ctx.handle, a.ctypes.data, M, K, bt.ctypes.data, N, L.B_NK, bias.ctypes.data if epi != "none" else None, code,
                                  c.ctypes.data))
    ref = O.hgemm_trans(a, bt)
    if epi != "none":
        ref = O.bias_add(ref, bias)
    if epi == "bias_gelu":
        ref = O.gelu(ref)
    assert O.rel_frobenius(c, ref) <= TOL
    # every row and column was written by the tile that owns it (a tile written at a wrong offset shows up as a large error there)
    err = np.abs(c.astype(np.float32) - ref.astype(np.float32))
    assert err.max() <= 0.05 * max(1.0, float(np.abs(ref.astype(np.float32)).max()))


# the reference's own test shapes: non-square, tile-edge sizes around T=168 and 158..162 (matmul_test.zig:214-322, 494-496)
@pytest.mark.parametrize("M,K,N", [(4, 3, 4), (50, 30, 70), (25, 80, 35), (100, 20, 100), (32, 32, 32), (167, 167, 167), (168, 168, 168),
                                   (169, 169, 169), (158, 158, 158), (159, 160, 161), (162, 162, 162), (2000, 180, 1600), (1, 1, 1), (3, 1, 3)])
def test_hgemm_reference_test_shapes(moon, O, ctx, M, K, N):
    a = (O.fill_normal_f16((M, K), 1, 0, 1.0).astype(np.float32) * 0.5).astype(np.float16)
    b = O.fill_normal_f16((K, N), 1, 1, 0.05)
    c = moon.hgemm.matmul(a, b, ctx=ctx)
    assert O.rel_frobenius(c, O.hgemm(a, b)) <= TOL
    ct = moon.hgemm_trans.matmul(a, np.ascontiguousarray(b.T), ctx=ctx)
    # NT and NN agree (bench.zig:204-209 relies on it)
    assert O.rel_frobenius(ct, c) <= TOL


# A [K, N] operand read in place (hgemm.zig:210-216) against the same product over a transposed copy: the two paths multiply
# and add in the same order, so the results are the same bits.  Vision shapes (with and without a split of K), a partial last
# k-tile (K = 16 * 71), ragged last tiles in m and n, one k-step, one row, and shapes that take the larger tiles.
@pytest.mark.parametrize("M,K,N", [(729, 1152, 4304), (729, 4304, 1152), (300, 1136, 1000), (130, 2064, 264), (64, 16, 8), (1, 32, 128),
                                   (729, 1152, 1152),
                                   # more tiles than compute units: the 256- and the 192-row kernels, the latter also with a ragged last column tile
                                   (1458, 1152, 4304), (768, 2048, 8192), (700, 128, 8000)])
def test_hgemm_operand_read_in_place_equals_the_transposed_copy(moon, O, ctx, monkeypatch, M, K, N):
    a = O.fill_normal_f16((M, K), 6, 0, 1.0)
    b = O.fill_normal_f16((K, N), 6, 1, 0.05)
    c = moon.hgemm.matmul(a, b, ctx=ctx)
    assert "read in place" in ctx.last_kernel()
    monkeypatch.setenv("MOON_GEMM_KN_TRANSPOSE", "1")
    ct = moon.hgemm.matmul(a, b, ctx=ctx)
    assert "read in place" not in ctx.last_kernel()
    monkeypatch.delenv("MOON_GEMM_KN_TRANSPOSE")
    assert np.array_equal(c.view(np.uint16), ct.view(np.uint16))
    assert O.rel_frobenius(c, O.hgemm(a, b)) <= TOL


def test_hgemm_known_answers(moon, O, ctx):
    # A x I = A (matmul_test.zig:251-276)
    a = O.fill_normal_f16((32, 32), 2, 0, 1.0)
    assert np.array_equal(moon.hgemm.matmul(a, np.eye(32, dtype=np.float16), ctx=ctx), a)
    # all-ones 32x32 -> 32 ; 0.01 fill -> 32 * f16(0.01)^2 (matmul_test.zig:324-367)
    ones = np.ones((32, 32), dtype=np.float16)
    assert np.all(moon.hgemm.matmul(ones, ones, ctx=ctx) == np.float16(32.0))
    small = np.full((32, 32), 0.01, dtype=np.float16)
    want = np.float16(np.float32(32.0) * np.float32(small[0, 0]) * np.float32(small[0, 0]))
    got = moon.hgemm.matmul(small, small, ctx=ctx)
    assert np.all(np.abs(got.astype(np.float32) - np.float32(want)) <= 1e-5)
    # 2x2 known answer {19,22,43,50} (matmul_test.zig:608-637)
    a2 = np.array([[1, 2], [3, 4]], dtype=np.float16)
    b2 = np.array([[5, 6], [7, 8]], dtype=np.float16)
    assert np.array_equal(moon.hgemm.matmul(a2, b2, ctx=ctx), np.array([[19, 22], [43, 50]], dtype=np.float16))


def test_hgemm_shape_errors(moon, ctx):
    a = np.zeros((4, 3), dtype=np.float16)
    with pytest.raises(moon.IncompatibleTensorShapes):  # matmul_test.zig:278-290
        moon.hgemm.matmul(a, np.zeros((4, 4), dtype=np.float16), ctx=ctx)
    with pytest.raises(moon.IncompatibleTensorShapes):
        moon.hgemm_trans.matmul(a, np.zeros((4, 4), dtype=np.float16), ctx=ctx)
    with pytest.raises(moon.InvalidTensorDimension):
        moon.hgemm.matmul(np.zeros((4, 3, 1), dtype=np.float16), a, ctx=ctx)


def test_registered_weight_is_reused(moon, O, ctx):
    x = O.fill_normal_f16((1, 2048), 0, 0, 1.0)
    w = O.fill_normal_f16((2048, 2048), 0, 1, 0.02)
    ref = O.hgemm_trans(x, w)
    ctx.register_weight(w)
    y1 = moon.hgemm_trans.matmul(x, w, ctx=ctx)
    keep = w.copy()
    w[:] = 0  # the resident copy, not the host buffer, must be what is multiplied now
    y2 = moon.hgemm_trans.matmul(x, w, ctx=ctx)
    ctx.unregister_weight(w)
    y3 = moon.hgemm_trans.matmul(x, w, ctx=ctx)
    assert O.rel_frobenius(y1, ref) <= TOL and np.array_equal(y1, y2)
    assert np.all(y3 == 0)
    w[:] = keep


def test_registered_weight_in_hgemm_layout(moon, O, ctx):
    """hgemm.matmul reads B as [K, N] (hgemm.zig:210-216).  A registered weight used that way gets its [N, K] copy once, on
    the first call; later calls (also with another row count, and as a one-row product) use it and give the bits of the
    unregistered path, and a weight registered again takes its new contents."""
    a = O.fill_normal_f16((729, 1152), 0, 0, 1.0)
    w = O.fill_normal_f16((1152, 776), 0, 1, 0.02)  # [K, N]
    plain = moon.hgemm.matmul(a, w, ctx=ctx)
    assert O.rel_frobenius(plain, O.hgemm(a, w)) <= TOL
    ctx.register_weight(w)
    first = moon.hgemm.matmul(a, w, ctx=ctx)
    keep = w.copy()
    w[:] = 0  # the resident copies are what is multiplied now
    again = moon.hgemm.matmul(a, w, ctx=ctx)
    fewer = moon.hgemm.matmul(a[:33], w, ctx=ctx)
    one = moon.hgemm.matmul(a[:1], w, ctx=ctx)
    w[:] = keep
    assert np.array_equal(first, plain) and np.array_equal(again, plain)
    assert np.array_equal(fewer, moon.hgemm.matmul(a[:33], keep, ctx=ctx))
    assert O.rel_frobenius(one, O.hgemm(a[:1], keep)) <= TOL
    w[:] = keep * np.float16(2)
    ctx.register_weight(w)  # again: both resident copies are replaced
    doubled = moon.hgemm.matmul(a, w, ctx=ctx)
    ctx.unregister_weight(w)
    assert O.rel_frobenius(doubled, O.hgemm(a, w)) <= TOL
    assert np.array_equal(moon.hgemm.matmul(a, w, ctx=ctx), doubled)


# The product kernels that the default choice takes only for some shapes (or never), each named through the context's knob:
# the same products to the same bar.  Shapes cover ragged tile edges, a partial last k-tile (K % 64 == 16, 32, 48), K short
# of the stage count, the split K, and every epilogue.
@pytest.mark.parametrize("kernel", ["w114", "w212", "w221", "dma", "dma256", "regs"])
def test_named_product_kernels(moon, O, ctx, kernel):
    L = moon._lib
    shapes = [(200, 320, 264, "bias"), (300, 80, 520, "none"), (729, 1152, 1152, "bias"), (513, 144, 776, "bias_gelu"),
              (130, 2096, 136, "bias"), (257, 48, 264, "none")]
    ctx.set_gemm_kernel(kernel)
    try:
        for M, K, N, epi in shapes:
            a = O.fill_normal_f16((M, K), 0, 0, 1.0)
            w = O.fill_normal_f16((N, K), 0, 1, 0.05)
            b = O.fill_normal_f16((N,), 0, 2, 0.1)
            code = {"none": L.EPI_NONE, "bias": L.EPI_BIAS, "bias_gelu": L.EPI_BIAS_GELU}[epi]
            got = np.empty((M, N), dtype=np.float16)
            ctx.check(ctx.lib.moon_linear(ctx.handle, a.ctypes.data, M, K, w.ctypes.data, N, L.B_NK, b.ctypes.data if epi != "none" else None, code,
                                          got.ctypes.data))
            ref = O.hgemm_trans(a, w)
            if epi != "none":
                ref = O.bias_add(ref, b)
            if epi == "bias_gelu":
                ref = O.gelu(ref)
            err = O.rel_frobenius(got, ref)
            assert err <= TOL, (kernel, M, K, N, epi, err)
    finally:
        ctx.set_gemm_kernel("")
    with pytest.raises(moon.InvalidArgument):
        ctx.set_gemm_kernel("nonesuch")
