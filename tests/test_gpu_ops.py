"""GPU parity of normalisation, element-wise, rotary and arg-max ops against the CPU oracle."""
import numpy as np
import pytest

from conftest import TOL

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,dim", [(1, 2048), (768, 2048), (729, 1152), (3, 3), (5, 100), (3, 2047), (4, 2044), (2, 4000)])
def test_layernorm(moon, O, ctx, rows, dim):
    x = O.fill_normal_f16((rows, dim), 0, 0, 1.5)
    g = (O.fill_normal_f16((dim,), 0, 1, 0.1).astype(np.float32) + 1).astype(np.float16)
    b = O.fill_normal_f16((dim,), 0, 2, 0.1)
    y = moon.ops.layer_norm(x, g, b, ctx=ctx)
    assert O.rel_frobenius(y, O.layernorm(x, g, b)) <= TOL


def test_layernorm_reference_cases(moon, ctx):
    # ops_test.zig:1773-1884: {-1,0,1} -> mean 0 / var 1; zero variance stays finite; eps <= 0 -> InvalidEpsilon
    x = np.array([[-1, 0, 1]], dtype=np.float16)
    one, zero = np.ones(3, dtype=np.float16), np.zeros(3, dtype=np.float16)
    y = moon.ops.layer_norm(x, one, zero, ctx=ctx).astype(np.float32)
    assert abs(y.mean()) < 1e-3 and abs(y.var() - 1.0) < 1e-2
    y = moon.ops.layer_norm(np.full((1, 3), 2.0, dtype=np.float16), one, zero, ctx=ctx)
    assert np.all(np.isfinite(y.astype(np.float32)))
    with pytest.raises(moon.InvalidEpsilon):
        moon.ops.layer_norm(x, one, zero, eps=-1e-5, ctx=ctx)


def test_gelu(moon, O, ctx):
    x = np.concatenate([O.fill_normal_f16((8192,), 0, 0, 2.0), np.array([0, -0.0, 10, -10, 65504, -65504], dtype=np.float16)])
    assert O.rel_frobenius(moon.ops.gelu(x, ctx=ctx), O.gelu(x)) <= TOL


def test_broadcast_add_and_add(moon, O, ctx):
    a = O.fill_normal_f16((729, 1152), 0, 0, 1.0)
    b = O.fill_normal_f16((1152,), 0, 1, 0.5)
    assert np.array_equal(moon.ops.broadcast_add_simd(a, b, ctx=ctx), O.bias_add(a, b))  # one IEEE add: exact
    a3 = O.fill_normal_f16((2, 27, 16), 0, 2, 1.0)
    p3 = O.fill_normal_f16((1, 27, 16), 0, 3, 1.0)
    want = np.stack([O.add(a3[0], p3[0]), O.add(a3[1], p3[0])])
    assert np.array_equal(moon.ops.broadcast_add_simd(a3, p3, ctx=ctx), want)  # ops.zig:1796-1857 pos-emb case
    c = O.fill_normal_f16((729, 1152), 0, 4, 1.0)
    assert np.array_equal(moon.ops.add(a, c, ctx=ctx), O.add(a, c))


def test_argmax_first_max_wins(moon, O, ctx):
    x = O.fill_normal_f16((51200,), 0, 0, 0.9)
    assert moon.sampling.argmax(x, ctx=ctx) == O.argmax(x) == int(np.argmax(x.astype(np.float32)))
    x[:] = 0
    x[[40000, 7, 30000]] = 3.0  # ties: lowest index (sampling.zig:265 strict '>')
    assert moon.sampling.argmax(x, ctx=ctx) == 7
    x[:] = -np.inf
    assert moon.sampling.argmax(x, ctx=ctx) == 0
    x[0] = np.nan
    x[5] = 1.0
    assert moon.sampling.argmax(x, ctx=ctx) == O.argmax(x) == 0  # nothing compares greater than NaN


@pytest.mark.parametrize("H,S,D,rot,pos0", [(32, 1, 64, 32, 1023), (32, 768, 64, 32, 0), (2, 5, 64, 64, 3), (4, 9, 16, 8, 100)])
def test_rope_apply(moon, O, ctx, H, S, D, rot, pos0):
    x = O.fill_normal_f16((H, S, D), 0, 0, 1.0)
    table = O.rope_table(rot, 2048, 10000.0)
    pos = np.arange(pos0, pos0 + S)
    y = moon.rope.apply_rot_emb(x, H, D, table, pos, rot, ctx=ctx)
    ref = O.rope_apply(x, table, pos, rot)
    assert O.rel_frobenius(y, ref) <= TOL
    assert np.array_equal(y[..., rot:], x[..., rot:])  # pass-through tail is a bit copy (rope.zig:256-269)
    with pytest.raises(moon.InvalidRotationDimension):
        moon.rope.apply_rot_emb(x, H, D, table, pos, rot + 2, ctx=ctx)


def test_device_copy_is_exact_and_rejects_unaligned_sizes(moon, ctx):
    n = 1 << 20
    src = ctx.alloc(n * 2)
    dst = ctx.alloc(n * 2)
    src.fill_normal(n, 3, 7, 1.0)
    dst.fill_const(n, 0.0)
    dst.copy_from(src, n * 2)
    assert np.array_equal(dst.to_host((n,)).view(np.uint16), src.to_host((n,)).view(np.uint16))
    rc = ctx.lib.moon_dev_copy(ctx.handle, dst.ptr, src.ptr, 24)
    assert rc == moon._lib.EINVAL
    src.free()
    dst.free()


def test_greedy_profile_advances_like_greedy(moon, ctx):
    """The per-launch event timing variant decodes the same tokens as the plain loop and reports every launch."""
    cfg = moon.text_model.make_config(vocab=512, dim=2048, hidden_dim=8192, n_layers=2, n_heads=32, max_seq=64)
    m = moon.text_model.TextModel(cfg, seed=5, std=0.02, ctx=ctx)
    ids = np.arange(7, dtype=np.uint32)
    m.forward(ids)
    want = m.greedy(6)
    # (the LM head launch also takes the arg-max and moves the position on: those two kinds report no launch of their own)
    for mode, counts in ((2, [[12, 12, 12, 6, 0, 0]]), (0, [[12, 0, 0, 6, 0, 0], [12, 0, 12, 6, 0, 0], [12, 12, 12, 6, 0, 0]]), (3, [[12, 0, 12, 6, 0, 0], [12, 12, 12, 6, 0, 0]])):
        m.reset()
        m.set_decode_mode(mode)
        m.forward(ids)
        got, prof = m.greedy_profile(6)
        assert got.tolist() == want.tolist()
        assert [prof[k][1] for k in m.PROFILE_KERNELS] in counts  # modes 0 and 3 fold kernels together where the device allows
        assert all(us > 0 for us, n in prof.values() if n)
    m.close()


def test_device_rope_table_matches_oracle(moon, O, ctx):
    """rope.precomputeFreqsCis (rope.zig:32-128) as the device builds it for the text session: all 2048 x 16 x 2 entries
    against the oracle's table.  Both evaluate the reference's f32 steps; pow, cos and sin come from different libraries, each
    within an ulp or two of the true value, and the entries are in [-1, 1]: the bound is 2 ulp of 1.0 in absolute terms."""
    want = O.rope_table(32, 2048, 10000.0)
    got = moon.rope.precompute_freqs_cis_device(32, 2048, 10000.0, ctx=ctx)
    assert got.shape == want.shape == (2048, 16, 2)
    diff = np.abs(got.astype(np.float64) - want.astype(np.float64))
    print(f"device rope table: max |diff| {diff.max():.3e}, entries that differ {int((diff > 0).sum())} of {diff.size}")
    assert diff.max() <= 2.0 ** -22
    assert np.array_equal(got[0], want[0])  # position 0: cos 1, sin 0 exactly
    # a smaller table with another base
    want = O.rope_table(8, 33, 500.0)
    got = moon.rope.precompute_freqs_cis_device(8, 33, 500.0, ctx=ctx)
    assert np.abs(got.astype(np.float64) - want).max() <= 2.0 ** -22
    with pytest.raises(moon.context.InvalidRotationDimension):
        moon.rope.precompute_freqs_cis_device(7, 4, ctx=ctx)
