"""The decode-attention entry point that allocates nothing (its split partials live in a static device array) against
moon_dev_decode_attention, through the C ABI: same bits, on two calls in a row, the second with a smaller input."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _case(O, ctx, H, pos, seed):
    D, rot, S = 64, 32, 2048
    qkv = O.fill_normal_f16((3 * H * D,), seed, 0, 1.0)
    ck = np.zeros((H, S, D), dtype=np.float16)
    cv = np.zeros((H, S, D), dtype=np.float16)
    ck[:, :pos] = O.fill_normal_f16((H, pos, D), seed, 1, 1.0)
    cv[:, :pos] = O.fill_normal_f16((H, pos, D), seed, 2, 1.0)
    return qkv, ck, cv


def _run(ctx, entry, qkv, ck, cv, table, H, pos):
    D, rot, S = 64, 32, 2048
    d_qkv, d_ck, d_cv = ctx.to_device(qkv), ctx.to_device(ck), ctx.to_device(cv)
    d_out = ctx.alloc(H * D * 2)
    ctx.check(entry(ctx.handle, d_qkv.ptr, d_ck.ptr, d_cv.ptr, table.ptr, d_out.ptr, H, D, rot, S, pos))
    ctx.sync()
    res = d_out.to_host((H * D,)), d_ck.to_host((H, S, D)), d_cv.to_host((H, S, D))
    for b in (d_qkv, d_ck, d_cv, d_out):
        b.free()
    return res


def test_no_alloc_decode_attention_equals_the_allocating_entry_point(moon, O, ctx):
    table = ctx.to_device(O.rope_table(32, 2048, 10000.0))
    # second call smaller in both heads and keys: stale partials of the first call stay in the array and must not be read
    for H, pos, seed in ((32, 1023, 0), (5, 6, 1), (128, 300, 2), (1, 0, 3)):
        qkv, ck, cv = _case(O, ctx, H, pos, seed)
        want = _run(ctx, ctx.lib.moon_dev_decode_attention, qkv, ck, cv, table, H, pos)
        got = _run(ctx, ctx.lib.moon_dev_decode_attention_noalloc, qkv, ck, cv, table, H, pos)
        for g, w in zip(got, want):
            assert np.array_equal(g.view(np.uint16), w.view(np.uint16)), f"H={H} pos={pos}"
        # and against the oracle, to the parity bar of the allocating entry point
        q, k, v = (O.split_heads(qkv.reshape(1, -1), i, H, 64) for i in range(3))
        tab = O.rope_table(32, 2048, 10000.0)
        pid = np.array([pos])
        qr, kr = O.rope_apply(q, tab, pid, 32), O.rope_apply(k, tab, pid, 32)
        ck[:, pos], cv[:, pos] = kr[:, 0], v[:, 0]
        ref = O.merge_heads(O.sdpa_single(qr, np.ascontiguousarray(ck[:, :pos + 1]), np.ascontiguousarray(cv[:, :pos + 1]),
                                          np.ones((1, 1, pos + 1), bool)))
        assert O.rel_frobenius(got[0].reshape(1, -1), ref) <= 1e-3
    with pytest.raises(moon.context.InvalidTensorDimension):  # beyond the static workspace
        ctx.check(ctx.lib.moon_dev_decode_attention_noalloc(ctx.handle, table.ptr, table.ptr, table.ptr, table.ptr, table.ptr, 129, 64, 32, 2048, 0))
    table.free()
