"""GPU parity of the attention kernels against the CPU oracle."""
import ctypes as C

import numpy as np
import pytest

from conftest import TOL

pytestmark = pytest.mark.gpu


def _qkv(O, H, Lq, Lk, D, seed=0):
    return (O.fill_normal_f16((H, Lq, D), seed, 0, 1.0), O.fill_normal_f16((H, Lk, D), seed, 1, 1.0),
            O.fill_normal_f16((H, Lk, D), seed, 2, 1.0))


# config 3 decode: 32 heads x 64, kv = 1024; plus short / ragged lengths and the 2048 limit
@pytest.mark.parametrize("kv", [1, 2, 7, 8, 9, 63, 100, 1024, 2047, 2048])
def test_single_masked_sdpa(moon, O, ctx, kv):
    q, k, v = _qkv(O, 32, 1, kv, 64)
    mask = np.ones((1, 1, kv), dtype=bool)
    out = moon.attention.single_masked_sdpa(q, k, v, mask, ctx=ctx)
    assert O.rel_frobenius(out, O.sdpa_single(q, k, v, mask)) <= TOL


def test_single_masked_sdpa_with_holes_and_limit(moon, O, ctx):
    q, k, v = _qkv(O, 32, 1, 300, 64)
    mask = np.ones((1, 1, 300), dtype=bool)
    mask[0, 0, 10:200:3] = False
    out = moon.attention.single_masked_sdpa(q, k, v, mask, ctx=ctx)
    assert O.rel_frobenius(out, O.sdpa_single(q, k, v, mask)) <= TOL
    q, k, v = _qkv(O, 32, 1, 2049, 64)
    with pytest.raises(moon.SequenceTooLong):  # attention.zig:769
        moon.attention.single_masked_sdpa(q, k, v, np.ones((1, 1, 2049), dtype=bool), ctx=ctx)


# config 3 prefill: causal 768; continuation (pos > 0); tiny and ragged cases
@pytest.mark.parametrize("H,S,pos,D", [(32, 768, 0, 64), (32, 39, 729, 64), (4, 5, 0, 64), (2, 130, 3, 64), (3, 17, 0, 32)])
def test_multi_masked_sdpa_causal(moon, O, ctx, H, S, pos, D):
    q, k, v = _qkv(O, H, S, pos + S, D)
    mask = moon.attention.create_attention_mask(pos, S)
    assert np.array_equal(mask, O.attention_mask(pos, S))
    out = moon.attention.multi_masked_sdpa(q, k, v, mask, H, D, ctx=ctx)
    assert O.rel_frobenius(out, O.sdpa_multi(q, k, v, mask)) <= TOL


def test_multi_masked_sdpa_arbitrary_mask(moon, O, ctx):
    H, S, D = 4, 70, 64
    q, k, v = _qkv(O, H, S, S, D)
    rng = np.random.default_rng(0)
    mask = rng.random((1, S, S)) < 0.7
    mask[0, np.arange(S), np.arange(S)] = True  # no fully masked row
    out = moon.attention.multi_masked_sdpa(q, k, v, mask, H, D, ctx=ctx)
    assert O.rel_frobenius(out, O.sdpa_multi(q, k, v, mask)) <= TOL


# config 4 attention: 16 heads x 72, 729 tokens (and the reference's duplicated-crop 1458)
@pytest.mark.parametrize("H,L,D", [(16, 729, 72), (16, 1458, 72), (2, 50, 72), (1, 1, 72), (3, 65, 64)])
def test_multi_maskless_sdpa(moon, O, ctx, H, L, D):
    q, k, v = _qkv(O, H, L, L, D)
    out = moon.attention.multi_maskless_sdpa(H, D, q, k, v, ctx=ctx)
    assert O.rel_frobenius(out, O.sdpa_multi(q, k, v, None)) <= TOL


def test_duplicated_keys_leave_output_unchanged(moon, O, ctx):
    # the reference encodes the same crop twice and attends jointly over 2x729 tokens (vision_model.zig:36-38,308-310)
    q, k, v = _qkv(O, 16, 100, 100, 72)
    one = moon.attention.multi_maskless_sdpa(16, 72, q, k, v, ctx=ctx)
    two = moon.attention.multi_maskless_sdpa(16, 72, q, np.concatenate([k, k], 1), np.concatenate([v, v], 1), ctx=ctx)
    assert O.rel_frobenius(two, one) <= TOL


@pytest.mark.parametrize("pos", [0, 1, 8, 100, 1023, 2047])
def test_fused_decode_attention_step(moon, O, ctx, pos):
    """rope(q,k) + cache append + attention over pos+1 keys, on a cache in the reference layout."""
    H, D, rot, S = 32, 64, 32, 2048
    qkv = O.fill_normal_f16((3 * H * D,), 0, 0, 1.0)
    ck = np.zeros((H, S, D), dtype=np.float16)
    cv = np.zeros((H, S, D), dtype=np.float16)
    ck[:, :pos] = O.fill_normal_f16((H, pos, D), 0, 1, 1.0)
    cv[:, :pos] = O.fill_normal_f16((H, pos, D), 0, 2, 1.0)
    table = O.rope_table(rot, S, 10000.0)
    # oracle: text_model.zig:198-286
    q, k, v = (O.split_heads(qkv.reshape(1, -1), i, H, D) for i in range(3))
    pid = np.array([pos])
    qr, kr = O.rope_apply(q, table, pid, rot), O.rope_apply(k, table, pid, rot)
    ck_ref, cv_ref = ck.copy(), cv.copy()
    ck_ref[:, pos] = kr[:, 0]
    cv_ref[:, pos] = v[:, 0]
    want = O.merge_heads(O.sdpa_single(qr, np.ascontiguousarray(ck_ref[:, :pos + 1]), np.ascontiguousarray(cv_ref[:, :pos + 1]),
                                       np.ones((1, 1, pos + 1), bool)))
    d_qkv, d_ck, d_cv, d_tab = ctx.to_device(qkv), ctx.to_device(ck), ctx.to_device(cv), ctx.to_device(table)
    d_out = ctx.alloc(H * D * 2)
    ctx.check(ctx.lib.moon_dev_decode_attention(ctx.handle, d_qkv.ptr, d_ck.ptr, d_cv.ptr, d_tab.ptr, d_out.ptr, H, D, rot, S, pos))
    ctx.sync()
    got = d_out.to_host((1, H * D))
    assert O.rel_frobenius(got, want) <= TOL
    # the append wrote exactly k' and v at position pos and nothing else
    assert O.rel_frobenius(d_ck.to_host((H, S, D))[:, pos], ck_ref[:, pos]) <= TOL
    assert np.array_equal(d_cv.to_host((H, S, D)), cv_ref)
    got_ck = d_ck.to_host((H, S, D))
    got_ck[:, pos] = 0
    ck[:, pos] = 0
    assert np.array_equal(got_ck, ck)


@pytest.mark.parametrize("H,S,pos,D", [(2, 16, 0, 64), (2, 33, 31, 64), (1, 64, 0, 64), (3, 65, 1, 64), (2, 257, 300, 64),
                                       (2, 96, 64, 72), (1, 31, 0, 72), (2, 200, 0, 72)])
def test_matrix_core_attention_edge_shapes_causal(moon, O, ctx, H, S, pos, D):
    """Query blocks of 32 and key tiles of 64 with ragged ends, causal with and without a cached prefix."""
    q, k, v = _qkv(O, H, S, pos + S, D)
    mask = moon.attention.create_attention_mask(pos, S)
    out = moon.attention.multi_masked_sdpa(q, k, v, mask, H, D, ctx=ctx)
    err = O.rel_frobenius(out, O.sdpa_multi(q, k, v, mask))
    print(f"causal H={H} S={S} pos={pos} D={D}: rel-Frobenius {err:.2e}")
    assert err <= TOL


@pytest.mark.parametrize("H,Lq,Lkv,D", [(2, 16, 1, 64), (2, 40, 63, 64), (2, 40, 64, 64), (2, 40, 65, 64), (1, 100, 257, 72), (2, 729, 300, 72)])
def test_matrix_core_attention_rectangular_maskless(moon, O, ctx, H, Lq, Lkv, D):
    q = O.fill_normal_f16((H, Lq, D), 0, 1, 1.0)
    k = O.fill_normal_f16((H, Lkv, D), 0, 2, 1.0)
    v = O.fill_normal_f16((H, Lkv, D), 0, 3, 1.0)
    out = moon.attention.multi_maskless_sdpa(H, D, q, k, v, ctx=ctx)
    err = O.rel_frobenius(out, O.sdpa_multi(q, k, v, None))
    print(f"maskless H={H} Lq={Lq} Lkv={Lkv} D={D}: rel-Frobenius {err:.2e}")
    assert err <= TOL


def test_matrix_core_attention_peaked_softmax(moon, O, ctx):
    """Large score spread (one key dominates most rows): the running maximum has to rescale correctly."""
    H, L, D = 2, 300, 64
    q = O.fill_normal_f16((H, L, D), 0, 1, 4.0)
    k = O.fill_normal_f16((H, L, D), 0, 2, 4.0)
    v = O.fill_normal_f16((H, L, D), 0, 3, 1.0)
    out = moon.attention.multi_maskless_sdpa(H, D, q, k, v, ctx=ctx)
    assert np.isfinite(out.astype(np.float32)).all()
    assert O.rel_frobenius(out, O.sdpa_multi(q, k, v, None)) <= TOL


def test_matrix_core_attention_over_seeded_random_shapes(moon, O, ctx):
    """The matrix-core kernel over shapes no other test names: head counts 1..32 (multiples of 8 take the die-wise work
    mapping), 16..300 rows, head_dim 64 (causal with a past, and maskless) and 72, keys not a multiple of the 64-key tile."""
    rng = np.random.default_rng(1)
    worst = 0.0
    for it in range(48):
        D = 72 if it % 2 else 64
        H = int(rng.integers(1, 9)) if it % 5 else 8 * int(rng.integers(1, 5))
        S = int(rng.integers(16, 300))
        q = O.fill_normal_f16((H, S, D), it, 0, 1.0)
        if D == 64 and it % 3 == 0:
            pos = int(rng.integers(0, 200))
            k, v = O.fill_normal_f16((H, pos + S, D), it, 1, 1.0), O.fill_normal_f16((H, pos + S, D), it, 2, 1.0)
            mask = moon.attention.create_attention_mask(pos, S)
            out, want = moon.attention.multi_masked_sdpa(q, k, v, mask, H, D, ctx=ctx), O.sdpa_multi(q, k, v, mask)
        else:
            k, v = O.fill_normal_f16((H, S, D), it, 1, 1.0), O.fill_normal_f16((H, S, D), it, 2, 1.0)
            out, want = moon.attention.multi_maskless_sdpa(H, D, q, k, v, ctx=ctx), O.sdpa_multi(q, k, v, None)
        err = O.rel_frobenius(out, want)
        assert err <= TOL, (it, D, H, S, err)
        worst = max(worst, err)
    print(f"\nworst rel-Frobenius over 48 shapes: {worst:.2e}")


def test_decode_attention_after_cleanup_starts_from_fresh_counters(moon, O, ctx):
    """moon_cleanup frees the workspace that holds the per-head counters of the one-launch decode attention
    (cleanupThreadPool, attention.zig:814).  The next call gets new memory, whatever it holds, at whatever address, and must
    give the same bits as before: counters that were believed to be still cleared would make the merge run early or never."""
    H, D, rot, S, pos = 32, 64, 32, 2048, 300
    qkv = O.fill_normal_f16((3 * H * D,), 0, 10, 1.0)
    ck = np.zeros((H, S, D), dtype=np.float16)
    cv = np.zeros((H, S, D), dtype=np.float16)
    ck[:, :pos] = O.fill_normal_f16((H, pos, D), 0, 11, 1.0)
    cv[:, :pos] = O.fill_normal_f16((H, pos, D), 0, 12, 1.0)
    d_qkv, d_tab = ctx.to_device(qkv), ctx.to_device(O.rope_table(rot, S, 10000.0))
    d_out = ctx.alloc(H * D * 2)

    def step():
        d_ck, d_cv = ctx.to_device(ck), ctx.to_device(cv)
        ctx.check(ctx.lib.moon_dev_decode_attention(ctx.handle, d_qkv.ptr, d_ck.ptr, d_cv.ptr, d_tab.ptr, d_out.ptr, H, D, rot, S, pos))
        ctx.sync()
        return d_out.to_host((1, H * D))

    first = step()
    assert np.array_equal(step(), first)  # the counters count on from launch to launch
    for nbytes in (1 << 16, 1 << 18, 1 << 20, 1 << 22):
        ctx.cleanup()
        junk = [ctx.to_device(np.full(nbytes, 0xFF, dtype=np.uint8)) for _ in range(4)]  # what freed memory may come back as
        del junk
        assert np.array_equal(step(), first)
        assert np.array_equal(step(), first)
