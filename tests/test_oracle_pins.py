"""Pins of the CPU oracle (oracle/moon_oracle.c) that do not depend on its own formulas:
the reference's known-answer tests, torch CPU library routines, f64 brute force written here, and invariants.
A plausible mistake (dropped term, wrong sign or index, transposed operand) must fail one of them."""
import math

import numpy as np
import pytest
import torch


def compare_results_f16(expected, actual, eps):
    """compareResultsF16 of the reference (matmul_test.zig:108-152): relative error above 1, absolute below."""
    e, a = expected.astype(np.float32), actual.astype(np.float32)
    diff = np.abs(e - a)
    big = np.abs(e) > 1.0
    rel = np.where(big, diff / np.maximum(np.abs(e), 1e-30), diff)
    thr = np.where(big, eps, eps * 0.1)
    return int((rel > thr).sum())


# ------------------------------------------------------------------ f16 <-> f32 (ops_test.zig:2641-2806)
def test_f16_conversions_exact_values(O):
    cases = [(1.0, 0x3C00), (0.5, 0x3800), (-1.0, 0xBC00), (0.0, 0x0000), (65504.0, 0x7BFF), (-65504.0, 0xFBFF),
             (0.00006103515625, 0x0400), (float("inf"), 0x7C00), (float("-inf"), 0xFC00), (-0.0, 0x8000)]
    for f, bits in cases:
        assert O.f2h(f) == bits
        back = O.h2f(bits)
        assert back == f and math.copysign(1, back) == math.copysign(1, f)
    assert math.isnan(O.h2f(O.f2h(float("nan"))))
    # round to nearest even at the half-way points (vcvtps2ph $0, tensor.zig:258-268)
    assert O.f2h(1.0 + 2**-11) == 0x3C00 and O.f2h(1.0 + 3 * 2**-11) == 0x3C02
    assert O.f2h(65520.0) == 0x7C00  # overflow to inf at the rounding boundary
    for bits in range(0, 0x7C00, 37):  # round trip of every 37th finite value equals numpy's view
        assert O.h2f(bits) == float(np.array([bits], dtype=np.uint16).view(np.float16)[0])


# ------------------------------------------------------------------ GEMM
def test_hgemm_reference_known_answers(O):
    # sequential pattern 4x3 . 3x4 with eps 0.005 (matmul_test.zig:154-180), expected from an independent f64 product
    a = (np.arange(12, dtype=np.float32) * np.float32(0.01)).astype(np.float16).reshape(4, 3)
    b = (np.arange(12, dtype=np.float32) * np.float32(0.01)).astype(np.float16).reshape(3, 4)
    want = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float16)
    assert compare_results_f16(want, O.hgemm(a, b), 0.005) == 0
    # A x I = A (matmul_test.zig:251-276)
    a = O.fill_normal_f16((32, 32), 2, 0, 1.0)
    assert np.array_equal(O.hgemm(a, np.eye(32, dtype=np.float16)), a)
    # all-ones 32x32 -> 32; 0.01 fill -> 32 * f16(0.01)^2 (matmul_test.zig:324-367)
    ones = np.ones((32, 32), dtype=np.float16)
    assert np.all(O.hgemm(ones, ones) == np.float16(32))
    small = np.full((32, 32), 0.01, dtype=np.float16)
    assert np.allclose(O.hgemm(small, small).astype(np.float32), 32.0 * float(small[0, 0]) ** 2, atol=1e-5)
    # sgemm known answers (matmul_test.zig:608-731): 2x2 {19,22,43,50}, 1x1, 3x1 . 1x3, zeros
    assert np.array_equal(O.sgemm([[1, 2], [3, 4]], [[5, 6], [7, 8]]), np.array([[19, 22], [43, 50]], dtype=np.float32))
    assert np.array_equal(O.sgemm([[3]], [[4]]), [[12]])
    assert np.array_equal(O.sgemm([[1], [2], [3]], [[4, 5, 6]]), np.outer([1, 2, 3], [4, 5, 6]).astype(np.float32))
    assert np.all(O.sgemm(np.zeros((5, 7)), np.ones((7, 3))) == 0)
    assert np.array_equal(O.hgemm(np.array([[1, 2], [3, 4]], np.float16), np.array([[5, 6], [7, 8]], np.float16)),
                          np.array([[19, 22], [43, 50]], np.float16))


def test_hgemm_shape_errors(O):
    a = np.zeros((4, 3), np.float16)
    with pytest.raises(O.IncompatibleTensorShapes):  # matmul_test.zig:278-290
        O.hgemm(a, np.zeros((4, 4), np.float16))
    with pytest.raises(O.IncompatibleTensorShapes):
        O.hgemm_trans(a, np.zeros((4, 4), np.float16))
    with pytest.raises(O.InvalidTensorDimension):
        O.hgemm(np.zeros((4, 3, 1), np.float16), a)


@pytest.mark.parametrize("M,K,N", [(50, 30, 70), (25, 80, 35), (100, 20, 100), (167, 168, 169), (158, 160, 162), (2000, 180, 1600),
                                   (1, 2048, 512), (729, 1152, 64), (3, 7, 5)])
def test_hgemm_against_torch_and_its_own_f64(O, M, K, N):
    a = (O.fill_normal_f16((M, K), 1, 0, 1.0))
    b = O.fill_normal_f16((K, N), 1, 1, 0.05)
    got = O.hgemm(a, b)
    want = (torch.from_numpy(a).float() @ torch.from_numpy(b).float()).half().numpy()  # library routine, f32 accumulate
    assert compare_results_f16(want, got, 0.05) == 0  # the reference's own bar for 2000x180x1600 (matmul_test.zig:182-212)
    assert O.rel_frobenius(got, want) < 3e-4
    want64 = (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float16)
    assert O.rel_frobenius(got, want64) < 3e-4 and O.rel_frobenius(O.hgemm(a, b, f64=True), want64) < 1e-4
    # transposed-B entry point == plain one (bench.zig:204-209); a transposed-operand slip shows here
    bt = np.ascontiguousarray(b.T)
    assert np.array_equal(O.hgemm_trans(a, bt).view(np.uint16), got.view(np.uint16)) or O.rel_frobenius(O.hgemm_trans(a, bt), got) < 2e-4
    if M != N:  # non-square: swapping the operands cannot be right
        assert O.hgemm_trans(a, bt).shape == (M, N)


def test_refstyle_kernels_agree_with_oracle(O):
    """The 'reference-style' timed kernels (T=168 tiles / 32-output GEMV chunks) compute the same products."""
    for M, K, N in [(1, 2048, 1000), (170, 200, 340), (729, 1152, 96)]:
        a = O.fill_normal_f16((M, K), 3, 0, 1.0)
        b = O.fill_normal_f16((K, N), 3, 1, 0.02)
        ref = O.hgemm(a, b)
        assert O.rel_frobenius(O.refstyle_hgemm(a, b, False, 4), ref) < 1e-4
        assert O.rel_frobenius(O.refstyle_hgemm(a, np.ascontiguousarray(b.T), True, 4), ref) < 1e-4
    q, k, v = (O.fill_normal_f16(s, 3, i, 1.0) for i, s in enumerate([(32, 1, 64), (32, 77, 64), (32, 77, 64)]))
    assert O.rel_frobenius(O.refstyle_sdpa_single(q, k, v, 4), O.sdpa_single(q, k, v, np.ones((1, 1, 77), bool))) < 1e-4


# ------------------------------------------------------------------ element-wise
def test_bias_add_reference_cases(O):
    # [3,4] + [4] and the positional-embedding case [2,3,4] + [1,3,4] (ops_test.zig:2547-2639)
    a = np.arange(12, dtype=np.float16).reshape(3, 4)
    b = (np.arange(4) * 2).astype(np.float16)
    assert np.array_equal(O.bias_add(a, b), (a.astype(np.float32) + b.astype(np.float32)).astype(np.float16))
    a3 = np.arange(24, dtype=np.float16).reshape(2, 3, 4)
    b3 = (np.arange(12) * 2).astype(np.float16).reshape(3, 4)
    got = np.stack([O.add(a3[0], b3), O.add(a3[1], b3)])
    assert np.array_equal(got, (a3.astype(np.float32) + b3.astype(np.float32)[None]).astype(np.float16))
    # rounding: f16(f32(a)+f32(b)), one rounding of the exact sum
    x = O.fill_normal_f16((1000,), 0, 0, 3.0)
    y = O.fill_normal_f16((1000,), 0, 1, 0.01)
    assert np.array_equal(O.add(x, y), (x.astype(np.float64) + y.astype(np.float64)).astype(np.float16))


def test_gelu_closed_form_and_torch(O):
    x = np.concatenate([O.fill_normal_f16((4096,), 0, 0, 2.0), np.array([0, -0.0, 8, -8, 65504, -65504], np.float16)])
    got = O.gelu(x).astype(np.float64)
    xd = x.astype(np.float64)
    c, alpha = 0.7978515625, 0.044708251953125  # the reference's f16-typed constants (ops.zig:1641-1642)
    want = 0.5 * xd * (1.0 + np.tanh(c * (xd + alpha * xd**3)))
    # one f16 rounding of the result, plus the f32 cancellation in (1 + tanh) for negative inputs
    ulp = np.maximum(np.abs(want) * 2.0**-10, 2.0**-24) + 3e-7 * np.abs(xd)
    assert np.all(np.abs(got - want) <= ulp)
    # library routine: tanh GELU with exact constants differs by at most the constant rounding (~5e-5 relative) + 1 f16 ulp
    tg = torch.nn.functional.gelu(torch.from_numpy(x).float(), approximate="tanh").double().numpy()
    assert np.all(np.abs(got - tg) <= 2 * ulp + 1e-4 * np.abs(tg))
    assert O.f2h(0.7978845608) == O.f2h(0.7978515625) and abs(O.h2f(O.f2h(0.044715)) - alpha) == 0


def test_layernorm_reference_cases_and_torch(O):
    # {-1,0,1}: mean 0, variance 1 after normalisation; zero variance stays finite; eps <= 0 is an error (ops_test.zig:1773-1884)
    one, zero = np.ones(3, np.float16), np.zeros(3, np.float16)
    y = O.layernorm(np.array([[-1, 0, 1]], np.float16), one, zero).astype(np.float32)
    assert abs(y.mean()) < 1e-3 and abs(y.var() - 1) < 1e-2
    assert np.all(np.isfinite(O.layernorm(np.full((1, 3), 2.0, np.float16), one, zero).astype(np.float32)))
    with pytest.raises(ValueError):
        O.layernorm(np.zeros((1, 3), np.float16), one, zero, eps=-1e-5)
    for rows, dim in [(4, 2048), (3, 1152), (2, 100)]:
        x = O.fill_normal_f16((rows, dim), 0, 0, 1.7)
        g = (O.fill_normal_f16((dim,), 0, 1, 0.2).astype(np.float32) + 1).astype(np.float16)
        b = O.fill_normal_f16((dim,), 0, 2, 0.3)
        want = torch.nn.functional.layer_norm(torch.from_numpy(x).float(), (dim,), torch.from_numpy(g).float(),
                                              torch.from_numpy(b).float(), eps=O.EPS_F16).half().numpy()
        assert O.rel_frobenius(O.layernorm(x, g, b), want) < 3e-4
    assert abs(O.EPS_F16 - 1.00135803e-5) < 1e-12  # 1e-5 rounded to f16 (text_model.zig:28,154-160)


def test_softmax_rows(O):
    s = np.random.default_rng(0).normal(0, 5, (7, 33)).astype(np.float32)
    s[2, 5:] = -np.inf
    got = O.softmax_rows(s)
    assert np.allclose(got, torch.softmax(torch.from_numpy(s), -1).numpy(), atol=1e-6)
    assert np.allclose(got.sum(-1), 1.0, atol=1e-5)
    # below -88 the exponential is clamped to exactly 0 (ops.zig:1590)
    t = np.array([[0.0, -89.0, -100.0]], np.float32)
    assert np.array_equal(O.softmax_rows(t), [[1.0, 0.0, 0.0]])
    # a row whose sum is 0 is left untouched (ops.zig:1595): only -inf rows qualify
    u = np.full((1, 4), -np.inf, np.float32)
    assert np.all(np.isneginf(O.softmax_rows(u)))


# ------------------------------------------------------------------ RoPE (rope.zig)
def test_rope_table_and_apply_properties(O):
    rot, S = 32, 2048
    table = O.rope_table(rot, S, 10000.0)
    assert table.shape == (S, rot // 2, 2)
    p = np.array([0, 1, 17, 1023, 2047])
    i = np.arange(rot // 2)
    ang = p[:, None].astype(np.float64) * (10000.0 ** (-(2 * i) / rot))[None, :]
    assert np.allclose(table[p, :, 0], np.cos(ang), atol=2e-4) and np.allclose(table[p, :, 1], np.sin(ang), atol=2e-4)
    assert np.all(table[0, :, 0] == 1) and np.all(table[0, :, 1] == 0)
    x = O.fill_normal_f16((4, 6, 64), 0, 0, 1.0)
    # position 0 is the identity; the tail beyond rot_dim is a bit copy (rope.zig:256-269)
    assert np.array_equal(O.rope_apply(x, table, np.zeros(6, int), rot), x)
    y = O.rope_apply(x, table, np.arange(100, 106), rot)
    assert np.array_equal(y[..., rot:], x[..., rot:])
    # each (i, i+16) pair is rotated: norm preserved up to f16 rounding; half-split pairing, not interleaved
    xf, yf = x.astype(np.float64), y.astype(np.float64)
    n_in = np.hypot(xf[..., :16], xf[..., 16:32])
    n_out = np.hypot(yf[..., :16], yf[..., 16:32])
    assert np.allclose(n_in, n_out, atol=3e-3)
    # HF "rotate_half" formulation in f64
    pos = np.arange(100, 106)
    inv = 10000.0 ** (-(np.arange(0, rot, 2)) / rot)
    fr = pos[:, None] * inv[None, :]
    cos, sin = np.cos(np.concatenate([fr, fr], -1)), np.sin(np.concatenate([fr, fr], -1))
    xr = xf[..., :rot]
    rot_half = np.concatenate([-xr[..., 16:], xr[..., :16]], -1)
    want = xr * cos[None] + rot_half * sin[None]
    assert np.allclose(yf[..., :rot], want, atol=4e-3)
    # angle additivity: rotating by p1 then p2 equals rotating by p1+p2 (up to the two f16 roundings)
    a = O.rope_apply(O.rope_apply(x, table, np.full(6, 40), rot), table, np.full(6, 60), rot)
    b = O.rope_apply(x, table, np.full(6, 100), rot)
    assert O.rel_frobenius(a, b) < 2e-3


# ------------------------------------------------------------------ attention (attention.zig)
def _attention_f64(q, k, v, mask):
    """Brute force written independently of the oracle."""
    q, k, v = (t.astype(np.float64) for t in (q, k, v))
    s = np.einsum("hqd,hkd->hqk", q, k) / math.sqrt(q.shape[-1])
    if mask is not None:
        s = np.where(mask[:, :, :k.shape[1]], s, -np.inf)
    s = s - s.max(-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(-1, keepdims=True)
    return np.einsum("hqk,hkd->hqd", p, v)


def test_attention_mask_closed_form(O):
    for pos, seq in [(0, 1), (0, 5), (3, 1), (7, 4), (729, 39)]:
        m = O.attention_mask(pos, seq)
        j = np.arange(pos + seq)[None, :]
        i = np.arange(seq)[:, None]
        assert m.shape == (1, seq, pos + seq) and np.array_equal(m[0], (j < pos) | (j - pos <= i))


@pytest.mark.parametrize("H,Lq,Lk,D", [(2, 8, 8, 64), (3, 5, 9, 72), (32, 1, 40, 64), (1, 1, 1, 64)])
def test_sdpa_against_brute_force_and_torch(O, H, Lq, Lk, D):
    q, k, v = (O.fill_normal_f16(s, 0, i, 1.0) for i, s in enumerate([(H, Lq, D), (H, Lk, D), (H, Lk, D)]))
    mask = O.attention_mask(Lk - Lq, Lq) if Lk >= Lq else None
    for m in (None, mask):
        want = _attention_f64(q, k, v, m)
        got = O.sdpa_multi(q, k, v, m).astype(np.float64)
        assert np.abs(got - want).max() < 3e-3
        assert np.abs(O.sdpa_f64(q, k, v, m) - want).max() < 1e-9
        tm = None if m is None else torch.from_numpy(m[:, :, :Lk])
        tw = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q).float(), torch.from_numpy(k).float(),
                                                              torch.from_numpy(v).float(), attn_mask=tm).numpy()
        assert np.abs(got - tw).max() < 3e-3
    if Lq == 1:
        ones = np.ones((1, 1, Lk), bool)
        assert np.abs(O.sdpa_single(q, k, v, ones).astype(np.float64) - _attention_f64(q, k, v, None)).max() < 3e-3


def test_sdpa_invariants(O):
    H, L, D = 4, 12, 64
    q, k, v = (O.fill_normal_f16((H, L, D), 1, i, 1.0) for i in range(3))
    causal = O.attention_mask(0, L)
    out = O.sdpa_multi(q, k, v, causal)
    assert np.array_equal(out[:, 0], v[:, 0])  # causal row 0 sees only key 0
    assert np.array_equal(O.sdpa_multi(q[:, :1], k[:, :1], v[:, :1], None), v[:, :1])  # kv_len == 1
    vconst = np.broadcast_to(v[:, :1], v.shape).copy()
    assert O.rel_frobenius(O.sdpa_multi(q, k, vconst, None), vconst) < 1e-3  # equal V rows -> that row
    # duplicating keys and values leaves the output unchanged (the reference's duplicated-crop batch, vision_model.zig:36-38)
    two = O.sdpa_multi(q, np.concatenate([k, k], 1), np.concatenate([v, v], 1), None)
    assert O.rel_frobenius(two, O.sdpa_multi(q, k, v, None)) < 1e-3
    # decode with an all-true mask == last row of the causal prefill
    last = O.sdpa_single(np.ascontiguousarray(q[:, -1:]), k, v, np.ones((1, 1, L), bool))
    assert O.rel_frobenius(last, np.ascontiguousarray(out[:, -1:])) < 1e-3
    with pytest.raises(O.SequenceTooLong):  # attention.zig:769
        O.sdpa_single(q[:, :1], np.zeros((H, 2049, D), np.float16), np.zeros((H, 2049, D), np.float16), np.ones((1, 1, 2049), bool))


# ------------------------------------------------------------------ cache, layout, arg-max
def test_kv_cache_append_then_read_is_concatenation(O):
    c = O.KVCache(2, 3, 64, max_seq=16)
    chunks = [O.fill_normal_f16((3, n, 64), 0, i, 1.0) for i, n in enumerate([5, 1, 1, 4])]
    for ch in chunks:
        c.update(1, ch, ch[:, ::-1].copy())
    k, v = c.active(1)
    assert np.array_equal(k, np.concatenate(chunks, 1)) and c.len == [0, 11]
    assert np.array_equal(v, np.concatenate([ch[:, ::-1] for ch in chunks], 1))
    with pytest.raises(O.SequenceTooLong):  # text_model.zig:478
        c.update(1, np.zeros((3, 6, 64), np.float16), np.zeros((3, 6, 64), np.float16))


def test_split_and_merge_heads(O):
    qkv = O.fill_normal_f16((5, 3 * 4 * 8), 0, 0, 1.0)
    q = O.split_heads(qkv, 0, 4, 8)
    v = O.split_heads(qkv, 2, 4, 8)
    assert np.array_equal(q, qkv[:, :32].reshape(5, 4, 8).transpose(1, 0, 2))
    assert np.array_equal(v, qkv[:, 64:].reshape(5, 4, 8).transpose(1, 0, 2))
    assert np.array_equal(O.merge_heads(q), qkv[:, :32])


def test_argmax_first_maximum_wins(O):
    x = O.fill_normal_f16((51200,), 0, 0, 0.9)
    assert O.argmax(x) == int(np.argmax(x.astype(np.float32)))
    x[:] = 0
    x[[40000, 7, 30000]] = 3
    assert O.argmax(x) == 7  # strict '>' (sampling.zig:265)
    x[0] = np.nan
    assert O.argmax(x) == 0  # nothing compares greater than NaN


# ------------------------------------------------------------------ model composition vs an independent torch module
def test_text_decoder_composition_against_torch(O):
    cfg = dict(vocab=300, dim=128, hidden_dim=256, n_layers=2, n_heads=2, head_dim=64, rot_dim=32, theta=10000.0, max_seq=32)
    w = O.synth_text_weights(cfg, 5)
    ids = O.fill_uniform_u32(9, 5, 50, cfg["vocab"])
    model = O.TextModel(w, cfg)
    cache = model.new_cache()
    hidden = model.text_decoder(model.text_encoder(ids), cache)
    logits = model.lm_head(hidden)

    t = {k: torch.from_numpy(v).float() for k, v in w.items()}
    F = torch.nn.functional
    x = t["wte"][torch.from_numpy(ids.astype(np.int64))]
    S, H, D, rot = len(ids), 2, 64, 32
    inv = 1.0 / (10000.0 ** (torch.arange(0, rot, 2).float() / rot))
    fr = torch.arange(S).float()[:, None] * inv[None]
    cos, sin = torch.cat([fr, fr], -1).cos(), torch.cat([fr, fr], -1).sin()

    def rope(u):  # [H,S,D]
        r, rest = u[..., :rot], u[..., rot:]
        rh = torch.cat([-r[..., rot // 2:], r[..., :rot // 2]], -1)
        return torch.cat([r * cos + rh * sin, rest], -1)

    for l in range(2):
        ln = F.layer_norm(x, (128,), t["ln_w"][l], t["ln_b"][l], eps=1e-5)
        qkv = ln @ t["Wqkv_w"][l].T + t["Wqkv_b"][l]
        q, k, v = (qkv[:, i * 128:(i + 1) * 128].reshape(S, H, D).transpose(0, 1) for i in range(3))
        a = F.scaled_dot_product_attention(rope(q), rope(k), v, is_causal=True).transpose(0, 1).reshape(S, 128)
        a = a @ t["out_proj_w"][l].T + t["out_proj_b"][l]
        m = F.gelu(ln @ t["fc1_w"][l].T + t["fc1_b"][l], approximate="tanh") @ t["fc2_w"][l].T + t["fc2_b"][l]
        x = x + a + m  # parallel block: one LayerNorm feeds both branches (text_model.zig:154-171)
    want_logits = F.layer_norm(x[-1:], (128,), t["ln_out_w"], t["ln_out_b"], eps=1e-5) @ t["linear_w"].T + t["linear_b"]
    assert O.rel_frobenius(hidden, x.half().numpy()) < 3e-3
    assert O.rel_frobenius(logits, want_logits.half().numpy()) < 5e-3


def test_vision_block_composition_against_torch(O):
    cfg = dict(dim=144, hidden_dim=304, n_layers=2, n_heads=2, head_dim=72)
    w = O.synth_vision_weights(cfg, 1)
    x0 = O.fill_normal_f16((20, 144), 1, 200, 1.0)
    got = O.VisionEncoder(w, cfg).encode(x0)
    t = {k: torch.from_numpy(v).float() for k, v in w.items()}
    F = torch.nn.functional
    x = torch.from_numpy(x0).float()
    for l in range(2):
        ln = F.layer_norm(x, (144,), t["norm1_w"][l], t["norm1_b"][l], eps=1e-5)
        qkv = ln @ t["Wqkv_w"][l] + t["Wqkv_b"][l]  # vision weights are [in, out]
        q, k, v = (qkv[:, i * 144:(i + 1) * 144].reshape(20, 2, 72).transpose(0, 1) for i in range(3))
        a = F.scaled_dot_product_attention(q, k, v).transpose(0, 1).reshape(20, 144) @ t["out_proj_w"][l] + t["out_proj_b"][l]
        x = x + a  # pre-LN ViT block (vision_model.zig:239-262)
        ln = F.layer_norm(x, (144,), t["norm2_w"][l], t["norm2_b"][l], eps=1e-5)
        x = x + F.gelu(ln @ t["fc1_w"][l] + t["fc1_b"][l], approximate="tanh") @ t["fc2_w"][l] + t["fc2_b"][l]
    want = F.layer_norm(x, (144,), t["norm_out_w"], t["norm_out_b"], eps=1e-5)
    assert O.rel_frobenius(got, want.half().numpy()) < 3e-3


def test_encode_image_composition_against_torch(O):
    """encode_image (vision_model.zig:186-229, 366-387) with torch as the second implementation: patch embedding + bias + the
    positional embedding on both crops, the blocks on all 2T rows as ONE sequence (the reference's q_len = B * M), the two crops'
    features side by side, the projection MLP.  A per-crop attention, a missing positional term on the second crop or a
    swapped concatenation fail this."""
    cfg = dict(dim=144, hidden_dim=304, n_layers=1, n_heads=2, head_dim=72)
    io = dict(patch_dim=20, tokens=9, proj_hidden=64, out_dim=24)
    w, iw = O.synth_vision_weights(cfg, 2), O.synth_vision_io_weights(cfg, io, 2, std=0.1)
    p0 = O.fill_normal_f16((18, 20), 2, 300, 1.0)
    got = O.VisionModel(w, iw, cfg, io).encode_image(p0)
    t = {k: torch.from_numpy(v).float() for k, v in {**w, **iw}.items()}
    F = torch.nn.functional
    x = torch.from_numpy(p0).float() @ t["patch_embedding_linear_w"] + t["patch_embedding_linear_b"]
    x = (x.reshape(2, 9, 144) + t["pos_embedding"]).reshape(18, 144)
    ln = F.layer_norm(x, (144,), t["norm1_w"][0], t["norm1_b"][0], eps=1e-5)
    qkv = ln @ t["Wqkv_w"][0] + t["Wqkv_b"][0]
    q, k, v = (qkv[:, i * 144:(i + 1) * 144].reshape(18, 2, 72).transpose(0, 1) for i in range(3))
    x = x + F.scaled_dot_product_attention(q, k, v).transpose(0, 1).reshape(18, 144) @ t["out_proj_w"][0] + t["out_proj_b"][0]
    ln = F.layer_norm(x, (144,), t["norm2_w"][0], t["norm2_b"][0], eps=1e-5)
    x = x + F.gelu(ln @ t["fc1_w"][0] + t["fc1_b"][0], approximate="tanh") @ t["fc2_w"][0] + t["fc2_b"][0]
    x = F.layer_norm(x, (144,), t["norm_out_w"], t["norm_out_b"], eps=1e-5)
    cat = torch.cat([x[:9], x[9:]], dim=1)
    want = F.gelu(cat @ t["proj_fc1_w"] + t["proj_fc1_b"], approximate="tanh") @ t["proj_fc2_w"] + t["proj_fc2_b"]
    assert got.shape == (9, 24)
    assert O.rel_frobenius(got, want.half().numpy()) < 3e-3


def test_generator_statistics_and_determinism(O):
    a = O.fill_normal_f16((1 << 16,), 0, 3, 1.0).astype(np.float64)
    assert abs(a.mean()) < 0.02 and abs(a.std() - 1.0) < 0.02 and np.abs(a).max() < 5.0
    assert np.array_equal(O.fill_normal_f16((100,), 0, 3, 1.0), O.fill_normal_f16((1 << 16,), 0, 3, 1.0)[:100])  # counter based
    assert not np.array_equal(O.fill_normal_f16((100,), 0, 3, 1.0), O.fill_normal_f16((100,), 0, 4, 1.0))
    ids = O.fill_uniform_u32(10000, 0, 50, 51200)
    assert ids.max() < 51200 and len(np.unique(ids)) > 9000


# ---------------------------------------------------------------------------------------------- sampling
def _sampling_logits(seed, n, spread=3.0):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal(n) * spread).astype(np.float16)


@pytest.mark.parametrize("method,kw", [
    ("multinomial", dict(temperature=1.0)), ("multinomial", dict(temperature=0.5)), ("multinomial", dict(temperature=2.5)),
    ("top_k", dict(temperature=0.5, top_k=1)), ("top_k", dict(temperature=0.7, top_k=3)), ("top_k", dict(temperature=1.0, top_k=50)),
    ("top_k", dict(temperature=3.0, top_k=5000)),  # k above the vocabulary: all of it, sorted
    ("min_p", dict(temperature=1.0, min_p=0.05)), ("min_p", dict(temperature=2.0, min_p=0.3)), ("min_p", dict(temperature=4.0, min_p=0.01)),
])
def test_sampling_is_inverse_cdf_over_the_candidates(O, method, kw):
    """Pins orc_sample_f16 against the float64 closed form: temperature, softmax, the candidate set and its order,
    the renormalisation by the candidates' total, and the strict r < cumsum rule."""
    from sampling_ref import TOL, expected

    logits = _sampling_logits(11, 1200)
    us = np.concatenate([[0.0], (np.arange(400) + 0.37) / 400, [np.float32(1.0) - np.float32(2.0 ** -24)]]).astype(np.float32)
    checked = 0
    for u in us:
        want, margin = expected(logits, method, u, **kw)
        got = O.sample(logits, method, float(u), **kw)
        if margin > TOL:
            assert got == want, (method, kw, float(u), margin)
            checked += 1
    assert checked >= 0.9 * us.size


def test_sampling_ties_keep_index_order(O):
    """Equal probabilities: top_k takes the lowest indices of the tied value first (stable sort), and walks them in
    that order; multinomial and min_p walk in index order."""
    logits = np.zeros(64, dtype=np.float16)
    top = [5, 9, 17, 18, 40, 41, 63]
    logits[top] = 2.0
    logits[[3, 30]] = 1.0
    for j in range(5):  # five equal candidates: u picks the j-th of them
        assert O.sample(logits, "top_k", (j + 0.5) / 5, temperature=1.0, top_k=5) == top[j]
    order = top + [3, 30] + [i for i in range(64) if i not in top + [3, 30]]
    w = np.exp(logits[order].astype(np.float64))
    cdf = np.cumsum(w[:12]) / w[:12].sum()
    for j in range(12):
        u = (cdf[j] + (cdf[j - 1] if j else 0.0)) / 2
        assert O.sample(logits, "top_k", u, temperature=1.0, top_k=12) == order[j]
    # min_p = 1: only the maxima survive, in index order
    for j in range(7):
        assert O.sample(logits, "min_p", (j + 0.5) / 7, temperature=1.0, min_p=1.0) == top[j]
    # nothing reaches 1.5 * max_prob: the first maximum is kept (sampling.zig:183-197)
    assert O.sample(logits, "min_p", 0.9, temperature=1.0, min_p=1.5) == 5


def test_sampling_limits_and_errors(O):
    logits = _sampling_logits(5, 300)
    best = O.argmax(logits)
    assert O.sample(logits, "greedy", 0.3, temperature=0.0) == best  # greedy never applies the temperature
    assert O.sample(logits, "top_k", 0.999, temperature=0.8, top_k=1) == best
    assert O.sample(logits, "multinomial", 0.5, temperature=1e-3) == best  # T -> 0 concentrates on the maximum
    # a flat distribution: index = floor(u * n)
    flat = np.full(250, 0.75, dtype=np.float16)
    for u in (0.0, 0.1234, 0.5, 0.998):
        assert O.sample(flat, "multinomial", u, temperature=1.0) == int(u * 250 + 1e-4)
    for bad_t in (0.0, -1.0):
        with pytest.raises(ValueError, match="InvalidTemperature"):
            O.sample(logits, "top_k", 0.5, temperature=bad_t)
    with pytest.raises(ValueError, match="top_k"):
        O.sample(logits, "top_k", 0.5, top_k=0)


# ---------------------------------------------------------------------------------------------- image -> patches
def _rne_f16(x):
    """Exact rational -> nearest binary16 (ties to even), through a double (exact enough: see the caller)."""
    return np.float16(float(x))


def test_image_patches_values_and_layout(O):
    """Pins O.image_patches: the value map against exact rational arithmetic rounded to f16 after each of the reference's
    three f16 operations (v/255, -0.5, /0.5; a quotient by 255 is never within 2^-40 of an f16 tie, so rounding the
    rational through a double is exact), and the layout against einops' statement of the rearrangement."""
    from fractions import Fraction

    import einops

    lut = []
    for v in range(256):
        a = _rne_f16(Fraction(v, 255))
        b = _rne_f16(Fraction(float(a)) - Fraction(1, 2))
        lut.append(_rne_f16(Fraction(float(b)) * 2))
    lut = np.array(lut, dtype=np.float16)
    assert lut[0] == -1.0 and lut[255] == 1.0
    rng = np.random.default_rng(0)
    for (H, W, Cn, p) in ((28, 42, 3, 14), (6, 6, 3, 2), (8, 4, 4, 4), (3, 5, 1, 1)):
        img = rng.integers(0, 256, size=(H, W, Cn), dtype=np.uint8)
        if H * W * Cn >= 256:
            img.reshape(-1)[:256] = np.arange(256, dtype=np.uint8)  # every value occurs
        got = O.image_patches(img, p)
        bchw = lut[np.stack([img, img]).transpose(0, 3, 1, 2)]
        want = einops.rearrange(bchw, "b c (h p1) (w p2) -> b (h w) (c p1 p2)", p1=p, p2=p)
        assert got.dtype == np.float16 and got.shape == want.shape
        assert np.array_equal(got.view(np.uint16), np.ascontiguousarray(want).view(np.uint16))
        # the formula of reshape_handler.zig:50-56, element by element on a few places
        T, dim = got.shape[1], got.shape[2]
        for _ in range(20):
            b, t, col = rng.integers(0, 2), rng.integers(0, T), rng.integers(0, dim)
            c, ph, pw = col // (p * p), (col // p) % p, col % p
            y, x = (t // (W // p)) * p + ph, (t % (W // p)) * p + pw
            assert got[b, t, col] == lut[img[y, x, c]]
    with pytest.raises(ValueError, match="InvalidPatchSize"):
        O.image_patches(np.zeros((15, 14, 3), dtype=np.uint8), 14)


def test_sampling_expf_against_float64(O):
    """The exp the sampling paths share with the device (the classic two-part-reduction expf, error below one ulp): pinned
    against numpy's float64 exp over the range the -88 cut-off leaves, at the reduction's branch points and at 0."""
    x = np.concatenate([np.linspace(-88, 0, 200001), -np.logspace(-8, 1.9, 50000),
                        [0.0, -0.0, -87.999, -1e-5, -0.3465, -0.3466, -1.0397, -1.0398, -6.1e-5, -6.2e-5]]).astype(np.float32)
    y = O.sampling_expf(x)
    ref = np.exp(x.astype(np.float64))
    ulp = np.spacing(np.maximum(ref, 2.0 ** -126).astype(np.float32)).astype(np.float64)
    assert np.max(np.abs(y.astype(np.float64) - ref) / ulp) < 1.0
    assert O.sampling_expf(np.float32([0.0]))[0] == 1.0
