"""GPU parity of the device sampler (moon_sample / moon_dev_sample / moon_text_sample) against the oracle's restatement
of sampling.sample (src/utils/sampling.zig:353-389).

The index is integer work decided by float32 sums over the vocabulary.  The reference takes them in sequential loops;
the device evaluates the same loops bit for bit (sample.hip: seq_prefix) on exps both sides compute with one shared
definition, so the bar is the oracle's index for EVERY draw, however close u * total lies to a boundary between two
candidates.  Beside that, every draw must be a candidate whose interval of the float64 closed form's cumulative
distribution, widened by sampling_ref.TOL of the total, holds u * total (a check that does not go through the oracle)."""
import numpy as np
import pytest

from sampling_ref import TOL, acceptable, expected

pytestmark = pytest.mark.gpu

VOCAB = 51200


def _logits(seed, n, spread=3.0, step=None):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal(n) * spread
    if step:
        x = np.round(x / step) * step  # many exactly equal logits
    return x.astype(np.float16)


def _us(seed, count):
    rng = np.random.default_rng(seed)
    us = rng.random(count).astype(np.float32)
    us[0], us[1] = 0.0, np.float32(1.0) - np.float32(2.0 ** -24)
    return us


def _check(moon, O, ctx, logits, method, us, call=None, closed_form=True, **kw):
    cfg = moon.sampling.sampling_config(method, **kw)
    for u in us:
        got = call(cfg, float(u)) if call else moon.sampling.sample(logits, cfg, float(u), ctx=ctx)
        want = O.sample(logits, method, float(u), **kw)
        _, margin = expected(logits, method, u, **kw)
        assert got == want, (method, kw, float(u), margin, got, want)
        if closed_form:
            assert acceptable(logits, method, u, got, **kw), (method, kw, float(u), margin, got, want)


@pytest.mark.parametrize("method,kw", [
    ("multinomial", dict(temperature=1.0)), ("multinomial", dict(temperature=0.5)), ("multinomial", dict(temperature=1.7)),
    ("top_k", dict(temperature=0.5, top_k=3)), ("top_k", dict(temperature=1.0, top_k=1)), ("top_k", dict(temperature=0.9, top_k=50)),
    ("top_k", dict(temperature=2.0, top_k=1024)),
    ("min_p", dict(temperature=1.0, min_p=0.05)), ("min_p", dict(temperature=2.0, min_p=0.2)), ("min_p", dict(temperature=3.0, min_p=0.01)),
])
def test_sample_full_vocabulary(moon, O, ctx, method, kw):
    # multinomial over 51200 candidates: an interval is about as wide as the rounding error of the sequential f32 running
    # sum itself, so only the same additions in the same order give the same index
    _check(moon, O, ctx, _logits(21, VOCAB), method, _us(3, 48), **kw)


@pytest.mark.parametrize("shape", ["ascending", "descending", "grid", "flat", "peaked", "holes", "tiny_first"])
def test_sequential_sums_hard_cases(moon, O, ctx, shape):
    """Rows chosen to stress the bit-exact evaluation of the reference's sequential sums: running sums that climb through
    every binade one term at a time (ascending), that stop moving early (descending), terms that are exact halves of the
    running sum's ulp again and again (grid / flat: ties to even), one term that dwarfs the rest, -inf logits (terms that
    are exactly 0), and terms in the denormal range ahead of the first large one."""
    rng = np.random.default_rng(11)
    n = VOCAB
    x = rng.standard_normal(n) * 4.0
    if shape == "ascending":
        x = np.sort(x)
    elif shape == "descending":
        x = np.sort(x)[::-1]
    elif shape == "grid":
        x = np.round(x * 2) / 2 * np.log(2.0)  # exps close to powers of two
    elif shape == "flat":
        x = np.zeros(n)
    elif shape == "peaked":
        x[n // 3] = 40.0
    elif shape == "holes":
        x[rng.random(n) < 0.5] = -np.inf
    elif shape == "tiny_first":
        x[:2000] = -80.0 + rng.random(2000) * -7.0
        x[2000] = 8.0
    logits = x.astype(np.float16)
    us = _us(5, 32)
    # the oracle's index only: on these rows the sequential f32 sums themselves are far from the float64 closed form
    # (a descending row's running sum stops moving long before the end), which is the reference's behaviour to match
    _check(moon, O, ctx, logits, "multinomial", us, closed_form=False, temperature=1.0)
    _check(moon, O, ctx, logits, "multinomial", us, closed_form=False, temperature=0.7)
    _check(moon, O, ctx, logits, "min_p", us, closed_form=False, temperature=1.0, min_p=0.02)
    _check(moon, O, ctx, logits, "top_k", us, closed_form=False, temperature=1.0, top_k=40)


@pytest.mark.parametrize("n", [1, 2, 63, 1000, 1025, 4099])
def test_sample_ragged_sizes(moon, O, ctx, n):
    logits = _logits(100 + n, n)
    us = _us(n, 24)
    _check(moon, O, ctx, logits, "multinomial", us, temperature=1.3)
    _check(moon, O, ctx, logits, "top_k", us, temperature=0.8, top_k=7)  # clamps to n where n < 7
    _check(moon, O, ctx, logits, "min_p", us, temperature=1.5, min_p=0.1)


def test_sample_kernel_without_register_copy(moon, O, ctx):
    """Rows the register-resident kernel does not take (more than 65536 logits, or a row that does not start on a 4-byte
    boundary) go to the kernel that recomputes probabilities from the logits; same bar."""
    big = _logits(41, 70001)
    us = _us(8, 12)
    _check(moon, O, ctx, big, "top_k", us, temperature=0.6, top_k=9)
    _check(moon, O, ctx, big, "min_p", us, temperature=1.4, min_p=0.05)
    _check(moon, O, ctx, big, "multinomial", us, temperature=0.8)
    logits = _logits(42, 5120)
    buf = ctx.to_device(logits)
    odd = logits[1:]  # starts 2 bytes into the allocation
    for method, kw in (("top_k", dict(temperature=0.7, top_k=20)), ("min_p", dict(temperature=1.1, min_p=0.1)), ("multinomial", dict(temperature=0.5))):
        _check(moon, O, ctx, odd, method, us, call=lambda cfg, u: moon.sampling.sample_dev(buf.offset(2), odd.size, cfg, u, ctx=ctx), **kw)


@pytest.mark.parametrize("k", [2, 5, 64, 700])
def test_top_k_among_equal_logits(moon, O, ctx, k):
    """Logits on a coarse grid: hundreds share a value, so the k-th largest falls inside a run of equal probabilities
    and the stable sort's index order decides which of them are candidates and in what order they are walked."""
    logits = _logits(7, 20000, spread=1.0, step=0.5)
    _check(moon, O, ctx, logits, "top_k", _us(k, 40), temperature=1.0, top_k=k)
    flat = np.full(3000, -2.5, dtype=np.float16)  # every probability equal: candidate j is index j
    cfg = moon.sampling.sampling_config("top_k", temperature=0.5, top_k=k)
    for j in (0, k // 2, k - 1):
        assert moon.sampling.sample(flat, cfg, (j + 0.5) / k, ctx=ctx) == j


def test_min_p_edges(moon, O, ctx):
    logits = np.zeros(5000, dtype=np.float16)
    top = [17, 18, 2500, 4999]
    logits[top] = 3.0
    cfg = moon.sampling.sampling_config("min_p", temperature=1.0, min_p=1.0)  # only the maxima survive, in index order
    for j, t in enumerate(top):
        assert moon.sampling.sample(logits, cfg, (j + 0.5) / 4, ctx=ctx) == t
    cfg = moon.sampling.sampling_config("min_p", temperature=1.0, min_p=1.5)  # nothing survives: the first maximum is kept
    assert moon.sampling.sample(logits, cfg, 0.9, ctx=ctx) == 17
    assert O.sample(logits, "min_p", 0.9, temperature=1.0, min_p=1.5) == 17


def test_sample_limits_and_errors(moon, O, ctx):
    logits = _logits(9, 3000)
    best = O.argmax(logits)
    S = moon.sampling
    assert S.sample(logits, S.sampling_config("greedy", temperature=0.0), ctx=ctx) == best  # greedy never applies the temperature
    assert S.sample(logits, S.sampling_config("top_k", temperature=0.7, top_k=1), 0.99, ctx=ctx) == best
    assert S.sample(logits, S.sampling_config("multinomial", temperature=1e-3), 0.5, ctx=ctx) == best
    small = logits[:800]
    assert S.sample(small, S.sampling_config("top_k", temperature=1.0, top_k=5000), 0.0, ctx=ctx) == O.argmax(small)  # k clamps to n
    with pytest.raises(moon.context.InvalidArgument, match="1024"):
        S.sample(logits, S.sampling_config("top_k", top_k=2000), 0.5, ctx=ctx)  # more candidates than the device sorts
    with pytest.raises(moon.context.InvalidArgument, match="top_k of 0"):
        S.sample(logits, S.sampling_config("top_k", top_k=0), 0.5, ctx=ctx)
    for bad_t in (0.0, -2.0, float("nan")):
        with pytest.raises(moon.context.InvalidTemperature):
            S.sample(logits, S.sampling_config("min_p", temperature=bad_t), 0.5, ctx=ctx)
    with pytest.raises(moon.context.InvalidArgument):
        S.sample(logits, moon._lib.SamplingConfig(9, 1.0, 3, 0.05), 0.5, ctx=ctx)
    with pytest.raises(moon.context.InvalidArgument, match="EmptyTensor"):
        S.sample(np.zeros(0, dtype=np.float16), S.sampling_config("top_k"), 0.5, ctx=ctx)


def test_dev_sample_equals_host_pointer_call(moon, O, ctx):
    logits = _logits(33, VOCAB)
    buf = ctx.to_device(logits)
    for method, kw in (("top_k", dict(temperature=0.6, top_k=40)), ("min_p", dict(temperature=1.2, min_p=0.05)),
                       ("multinomial", dict(temperature=0.9)), ("greedy", {})):
        cfg = moon.sampling.sampling_config(method, **kw)
        for u in _us(1, 6):
            assert moon.sampling.sample_dev(buf.ptr, logits.size, cfg, float(u), ctx=ctx) == moon.sampling.sample(logits, cfg, float(u), ctx=ctx)


SMALL_TEXT = dict(vocab=1000, dim=256, hidden_dim=1024, n_layers=3, n_heads=4, head_dim=64, rot_dim=32, theta=10000.0, max_seq=128)


@pytest.mark.parametrize("method,kw", [("top_k", dict(temperature=0.8, top_k=5)), ("min_p", dict(temperature=1.5, min_p=0.05)),
                                       ("multinomial", dict(temperature=1.0))])
def test_text_sample_loop_is_lm_head_sample_forward(moon, O, ctx, method, kw):
    """moon_text_sample (everything on the device) against the same loop driven from the host, one call per stage:
    logits of the last position -> moon_sample -> forward([token]).  The two run different decode kernels, whose
    logits agree to the parity tolerance but not to the bit, so a step's tokens must agree wherever the draw is clear
    of a candidate boundary (by 1e-3 of the total here); the comparison ends at the first step that is not."""
    w = O.synth_text_weights(SMALL_TEXT, 4)
    mcfg = moon.text_model.make_config(vocab=SMALL_TEXT["vocab"], dim=SMALL_TEXT["dim"], hidden_dim=SMALL_TEXT["hidden_dim"],
                                       n_layers=SMALL_TEXT["n_layers"], n_heads=SMALL_TEXT["n_heads"], max_seq=SMALL_TEXT["max_seq"])
    dev = moon.text_model.TextModel(mcfg, weights=w, ctx=ctx)
    ids = O.fill_uniform_u32(20, 0, 77, SMALL_TEXT["vocab"])
    cfg = moon.sampling.sampling_config(method, **kw)
    us = _us(12, 24)[2:]
    dev.forward(ids)
    got = dev.sample(cfg, us).tolist()
    assert dev.position == 20 + len(us)
    dev.reset()
    dev.forward(ids)
    compared = 0
    for step, u in enumerate(us):
        logits = dev.logits()
        tok = moon.sampling.sample(logits, cfg, float(u), ctx=ctx)
        _, margin = expected(logits, method, u, **kw)
        if got[step] != tok:
            assert margin < 1e-3, (step, got[step], tok, margin)
            break
        compared += 1
        dev.forward([tok])
    print(f"{method}: {compared}/{len(us)} steps compared")
    assert compared >= len(us) // 2
    # the greedy method runs the arg-max loop
    dev.reset()
    dev.forward(ids)
    a = dev.sample(moon.sampling.sampling_config("greedy"), np.zeros(10, dtype=np.float32)).tolist()
    dev.reset()
    dev.forward(ids)
    assert a == dev.greedy(10).tolist()
    dev.close()


def test_text_sample_matches_oracle_model(moon, O, ctx):
    """End to end against the oracle: its decoder's logits + its sampler, step by step on the device's own tokens."""
    w = O.synth_text_weights(SMALL_TEXT, 5)
    mcfg = moon.text_model.make_config(vocab=SMALL_TEXT["vocab"], dim=SMALL_TEXT["dim"], hidden_dim=SMALL_TEXT["hidden_dim"],
                                       n_layers=SMALL_TEXT["n_layers"], n_heads=SMALL_TEXT["n_heads"], max_seq=SMALL_TEXT["max_seq"])
    ref, dev = O.TextModel(w, SMALL_TEXT), moon.text_model.TextModel(mcfg, weights=w, ctx=ctx)
    ids = O.fill_uniform_u32(16, 0, 78, SMALL_TEXT["vocab"])
    kw = dict(temperature=0.7, top_k=4)
    us = _us(13, 14)[2:]
    dev.forward(ids)
    got = dev.sample(moon.sampling.sampling_config("top_k", **kw), us).tolist()
    cache = ref.new_cache()
    h = ref.text_decoder(ref.text_encoder(ids), cache)
    compared = 0
    for step, u in enumerate(us):
        logits = ref.lm_head(h[-1:]).reshape(-1)
        want = O.sample(logits, "top_k", float(u), **kw)
        _, margin = expected(logits, "top_k", u, **kw)
        if got[step] != want:
            assert margin < 5e-3, (step, got[step], want, margin)  # f16 logits differ by up to 1e-3 relative between the two
            break
        compared += 1
        h = ref.text_decoder(ref.text_encoder([want]), cache)
    print(f"{compared}/{len(us)} steps compared")
    assert compared >= len(us) // 2
    dev.close()


def test_sample_f32_row(moon, O, ctx):
    """sampling.sample's own argument type (sample(tensor: *Tensor(f32), ...), sampling.zig:353-358): f32 logits that are not
    f16 values go through the same arithmetic, and an f16 row cast to f32 (what moondream.zig:335 hands over) gives the
    index of the f16 entry point; argmax(f32, ...) keeps the first maximum."""
    rng = np.random.default_rng(77)
    x = (rng.standard_normal(VOCAB) * 2.5).astype(np.float32)
    us = _us(9, 24)
    for method, kw in (("multinomial", dict(temperature=0.9)), ("top_k", dict(temperature=0.5, top_k=3)), ("min_p", dict(temperature=1.2, min_p=0.05))):
        cfg = moon.sampling.sampling_config(method, **kw)
        for u in us:
            assert moon.sampling.sample_f32(x, cfg, float(u), ctx=ctx) == O.sample_f32(x, method, float(u), **kw), (method, float(u))
    h = _logits(78, 5000)
    cfg = moon.sampling.sampling_config("top_k", temperature=0.7, top_k=5)
    for u in us:
        assert moon.sampling.sample_f32(h.astype(np.float32), cfg, float(u), ctx=ctx) == moon.sampling.sample(h, cfg, float(u), ctx=ctx)
    greedy = moon.sampling.sampling_config("greedy")
    x[[100, 40000]] = x.max() + 1.0
    assert moon.sampling.sample_f32(x, greedy, 0.0, ctx=ctx) == 100 == moon.sampling.argmax_f32(x, ctx=ctx) == O.sample_f32(x, "greedy", 0.0)


def _fixed_logits_model(moon, O, ctx, logits, max_seq=128):
    """A session whose LM head returns `logits` at every step whatever the hidden state is: a zero matrix and the row as the bias."""
    cfg = dict(SMALL_TEXT, vocab=logits.size, max_seq=max_seq)
    w = O.synth_text_weights(cfg, 6)
    w["linear_w"] = np.zeros_like(w["linear_w"])
    w["linear_b"] = np.ascontiguousarray(logits, dtype=np.float16)
    mcfg = moon.text_model.make_config(vocab=cfg["vocab"], dim=cfg["dim"], hidden_dim=cfg["hidden_dim"], n_layers=cfg["n_layers"],
                                       n_heads=cfg["n_heads"], max_seq=cfg["max_seq"])
    return moon.text_model.TextModel(mcfg, weights=w, ctx=ctx)


def _boundary_us(O, logits, kw, count, seed):
    """Draws on and next to the candidate boundaries (float32 neighbours of the closed form's cumulative sums), then random ones."""
    x = logits.astype(np.float64) / kw["temperature"]
    order = np.lexsort((np.arange(x.size), -x))[: kw["top_k"]]
    p = np.exp(x[order] - x.max())
    cum = np.cumsum(p) / p.sum()
    us = []
    for c in cum[:-1]:
        c32 = np.float32(c)
        us += [c32, np.nextafter(c32, np.float32(0)), np.nextafter(c32, np.float32(1)), np.float32(c * (1 - 3e-6)), np.float32(c * (1 + 3e-6))]
    us += list(_us(seed, count))
    return np.array([u for u in us if 0.0 <= u < 1.0], dtype=np.float32)[:count]


@pytest.mark.parametrize("kw", [dict(temperature=0.5, top_k=3), dict(temperature=1.0, top_k=1), dict(temperature=0.7, top_k=2),
                                dict(temperature=1.3, top_k=3)])
def test_top_k_decided_in_the_lm_head_kernel(moon, O, ctx, kw):
    """The sampled loop with top_k <= 3 decides the token in the LM-head launch wherever it can prove the choice from the four
    largest logits, and leaves the rest to sample_kernel.  Rows with the logits fixed (so every step draws from the same
    row): the oracle's index for every draw, among them draws on the candidate boundaries, ties inside the k, ties across
    the edge of the k, -inf logits, a row whose exps all but vanish; and the same ids as the loop that runs sample_kernel
    at every step (MOON_SAMPLE_SEPARATE)."""
    import os
    cfg = moon.sampling.sampling_config("top_k", **kw)
    n = 1000
    rows = {"normal": _logits(21, n), "steep": _logits(22, n, spread=30.0)}
    tie_in = _logits(23, n)
    tie_in[[700, 30]] = tie_in.max() + np.float16(1.0)  # two equal leaders: the lower index first
    rows["tie_inside"] = tie_in
    tie_edge = _logits(24, n)
    top = np.float16(tie_edge.max() + np.float16(2.0))
    tie_edge[[900, 5, 400, 77, 650]] = [top, top - np.float16(0.5), top - np.float16(1), top - np.float16(1), top - np.float16(1)]
    rows["tie_across_the_edge"] = tie_edge
    all_eq = np.full(n, 1.5, dtype=np.float16)
    rows["all_equal"] = all_eq
    ninf = _logits(25, n)
    ninf[::3] = -np.inf
    rows["minus_inf"] = ninf
    far = np.full(n, -200.0, dtype=np.float16)
    far[[10, 20, 30, 40]] = [50.0, -60.0, -61.0, -200.0]
    rows["vanishing"] = far
    for name, logits in rows.items():
        dev = _fixed_logits_model(moon, O, ctx, logits)
        us = _boundary_us(O, logits, kw, 60, 31)
        dev.forward(np.array([1, 2, 3], dtype=np.uint32))
        got = dev.sample(cfg, us).tolist()
        want = [O.sample(logits, "top_k", float(u), **kw) for u in us]
        assert got == want, (name, kw)
        os.environ["MOON_SAMPLE_SEPARATE"] = "1"
        try:
            dev.reset()
            dev.forward(np.array([1, 2, 3], dtype=np.uint32))
            assert dev.sample(cfg, us).tolist() == got, (name, kw)
        finally:
            del os.environ["MOON_SAMPLE_SEPARATE"]
        dev.close()


def test_top_k_in_the_lm_head_kernel_full_size(moon, O, ctx):
    """The reference CLI's default sampler (top_k 3 at temperature 0.5) on the full-size decoder: the loop that decides in the
    LM-head launch and the loop that runs sample_kernel at every step give the same 48 ids, and generate() stops both at
    the same token."""
    import os
    dev = moon.text_model.TextModel(moon.text_model.default_config(), seed=0, std=0.02, ctx=ctx)
    ids = O.fill_uniform_u32(300, 0, 50, 51200)
    cfg = moon.sampling.sampling_config("top_k", temperature=0.5, top_k=3)
    us = _us(41, 48)
    dev.forward(ids)
    got = dev.sample(cfg, us).tolist()
    dev.reset()
    dev.forward(ids)
    stopped = dev.generate(48, got[20], cfg, us).tolist()
    assert stopped == got[: got.index(got[20])]
    os.environ["MOON_SAMPLE_SEPARATE"] = "1"
    try:
        dev.reset()
        dev.forward(ids)
        assert dev.sample(cfg, us).tolist() == got
    finally:
        del os.environ["MOON_SAMPLE_SEPARATE"]
    dev.close()


@pytest.mark.parametrize("method,kw", [("multinomial", dict(temperature=1.0)), ("min_p", dict(temperature=1.2, min_p=0.02))])
def test_quick_walk_never_differs_from_the_exact_walk_next_to_a_boundary(moon, O, ctx, method, kw):
    """sample_kernel first takes its sums in whatever order is fast and keeps the answer only if the draw stays (6 m + 32) 2^-24
    of the total away from the running sums around the chosen candidate (m candidates); otherwise it evaluates the
    reference's sequential loops bit for bit.  Draws placed on the candidate boundaries of the float64 closed form and at
    0.5 and 1.5 times that distance on either side: whichever path answers, the index is the oracle's (whose loops are the
    sequential ones)."""
    n = 1000
    logits = _logits(51, n, spread=2.0)
    x = logits.astype(np.float64) / kw["temperature"]
    p = np.exp(x - x.max())
    p /= p.sum()
    cand = p >= kw["min_p"] * p.max() if method == "min_p" else np.ones(n, bool)
    m = int(cand.sum())
    cum = np.cumsum(np.where(cand, p, 0.0))
    bounds = (cum / cum[-1])[cand][:-1]
    if bounds.size > 150:
        bounds = bounds[:: bounds.size // 150]
    tol = (6.0 * m + 32.0) * 2.0 ** -24
    us = np.concatenate([bounds + f * tol for f in (-1.5, -0.5, 0.0, 0.5, 1.5)]).astype(np.float32)
    us = us[(us >= 0) & (us < 1)]
    assert us.size >= 40, (m, bounds.size)
    _check(moon, O, ctx, logits, method, us, closed_form=False, **kw)


@pytest.mark.parametrize("spread,step", [(3.0, None), (3.0, 0.25), (0.02, None)])
def test_top_k_in_the_lm_head_kernel_full_vocabulary(moon, O, ctx, spread, step):
    """The same decision at the real vocabulary (51200 logits over 1024 workgroups, 12 or 13 per wavefront): rows with the
    logits fixed, 100 draws each, the oracle's index on every draw.  A row quantised to steps of 0.25 has dozens of equal
    logits at the top (ties inside the three and across their edge: the full evaluation has to take over), a row of spread
    0.02 has its largest logits within a few f16 steps of each other."""
    logits = _logits(61, VOCAB, spread=spread, step=step)
    kw = dict(temperature=0.5, top_k=3)
    cfg = moon.sampling.sampling_config("top_k", **kw)
    dev = _fixed_logits_model(moon, O, ctx, logits)
    us = _boundary_us(O, logits, kw, 100, 62)
    dev.forward(np.array([5, 6], dtype=np.uint32))
    got = dev.sample(cfg, us).tolist()
    want = [O.sample(logits, "top_k", float(u), **kw) for u in us]
    assert got == want
    dev.close()
