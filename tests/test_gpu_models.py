"""GPU parity of the device-resident decoder and vision-encoder sessions against the oracle's model composition."""
import numpy as np
import pytest

from conftest import TOL

pytestmark = pytest.mark.gpu

SMALL_TEXT = dict(vocab=1000, dim=256, hidden_dim=1024, n_layers=3, n_heads=4, head_dim=64, rot_dim=32, theta=10000.0, max_seq=128)


def _text_pair(moon, O, ctx, cfg, seed=0):
    w = O.synth_text_weights(cfg, seed)
    mcfg = moon.text_model.make_config(vocab=cfg["vocab"], dim=cfg["dim"], hidden_dim=cfg["hidden_dim"], n_layers=cfg["n_layers"],
                                       n_heads=cfg["n_heads"], max_seq=cfg["max_seq"])
    return O.TextModel(w, cfg), moon.text_model.TextModel(mcfg, weights=w, ctx=ctx)


def test_text_prefill_hidden_and_logits(moon, O, ctx):
    ref, dev = _text_pair(moon, O, ctx, SMALL_TEXT)
    ids = O.fill_uniform_u32(40, 0, 50, SMALL_TEXT["vocab"])
    cache = ref.new_cache()
    h_ref = ref.text_decoder(ref.text_encoder(ids), cache)
    dev.forward(ids)
    assert dev.position == 40
    assert O.rel_frobenius(dev.hidden(40), h_ref) <= TOL
    assert O.rel_frobenius(dev.logits().reshape(1, -1), ref.lm_head(h_ref)) <= TOL
    dev.close()


def test_text_greedy_ids_match_oracle(moon, O, ctx):
    ref, dev = _text_pair(moon, O, ctx, SMALL_TEXT)
    ids = O.fill_uniform_u32(24, 0, 51, SMALL_TEXT["vocab"])
    want, margins, _ = ref.greedy(ids, 32)
    dev.forward(ids)
    got = dev.greedy(32).tolist()
    print("min top-2 margin over the steps:", min(margins))
    assert got == want
    assert dev.position == 24 + 32
    dev.close()


def test_text_decode_equals_prefill(moon, O, ctx):
    """Feeding tokens one at a time (decode kernels) gives the same next-token logits as one prefill (GEMM kernels)."""
    _, dev = _text_pair(moon, O, ctx, SMALL_TEXT)
    ids = O.fill_uniform_u32(12, 0, 52, SMALL_TEXT["vocab"])
    dev.forward(ids)
    a = dev.logits()
    dev.reset()
    for t in ids:
        dev.forward([t])
    b = dev.logits()
    assert O.rel_frobenius(a.reshape(1, -1), b.reshape(1, -1)) <= TOL
    dev.close()


def test_text_errors(moon, O, ctx):
    _, dev = _text_pair(moon, O, ctx, SMALL_TEXT)
    with pytest.raises(moon.TokenIdOutOfBounds):  # text_model.zig:125-128
        dev.forward([SMALL_TEXT["vocab"]])
    with pytest.raises(moon.SequenceTooLong):  # text_model.zig:478
        dev.forward(np.zeros(SMALL_TEXT["max_seq"] + 1, dtype=np.uint32))
    dev.close()


def test_device_synthetic_weights_match_host_generator(moon, O, ctx):
    """The on-device random-init decoder equals the one built from the host generator (same seed/streams)."""
    cfg = SMALL_TEXT
    ref, dev_host = _text_pair(moon, O, ctx, cfg, seed=3)
    mcfg = moon.text_model.make_config(vocab=cfg["vocab"], dim=cfg["dim"], hidden_dim=cfg["hidden_dim"], n_layers=cfg["n_layers"],
                                       n_heads=cfg["n_heads"], max_seq=cfg["max_seq"])
    dev_syn = moon.text_model.TextModel(mcfg, seed=3, std=0.02, ctx=ctx)
    ids = O.fill_uniform_u32(9, 0, 53, cfg["vocab"])
    dev_host.forward(ids)
    dev_syn.forward(ids)
    assert np.array_equal(dev_host.logits(), dev_syn.logits())
    dev_host.close()
    dev_syn.close()


SMALL_VISION = dict(dim=144, hidden_dim=304, n_layers=3, n_heads=2, head_dim=72)


def test_vision_encoder_blocks(moon, O, ctx):
    cfg = SMALL_VISION
    w = O.synth_vision_weights(cfg, 0)
    ref = O.VisionEncoder(w, cfg)
    mcfg = moon.vision_model.make_config(**cfg)
    dev = moon.vision_model.VisionModel(mcfg, weights=w, ctx=ctx)
    x = O.fill_normal_f16((50, cfg["dim"]), 0, 200, 1.0)
    assert O.rel_frobenius(dev.encode(x), ref.encode(x)) <= TOL
    dev_syn = moon.vision_model.VisionModel(mcfg, seed=0, std=0.02, ctx=ctx)
    assert np.array_equal(dev_syn.encode(x), dev.encode(x))
    dev.close()
    dev_syn.close()


def test_vision_one_full_size_block(moon, O, ctx):
    """One block at the real SigLIP shape (729 x 1152, 16 heads x 72, MLP 4304)."""
    cfg = dict(dim=1152, hidden_dim=4304, n_layers=1, n_heads=16, head_dim=72)
    w = O.synth_vision_weights(cfg, 0)
    dev = moon.vision_model.VisionModel(moon.vision_model.make_config(**cfg), weights=w, ctx=ctx)
    x = O.fill_normal_f16((729, 1152), 0, 200, 1.0)
    assert O.rel_frobenius(dev.encode(x), O.VisionEncoder(w, cfg).encode(x)) <= TOL
    dev.close()


def test_vision_encode_image_small(moon, O, ctx):
    """encode_image around the encoder: patch embedding (k = 20, padded to 32 on the device) + positional embedding, the
    encoder on both crops as one sequence, concatenation, projection MLP; from arrays and from seeded synthetic weights."""
    cfg = SMALL_VISION
    io = dict(patch_dim=20, tokens=27, proj_hidden=96, out_dim=40)
    w, iw = O.synth_vision_weights(cfg, 0), O.synth_vision_io_weights(cfg, io, 0)
    ref = O.VisionModel(w, iw, cfg, io)
    mcfg, mio = moon.vision_model.make_config(**cfg), moon.vision_model.make_io_config(**io)
    dev = moon.vision_model.VisionModel(mcfg, weights=w, ctx=ctx)
    patches = O.fill_normal_f16((2 * io["tokens"], io["patch_dim"]), 0, 300, 1.0)
    with pytest.raises(moon.MoonError):
        dev.encode_image(patches)  # nothing attached yet
    dev.attach_io(mio, weights=iw)
    got = dev.encode_image(patches)
    assert got.shape == (io["tokens"], io["out_dim"])
    assert O.rel_frobenius(got, ref.encode_image(patches)) <= TOL
    dev_syn = moon.vision_model.VisionModel(mcfg, seed=0, std=0.02, ctx=ctx)
    dev_syn.attach_io(mio, seed=0, std=0.02)
    assert np.array_equal(dev_syn.encode_image(patches), got)
    dev.close()
    dev_syn.close()


def test_vision_encode_image_full_size_front_and_back(moon, O, ctx):
    """The front and back ends at the real shapes (1458 x 588 -> 1152 with the 729 x 1152 positional embedding; 729 x 2304 ->
    8192 -> 2048) around one encoder block."""
    cfg = dict(dim=1152, hidden_dim=4304, n_layers=1, n_heads=16, head_dim=72)
    io = O.VISION_IO_CFG
    w, iw = O.synth_vision_weights(cfg, 0), O.synth_vision_io_weights(cfg, io, 0)
    dev = moon.vision_model.VisionModel(moon.vision_model.make_config(**cfg), weights=w, ctx=ctx)
    dev.attach_io(weights=iw)
    patches = O.fill_normal_f16((2 * io["tokens"], io["patch_dim"]), 0, 300, 1.0)
    assert O.rel_frobenius(dev.encode_image(patches), O.VisionModel(w, iw, cfg, io).encode_image(patches)) <= TOL
    dev.close()


@pytest.mark.parametrize("shape,p", [((378, 378, 3), 14), ((28, 42, 3), 14), ((8, 4, 4), 4), ((3, 5, 1), 1), ((6, 6, 3), 2)])
def test_image_patches_bit_exact(moon, O, ctx, shape, p):
    """u8 image -> normalised f16 patches: integer / f16 element-wise work, bit-exact against the oracle."""
    rng = np.random.default_rng(shape[0])
    img = rng.integers(0, 256, size=shape, dtype=np.uint8)
    if img.size >= 256:
        img.reshape(-1)[:256] = np.arange(256, dtype=np.uint8)
    got = moon.vision_model.image_patches(img, p, ctx=ctx)
    want = O.image_patches(img, p)
    assert got.shape == want.shape
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_image_patches_errors(moon, ctx):
    with pytest.raises(moon.context.InvalidTensorDimension, match="InvalidPatchSize"):
        moon.vision_model.image_patches(np.zeros((15, 14, 3), dtype=np.uint8), 14, ctx=ctx)
    with pytest.raises(moon.context.InvalidTensorDimension):
        moon.vision_model.image_patches(np.zeros((14, 14, 3), dtype=np.uint8), 0, ctx=ctx)


def test_vision_encode_image_from_resized_u8(moon, O, ctx):
    """encode_image from the resized image on: the same bits as encode_image on the oracle's patches (the preprocessing is
    exact and the rest is the same kernels), and the parity tolerance against the oracle's whole composition."""
    cfg = SMALL_VISION
    io = dict(patch_dim=12, tokens=9, proj_hidden=96, out_dim=40)  # 3 x 3 patches of 2 x 2 RGB pixels: a 6 x 6 image
    w, iw = O.synth_vision_weights(cfg, 1), O.synth_vision_io_weights(cfg, io, 1)
    dev = moon.vision_model.VisionModel(moon.vision_model.make_config(**cfg), weights=w, ctx=ctx)
    dev.attach_io(moon.vision_model.make_io_config(**io), weights=iw)
    img = np.random.default_rng(3).integers(0, 256, size=(6, 6, 3), dtype=np.uint8)
    patches = O.image_patches(img, 2).reshape(2 * io["tokens"], io["patch_dim"])
    got = dev.encode_image_u8(img)
    assert np.array_equal(got, dev.encode_image(patches))
    assert O.rel_frobenius(got, O.VisionModel(w, iw, cfg, io).encode_image(patches)) <= TOL
    with pytest.raises(ValueError):
        dev.encode_image_u8(img[:4])
    dev.close()
    # a token count that is not a square grid is refused by the library
    io_bad = dict(patch_dim=12, tokens=10, proj_hidden=96, out_dim=40)
    dev = moon.vision_model.VisionModel(moon.vision_model.make_config(**cfg), seed=0, std=0.02, ctx=ctx)
    dev.attach_io(moon.vision_model.make_io_config(**io_bad), seed=0, std=0.02)
    with pytest.raises(moon.context.InvalidTensorDimension):
        dev.ctx.check(dev.ctx.lib.moon_vision_encode_image_u8(dev.handle, img.ctypes.data, np.empty((10, 40), np.float16).ctypes.data))
    dev.close()


def test_vision_encode_image_u8_full_size_front(moon, O, ctx):
    """The real 378 x 378 x 3 image through one encoder block with the real front and back ends."""
    cfg = dict(dim=1152, hidden_dim=4304, n_layers=1, n_heads=16, head_dim=72)
    io = O.VISION_IO_CFG
    w, iw = O.synth_vision_weights(cfg, 0), O.synth_vision_io_weights(cfg, io, 0)
    dev = moon.vision_model.VisionModel(moon.vision_model.make_config(**cfg), weights=w, ctx=ctx)
    dev.attach_io(weights=iw)
    img = np.random.default_rng(5).integers(0, 256, size=(378, 378, 3), dtype=np.uint8)
    patches = O.image_patches(img, 14).reshape(2 * io["tokens"], io["patch_dim"])
    got = dev.encode_image_u8(img)
    assert np.array_equal(got, dev.encode_image(patches))
    assert O.rel_frobenius(got, O.VisionModel(w, iw, cfg, io).encode_image(patches)) <= TOL
    dev.close()


def _all_modes(dev, ids, n_steps):
    """(tokens, logits, position) for decode modes 1 (persistent kernel), 0 (one kernel per layer where the device supports
    it), 2 (three kernels per layer) and 3 (two kernels per layer)."""
    out = []
    for mode in (1, 0, 2, 3):
        dev.reset()
        dev.set_decode_mode(mode)
        dev.forward(ids)
        toks = dev.greedy(n_steps).tolist()
        out.append((toks, dev.logits().copy(), dev.position))
    return out


def test_persistent_decode_kernel_equals_per_op_kernels_small(moon, O, ctx):
    """The one-launch greedy loop and the kernel-per-op loop share arithmetic and summation order: same bits."""
    _, dev = _text_pair(moon, O, ctx, SMALL_TEXT)
    ids = O.fill_uniform_u32(20, 0, 54, SMALL_TEXT["vocab"])
    (t1, l1, p1), *others = _all_modes(dev, ids, 40)
    assert p1 == 60
    for t, l, p in others:
        assert t == t1 and p == p1
        assert np.array_equal(l.view(np.uint16), l1.view(np.uint16))
    dev.close()


def test_persistent_decode_kernel_equals_per_op_kernels_full_size(moon, O, ctx):
    """Same check on the real decoder shape (24 x 2048, random-init on the device)."""
    dev = moon.text_model.TextModel(moon.text_model.default_config(), seed=0, std=0.02, ctx=ctx)
    ids = O.fill_uniform_u32(100, 0, 50, 51200)
    (t1, l1, _), *others = _all_modes(dev, ids, 12)
    for t, l, _ in others:
        assert t == t1
        assert np.array_equal(l.view(np.uint16), l1.view(np.uint16))
    dev.close()


def test_sessions_built_from_a_moondream_bin_file(moon, O, ctx, tmp_path):
    """Weights written in the reference's file layout, mapped by the library's reader and uploaded from the mapping: the
    decoder and the vision encoder give the same bits as when built from in-memory arrays, and match the oracle."""
    cfg = SMALL_TEXT
    vcfg = dict(dim=128, hidden_dim=256, n_layers=2, n_heads=2, head_dim=64)
    tw, vw = O.synth_text_weights(cfg, 5), O.synth_vision_weights(vcfg, 6)
    tensors = O.text_bin_tensors(tw)
    tensors.update(O.vision_bin_tensors(vw))
    path = str(tmp_path / "moondream.bin")
    O.write_moondream_bin(path, tensors)
    mcfg = moon.text_model.make_config(vocab=cfg["vocab"], dim=cfg["dim"], hidden_dim=cfg["hidden_dim"], n_layers=cfg["n_layers"],
                                       n_heads=cfg["n_heads"], max_seq=cfg["max_seq"])
    mvcfg = moon.vision_model.make_config(**vcfg)
    ids = O.fill_uniform_u32(17, 0, 9, cfg["vocab"])
    x = O.fill_normal_f16((50, vcfg["dim"]), 0, 8, 1.0)
    with moon.weights.BinFile(path) as f:
        from_file = moon.text_model.TextModel(mcfg, weights=f, ctx=ctx)
        vis_file = moon.vision_model.VisionModel(mvcfg, weights=f, ctx=ctx)
    # the mapping is closed: the sessions own device copies
    from_mem = moon.text_model.TextModel(mcfg, weights=tw, ctx=ctx)
    out = []
    for dev in (from_file, from_mem):
        dev.forward(ids)
        out.append((dev.logits().copy(), dev.greedy(8).tolist()))
        dev.close()
    assert np.array_equal(out[0][0].view(np.uint16), out[1][0].view(np.uint16)) and out[0][1] == out[1][1]
    ref = O.TextModel(tw, cfg)
    cache = ref.new_cache()
    h = ref.text_decoder(ref.text_encoder(ids), cache)
    assert O.rel_frobenius(out[0][0].reshape(1, -1), ref.lm_head(h).reshape(1, -1)) <= TOL
    assert O.rel_frobenius(vis_file.encode(x), O.VisionEncoder(vw, vcfg).encode(x)) <= TOL
    vis_file.close()


@pytest.mark.parametrize("case", ["ties", "nan_at_0", "nan_elsewhere", "all_neg_inf", "max_is_last"])
def test_greedy_argmax_rules_in_every_mode(moon, O, ctx, case):
    """The greedy loop's arg-max (fused into the LM-head launch in modes 0, 2, 3; inside the persistent kernel in mode 1)
    follows sampling.argmax (sampling.zig:257-273): start from logits[0], move on "greater" only.  The LM-head matrix is
    zero here, so the logits are exactly the crafted bias vector and every step must return the oracle's arg-max of it."""
    cfg = dict(SMALL_TEXT)
    w = O.synth_text_weights(cfg, 0)
    V = cfg["vocab"]
    b = O.fill_normal_f16((V,), 0, 77, 1.0).astype(np.float16)
    if case == "ties":  # the maximum occurs four times, far apart (different workgroups and wavefronts see it)
        b[[3, 250, 251, 999]] = np.float16(9.0)
    elif case == "nan_at_0":  # a NaN at index 0 is never displaced
        b[0] = np.float16(np.nan)
        b[17] = np.float16(np.inf)
    elif case == "nan_elsewhere":  # ... and a NaN anywhere else is never selected
        b[5] = np.float16(np.nan)
        b[600] = np.float16(np.nan)
    elif case == "all_neg_inf":
        b[:] = np.float16(-np.inf)
    elif case == "max_is_last":
        b[V - 1] = np.float16(50.0)
    w["linear_w"] = np.zeros_like(w["linear_w"])
    w["linear_b"] = b
    want = O.argmax(b)
    mcfg = moon.text_model.make_config(vocab=V, dim=cfg["dim"], hidden_dim=cfg["hidden_dim"], n_layers=cfg["n_layers"],
                                       n_heads=cfg["n_heads"], max_seq=cfg["max_seq"])
    dev = moon.text_model.TextModel(mcfg, weights=w, ctx=ctx)
    ids = O.fill_uniform_u32(5, 0, 60, V)
    for mode in (0, 1, 2, 3):
        dev.reset()
        dev.set_decode_mode(mode)
        dev.forward(ids)
        assert dev.greedy(3).tolist() == [want] * 3, (case, mode)
        assert dev.position == 5 + 3
    dev.close()


def test_session_recovers_after_a_failed_wait(moon, O, ctx):
    """The error word of the fused decode kernels raised from the host (every kernel still runs to its end; a workgroup that
    has to poll for long leaves early, as after an expired wait): the call fails with HipError, the session refuses work
    until reset, and after reset it decodes exactly like a fresh session."""
    dev = moon.text_model.TextModel(moon.text_model.default_config(), seed=0, std=0.02, ctx=ctx)
    ids = O.fill_uniform_u32(64, 0, 50, 51200)
    dev.forward(ids)
    want = dev.greedy(6).tolist()
    want_logits = dev.logits().copy()
    dev.reset()
    dev.forward(ids)
    ctx.check(ctx.lib.moon_text_debug_raise_wait_error(dev.handle))
    with pytest.raises(moon.context.HipError):
        dev.greedy(3)
    with pytest.raises(moon.context.HipError):
        dev.greedy(1)  # refused until reset
    with pytest.raises(moon.context.HipError):
        dev.forward(ids[:2])
    dev.reset()
    assert dev.position == 0
    dev.forward(ids)
    assert dev.greedy(6).tolist() == want
    assert np.array_equal(dev.logits().view(np.uint16), want_logits.view(np.uint16))
    # and once more through the two-kernel path and the streaming kernel, whose error words are raised by the same hook
    for mode in (3, 4):
        dev.reset()
        dev.set_decode_mode(mode)
        dev.forward(ids)
        ctx.check(ctx.lib.moon_text_debug_raise_wait_error(dev.handle))
        with pytest.raises(moon.context.HipError):
            dev.greedy(2)
        dev.reset()
        dev.forward(ids)
        assert dev.greedy(6).tolist() == want, f"decode mode {mode} after a reset"
    dev.close()


def test_streaming_decode_kernel_against_the_per_layer_kernels(moon, O, ctx):
    """Decode mode 4 (one launch for the whole greedy loop, weights streamed through LDS rings, workgroups exchanging q/k/v,
    attention partials, partial sums and the hidden state through tagged words): same ids as the per-layer kernels, hidden
    state and logits within the end-to-end bound of theirs (out_proj and fc2 are summed in another order), single steps,
    a run up to the last cache position, and interleaving with forward() calls."""
    dev = moon.text_model.TextModel(moon.text_model.default_config(), seed=0, std=0.02, ctx=ctx)
    ids = O.fill_uniform_u32(50, 0, 50, 51200)
    dev.forward(ids)
    want = dev.greedy(20).tolist()
    want_hidden, want_logits = dev.hidden(1).copy(), dev.logits().copy()
    dev.reset()
    dev.set_decode_mode(4)
    dev.forward(ids)
    got = dev.greedy(1).tolist() + dev.greedy(1).tolist() + dev.greedy(18).tolist()
    assert got == want
    assert dev.position == 70
    assert O.rel_frobenius(dev.hidden(1), want_hidden) <= 4 * TOL
    assert O.rel_frobenius(dev.logits().reshape(1, -1), want_logits.reshape(1, -1)) <= 4 * TOL
    # a prompt continuation through forward(), then the loop again: both paths read and extend the same cache
    more = O.fill_uniform_u32(7, 0, 51, 51200)
    dev.forward(more)
    a = dev.greedy(5).tolist()
    dev.reset()
    dev.set_decode_mode(0)
    dev.forward(ids)
    dev.greedy(20)
    dev.forward(more)
    assert dev.greedy(5).tolist() == a
    # up to the last position of the cache (2048), and not beyond
    dev.reset()
    dev.set_decode_mode(4)
    dev.forward(O.fill_uniform_u32(2040, 0, 52, 51200))
    b4 = dev.greedy(8).tolist()
    assert dev.position == 2048
    with pytest.raises(moon.SequenceTooLong):
        dev.greedy(1)
    dev.reset()
    dev.set_decode_mode(0)
    dev.forward(O.fill_uniform_u32(2040, 0, 52, 51200))
    assert dev.greedy(8).tolist() == b4
    dev.close()
