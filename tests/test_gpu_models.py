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
    """(tokens, logits, position) for decode modes 0 (one kernel per layer where the device supports it), 2 (three kernels
    per layer) and 3 (two kernels per layer)."""
    out = []
    for mode in (0, 2, 3):
        dev.reset()
        dev.set_decode_mode(mode)
        dev.forward(ids)
        toks = dev.greedy(n_steps).tolist()
        out.append((toks, dev.logits().copy(), dev.position))
    return out


def test_decode_modes_agree_small(moon, O, ctx):
    """The fused decode kernels of every mode share arithmetic and summation order: same bits."""
    _, dev = _text_pair(moon, O, ctx, SMALL_TEXT)
    ids = O.fill_uniform_u32(20, 0, 54, SMALL_TEXT["vocab"])
    (t1, l1, p1), *others = _all_modes(dev, ids, 40)
    assert p1 == 60
    for t, l, p in others:
        assert t == t1 and p == p1
        assert np.array_equal(l.view(np.uint16), l1.view(np.uint16))
    dev.close()


def test_decode_modes_agree_full_size(moon, O, ctx):
    """Same check on the real decoder shape (24 x 2048, random-init on the device)."""
    dev = moon.text_model.TextModel(moon.text_model.default_config(), seed=0, std=0.02, ctx=ctx)
    ids = O.fill_uniform_u32(100, 0, 50, 51200)
    (t1, l1, _), *others = _all_modes(dev, ids, 12)
    for t, l, _ in others:
        assert t == t1
        assert np.array_equal(l.view(np.uint16), l1.view(np.uint16))
    dev.close()


def test_prefill_with_out_proj_and_fc2_in_one_launch(moon, O, ctx, monkeypatch):
    """At 192 rows and more the prefill runs a block's out_proj and fc2 as ONE launch (their partial sums are finished
    together); MOON_GEMM_NO_PAIR keeps them apart.  Same arithmetic but other splits of K.  Three layers of the real width
    (the first two take the joint launch) on a ragged prompt (333 rows: the last row block of the 192-row tiles is partial):
    both forms match the oracle, agree with each other, and are not the same bits (which they would be if the joint launch
    had not been taken)."""
    cfg = dict(O.TEXT_CFG, n_layers=3, vocab=2048)
    ref, dev = _text_pair(moon, O, ctx, cfg, seed=4)
    ids = O.fill_uniform_u32(333, 0, 51, cfg["vocab"])
    h_ref = ref.text_decoder(ref.text_encoder(ids), ref.new_cache())
    dev.forward(ids)
    h_pair = dev.hidden(333).copy()
    monkeypatch.setenv("MOON_GEMM_NO_PAIR", "1")
    dev.reset()
    dev.forward(ids)
    h_one = dev.hidden(333).copy()
    monkeypatch.delenv("MOON_GEMM_NO_PAIR")
    dev.close()
    assert not np.array_equal(h_pair.view(np.uint16), h_one.view(np.uint16))
    errs = O.rel_frobenius(h_pair, h_ref), O.rel_frobenius(h_one, h_ref), O.rel_frobenius(h_pair, h_one)
    print("\njoint launch / separate launches against the oracle, and against each other: %.2e %.2e %.2e" % errs, flush=True)
    assert max(errs) <= TOL


@pytest.mark.parametrize("dim,hidden,heads,rows", [(512, 2048, 8, 300), (1024, 4096, 16, 700), (256, 1024, 4, 200)])
def test_prefill_of_other_widths_through_the_joint_launch(moon, O, ctx, dim, hidden, heads, rows):
    """The joint out_proj + fc2 launch at other model widths (its splits of K and its tile counts follow the shape), on
    prompts long enough to take it: hidden states, logits and the ids decoded afterwards against the oracle."""
    cfg = dict(vocab=1500, dim=dim, hidden_dim=hidden, n_layers=3, n_heads=heads, head_dim=64, rot_dim=32, theta=10000.0, max_seq=1024)
    ref, dev = _text_pair(moon, O, ctx, cfg, seed=8)
    ids = O.fill_uniform_u32(rows, 0, 56, cfg["vocab"])
    cache = ref.new_cache()
    h_ref = ref.text_decoder(ref.text_encoder(ids), cache)
    dev.forward(ids)
    assert O.rel_frobenius(dev.hidden(rows), h_ref) <= TOL
    assert O.rel_frobenius(dev.logits().reshape(1, -1), ref.lm_head(h_ref).reshape(1, -1)) <= TOL
    dev.close()


def test_prefill_with_the_rotation_in_the_qkv_product(moon, O, ctx, monkeypatch):
    """Where the qkv projection takes the 192- / 256-row kernels (more 128 x 128 tiles than compute units: from 641 rows on at
    this width) its epilogue rotates q and k and writes the cache rows itself; MOON_GEMM_NO_ROPE runs the projection and the
    rotation as two launches.  The same values, roundings and rotations: hidden states, logits and the ids decoded from the
    cache are the same bits, for a ragged first chunk at position 0 (700 rows: 192-row tiles, the last one partial) and a
    second chunk that starts at position 700 (1000 rows: 256-row tiles)."""
    cfg = dict(O.TEXT_CFG, n_layers=2, vocab=2048)
    ref, dev = _text_pair(moon, O, ctx, cfg, seed=5)
    a, b = O.fill_uniform_u32(700, 0, 52, cfg["vocab"]), O.fill_uniform_u32(1000, 0, 53, cfg["vocab"])
    out = []
    for fused in (True, False):
        if not fused:
            monkeypatch.setenv("MOON_GEMM_NO_ROPE", "1")
        dev.reset()
        dev.forward(a)
        h1 = dev.hidden(700).copy()
        dev.forward(b)
        h2, lg = dev.hidden(1000).copy(), dev.logits().copy()
        out.append((h1, h2, lg, dev.greedy(6).tolist()))
    monkeypatch.delenv("MOON_GEMM_NO_ROPE")
    dev.close()
    for x, y in zip(out[0][:3], out[1][:3]):
        assert np.array_equal(x.view(np.uint16), y.view(np.uint16))
    assert out[0][3] == out[1][3]
    cache = ref.new_cache()
    ref.text_decoder(ref.text_encoder(a), cache)
    h_ref = ref.text_decoder(ref.text_encoder(b), cache)
    assert O.rel_frobenius(out[0][1], h_ref) <= TOL


@pytest.mark.parametrize("prompt", [880, 1000, 1200, 1500, 1900])
def test_decode_modes_agree_at_long_contexts(moon, O, ctx, prompt):
    """The one-launch-per-layer kernel is instantiated for several prefetch depths of its attention tasks and the host picks
    one by the position (4, 5, 6, 8 and 10 steps of 32 keys per split at these prompt lengths; the other modes have two
    depths).  The depth only changes when a key is requested: the modes agree bit for bit at every context length, and at
    the shortest and the longest of them the decoded ids and logits match the oracle's."""
    cfg = dict(O.TEXT_CFG, n_layers=2, vocab=2048)
    ref, dev = _text_pair(moon, O, ctx, cfg, seed=7)
    ids = O.fill_uniform_u32(prompt, 0, 55, cfg["vocab"])
    (t1, l1, p1), *others = _all_modes(dev, ids, 10)
    assert p1 == prompt + 10
    for t, l, p in others:
        assert t == t1 and p == p1
        assert np.array_equal(l.view(np.uint16), l1.view(np.uint16))
    dev.close()
    if prompt in (880, 1900):
        want, margins, ref_logits = ref.greedy(ids, 11)  # (the session's logits after 10 tokens are those that pick the 11th)
        for step, (got, exp, margin) in enumerate(zip(t1, want, margins)):
            if margin < 2e-2:  # (a near-tie in the oracle's own logits: either token is within the products' tolerance)
                break
            assert got == exp, f"step {step}: {got} != {exp} (oracle top-2 margin {margin:.4f})"
        else:
            assert O.rel_frobenius(l1.reshape(1, -1), ref_logits[-1].reshape(1, -1)) <= TOL


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


@pytest.mark.timeout(900)
def test_full_size_moondream_bin_round_trip(moon, O, ctx, tmp_path):
    """A moondream.bin with all 36 tensors at the reference's sizes (weights.zig:397-523; 3.7 GB, offsets past 2^32),
    written in the reference's layout, mapped by the library's reader and uploaded from the mapping.  The decoder built from
    the file gives the same bits as the decoder whose weights the device generator made from the same seed (so every text
    tensor is found, has the expected shape and lands in its place), and the vision session with its patch embedding and
    projection the same bits as the one built from the in-memory arrays."""
    tcfg, vcfg, io = O.TEXT_CFG, O.VISION_CFG, O.VISION_IO_CFG
    tw = O.synth_text_weights(tcfg, 0)
    vw, iw = O.synth_vision_weights(vcfg, 0), O.synth_vision_io_weights(vcfg, io, 0)
    tensors = O.text_bin_tensors(tw)
    tensors.update(O.vision_bin_tensors(vw))
    tensors.update({"v_" + k: v for k, v in iw.items()})
    assert len(tensors) == 36
    path = str(tmp_path / "moondream.bin")
    O.write_moondream_bin(path, tensors)
    import os
    size = os.path.getsize(path)
    assert size > 3_600_000_000 and size == 8 + sum(12 + len(k) + 8 * v.ndim + 2 * v.size for k, v in tensors.items())
    del tensors, tw
    mvcfg = moon.vision_model.make_config(**vcfg)
    with moon.weights.BinFile(path) as f:
        assert len(f) == 36
        txt = moon.text_model.TextModel(moon.text_model.default_config(), weights=f, ctx=ctx)
        vis = moon.vision_model.VisionModel(mvcfg, weights=f, ctx=ctx)
        vis.attach_io(weights=f)
    os.remove(path)  # the mapping is closed: the sessions own device copies
    gen = moon.text_model.TextModel(moon.text_model.default_config(), seed=0, std=0.02, ctx=ctx)
    ids = O.fill_uniform_u32(40, 0, 54, tcfg["vocab"])
    out = []
    for dev in (txt, gen):
        dev.forward(ids)
        out.append((dev.hidden(40).copy(), dev.logits().copy(), dev.greedy(4).tolist()))
        dev.close()
    assert np.array_equal(out[0][0].view(np.uint16), out[1][0].view(np.uint16))
    assert np.array_equal(out[0][1].view(np.uint16), out[1][1].view(np.uint16)) and out[0][2] == out[1][2]
    mem = moon.vision_model.VisionModel(mvcfg, weights=vw, ctx=ctx)
    mem.attach_io(weights=iw)
    patches = O.fill_normal_f16((2 * io["tokens"], io["patch_dim"]), 0, 302, 1.0)
    a, b = vis.encode_image(patches), mem.encode_image(patches)
    assert np.isfinite(a.astype(np.float32)).all() and np.array_equal(a.view(np.uint16), b.view(np.uint16))
    vis.close()
    mem.close()


@pytest.mark.parametrize("case", ["ties", "nan_at_0", "nan_elsewhere", "all_neg_inf", "max_is_last"])
def test_greedy_argmax_rules_in_every_mode(moon, O, ctx, case):
    """The greedy loop's arg-max (fused into the LM-head launch)
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
    for mode in (0, 2, 3):
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
    # a single-token forward takes the same fused kernels: it reports the raised word as well, and does not move the position
    dev.reset()
    dev.forward(ids)
    ctx.check(ctx.lib.moon_text_debug_raise_wait_error(dev.handle))
    with pytest.raises(moon.context.HipError):
        dev.forward(ids[:1])
    assert dev.position == 64
    with pytest.raises(moon.context.HipError):
        dev.forward(ids[:1])  # refused until reset
    dev.reset()
    dev.forward(ids)
    assert dev.greedy(6).tolist() == want
    # and once more through the two-kernel path, whose error word is raised by the same hook
    for mode in (3,):
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


def test_generate_stops_at_the_end_of_sequence_token(moon, O, ctx):
    """moon_text_generate = the loop of moondream.zig:323-368: the tokens before the end-of-sequence token, which is not part
    of the output (moondream.zig:341); without that token in the stream it runs for max_tokens, or to the end of the cache
    (moondream.zig:324).  Arg-max and top_k, every decode mode."""
    ref, dev = _text_pair(moon, O, ctx, SMALL_TEXT)
    V = SMALL_TEXT["vocab"]
    ids = O.fill_uniform_u32(20, 0, 57, V)
    dev.forward(ids)
    free = dev.greedy(40).tolist()
    unused = next(t for t in range(V) if t not in free)
    for mode in (0, 2, 3):
        dev.set_decode_mode(mode)
        for stop_at in (0, 1, 7, 8, 9, 23, 39):
            eos = free[stop_at]
            first = free.index(eos)  # the token may have come up earlier than where it was picked
            dev.reset()
            dev.forward(ids)
            got = dev.generate(40, eos).tolist()
            assert got == free[:first], (mode, stop_at)
            assert dev.position == 20 + first
            with pytest.raises(moon.InvalidArgument):
                dev.greedy(1)  # the session needs a forward pass after a stop
            dev.forward(np.array([eos], dtype=np.uint32))  # ... for example to go on past the token
            assert dev.position == 20 + first + 1
        dev.reset()
        dev.forward(ids)
        assert dev.generate(40, unused).tolist() == free
        assert dev.position == 60
        nxt = dev.greedy(3).tolist()  # without a stop the loop can go on
        assert nxt == ref_continue(dev, ids, free, 3)
    dev.set_decode_mode(0)
    # the end of the cache ends the loop without an error
    dev.reset()
    dev.forward(O.fill_uniform_u32(SMALL_TEXT["max_seq"] - 5, 0, 58, V))
    tail = dev.generate(40, unused)
    assert tail.size == 5 and dev.position == SMALL_TEXT["max_seq"]
    assert dev.generate(4, unused).size == 0
    # sampled: the same tokens as moon_text_sample up to the stop
    cfg = moon.sampling.sampling_config("top_k", temperature=0.7, top_k=5)
    u = np.random.default_rng(3).random(30, dtype=np.float32)
    dev.reset()
    dev.forward(ids)
    sampled = dev.sample(cfg, u).tolist()
    eos = sampled[11]
    dev.reset()
    dev.forward(ids)
    assert dev.generate(30, eos, cfg, u).tolist() == sampled[: sampled.index(eos)]
    with pytest.raises(moon.TokenIdOutOfBounds):
        dev.generate(4, V)
    dev.close()


def ref_continue(dev, ids, free, n):
    """The next n arg-max tokens after ids + free, from a second pass over the same session (what the loop must go on with)."""
    dev.reset()
    dev.forward(np.concatenate([ids, np.array(free, dtype=np.uint32)]))
    return dev.greedy(n).tolist()


def test_host_stepped_loop_equals_the_device_loop(moon, O, ctx):
    """The reference keeps the loop on the host (moondream.zig:323-368): text_decoder on one token, lm_head, sampling.sample,
    text_encoder.  Through the session that is forward([token]) + next_token() (or logits() and a host-side arg-max) per
    step: the same 64 ids as moon_text_greedy on the full-size decoder."""
    dev = moon.text_model.TextModel(moon.text_model.default_config(), seed=0, std=0.02, ctx=ctx)
    ids = O.fill_uniform_u32(768, 0, 50, 51200)
    dev.forward(ids)
    want = dev.greedy(64).tolist()
    dev.reset()
    dev.forward(ids)
    got = []
    for step in range(64):
        tok = dev.next_token()
        if step % 16 == 0:  # the reference's own form: the logits come back and the host picks
            assert tok == O.argmax(dev.logits())
        got.append(tok)
        dev.forward(np.array([tok], dtype=np.uint32))
    assert got == want
    assert dev.position == 768 + 64
    cfg = moon.sampling.sampling_config("top_k", temperature=0.5, top_k=3)
    u = np.random.default_rng(1).random(8, dtype=np.float32)
    dev.reset()
    dev.forward(ids)
    want_s = dev.sample(cfg, u).tolist()
    dev.reset()
    dev.forward(ids)
    got_s = []
    for step in range(8):
        tok = dev.next_token(cfg, float(u[step]))
        got_s.append(tok)
        dev.forward(np.array([tok], dtype=np.uint32))
    assert got_s == want_s
    dev.close()


def test_reference_shaped_calls_of_the_text_session(moon, O, ctx):
    """TextModel.text_encoder / text_decoder / lm_head as the reference's loop calls them (moondream.zig:323-368), which is
    what the Zig TextModel drop-in binds: embeddings bit-exact, the decoder on embeddings = the decoder on ids, and the
    host-kept loop built from the three calls gives the oracle's arg-max ids."""
    ref, dev = _text_pair(moon, O, ctx, SMALL_TEXT)
    V = SMALL_TEXT["vocab"]
    ids = O.fill_uniform_u32(24, 0, 61, V)
    emb = dev.text_encoder(ids)
    assert np.array_equal(emb, ref.text_encoder(ids))
    with pytest.raises(moon.TokenIdOutOfBounds):
        dev.text_encoder(np.array([3, V], dtype=np.uint32))
    with pytest.raises(moon.InvalidTensorDimension):
        dev.text_decoder(emb[:, :-1])
    cache = ref.new_cache()
    h_ref = ref.text_decoder(ref.text_encoder(ids), cache)
    h = dev.text_decoder(emb)
    assert h.shape == h_ref.shape and O.rel_frobenius(h, h_ref) <= TOL
    assert dev.position == 24
    dev.reset()
    dev.forward(ids)
    assert np.array_equal(dev.hidden(24), h)  # ids or their embeddings: the same bits
    lg = dev.lm_head()
    assert lg.shape == (1, V) and O.rel_frobenius(lg, ref.lm_head(h_ref[-1:])) <= TOL
    want = dev.greedy(12).tolist()
    dev.reset()
    x, got = dev.text_encoder(ids), []
    for _ in range(12):  # the reference's loop, one row of embeddings per step after the prompt
        dev.text_decoder(x)
        tok = O.argmax(dev.lm_head())
        got.append(tok)
        x = dev.text_encoder(np.array([tok], dtype=np.uint32))
    assert got == want
    # embeddings that are not rows of the table (the image features in front of the prompt, moondream.zig:262-283)
    feats = O.fill_normal_f16((9, SMALL_TEXT["dim"]), 0, 62, 0.5)
    cache = ref.new_cache()
    h_ref = ref.text_decoder(np.concatenate([feats, ref.text_encoder(ids)]), cache)
    dev.reset()
    h = dev.text_decoder(np.concatenate([feats, emb]))
    assert O.rel_frobenius(h, h_ref) <= TOL and dev.position == 33
    with pytest.raises(moon.SequenceTooLong):
        dev.text_decoder(np.zeros((SMALL_TEXT["max_seq"], SMALL_TEXT["dim"]), dtype=np.float16))
    dev.close()


def test_vision_encoder_in_front_of_the_projection(moon, O, ctx):
    """VisionModel.vision_encoder (vision_model.zig:204-271): patch embedding, positional embedding, the blocks on both crops
    as one sequence and the final LayerNorm, [2 * tokens, dim]; projecting that on the host gives encode_image's result."""
    cfg = SMALL_VISION
    io = dict(patch_dim=20, tokens=27, proj_hidden=96, out_dim=40)
    w, iw = O.synth_vision_weights(cfg, 0), O.synth_vision_io_weights(cfg, io, 0)
    ref = O.VisionModel(w, iw, cfg, io)
    dev = moon.vision_model.VisionModel(moon.vision_model.make_config(**cfg), weights=w, ctx=ctx)
    patches = O.fill_normal_f16((2 * io["tokens"], io["patch_dim"]), 0, 301, 1.0)
    with pytest.raises(moon.MoonError):
        dev.vision_encoder(patches)  # nothing attached yet
    dev.attach_io(moon.vision_model.make_io_config(**io), weights=iw)
    got = dev.vision_encoder(patches)
    want = ref.enc.encode(ref.embed(patches))
    assert got.shape == (2, io["tokens"], cfg["dim"])  # the reference's shape (vision_model.zig:269)
    got = got.reshape(2 * io["tokens"], cfg["dim"])
    assert O.rel_frobenius(got, want) <= TOL
    assert O.rel_frobenius(dev.encode_image(patches), ref.project(got)) <= TOL
    dev.close()
