"""Config 4 at its stated size: the 27-block SigLIP-style encoder on [729, 1152] (vision_model.zig:231-271), random-init
weights ~N(0, 0.02) from seed 0, LayerNorm gamma = 1 / beta = 0, input ~N(0, 1), against the oracle's VisionEncoder."""
import numpy as np
import pytest

from conftest import TOL

pytestmark = pytest.mark.gpu

FULL_VISION = dict(dim=1152, hidden_dim=4304, n_layers=27, n_heads=16, head_dim=72)
# Every f16 rounding point of a block (two LayerNorms, four products each rounded twice, GELU, attention output, two residual
# adds: ~14 per element and block) may land on the neighbouring f16 value where the summation order differs; the residual
# stream carries those differences through the remaining blocks.  The per-op contract is 1e-3; as for the 24-layer decoder
# the end-to-end bound is a small multiple of it.
DEPTH_TOL = 4 * TOL


def test_full_depth_vision_encoder_matches_oracle(moon, O, ctx):
    cfg = FULL_VISION
    w = O.synth_vision_weights(cfg, 0)
    ref = O.VisionEncoder(w, cfg)
    x = O.fill_normal_f16((729, cfg["dim"]), 0, 200, 1.0)
    # the oracle first: activations ~N(0,1) through 27 random-init blocks must stay finite in f16
    xs = [np.ascontiguousarray(x)]
    for layer in range(cfg["n_layers"]):
        xs.append(ref.block(xs[-1], layer))
        assert np.isfinite(xs[-1].astype(np.float32)).all(), f"oracle overflows f16 after block {layer + 1}"
    want = O.layernorm(xs[-1], w["norm_out_w"], w["norm_out_b"])
    # device: error after k blocks (each with the final LayerNorm, as encode applies it), k on a coarse grid, then all 27
    for k in (1, 2, 4, 8, 16):
        sub = dict(cfg, n_layers=k)
        wk = {name: (a[:k] if name not in ("norm_out_w", "norm_out_b") else a) for name, a in w.items()}
        dev = moon.vision_model.VisionModel(moon.vision_model.make_config(**sub), weights=wk, ctx=ctx)
        err = O.rel_frobenius(dev.encode(x), O.layernorm(xs[k], w["norm_out_w"], w["norm_out_b"]))
        dev.close()
        print(f"vision encoder, {k:2d} blocks: rel-Frobenius {err:.2e}")
        assert err <= DEPTH_TOL
    dev = moon.vision_model.VisionModel(moon.vision_model.make_config(**cfg), weights=w, ctx=ctx)
    got = dev.encode(x)
    err = O.rel_frobenius(got, want)
    print(f"vision encoder, 27 blocks: rel-Frobenius {err:.2e}, max |x| in the oracle's residual stream "
          f"{max(float(np.abs(a.astype(np.float32)).max()) for a in xs):.1f}")
    assert np.isfinite(got.astype(np.float32)).all()
    assert err <= DEPTH_TOL
    # the session built from the seed on the device holds the same weights
    dev_syn = moon.vision_model.VisionModel(moon.vision_model.make_config(**cfg), seed=0, std=0.02, ctx=ctx)
    assert np.array_equal(dev_syn.encode(x), got)
    dev.close()
    dev_syn.close()
