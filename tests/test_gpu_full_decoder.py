"""Config 5 at full size: the 24-layer random-init decoder, prefill of 768 ids, then greedy decoding.
The parity contract is identical token ids over the first 64 decode steps against the CPU oracle
(first-max-wins arg-max, sampling.zig:257-273); the top-2 logit margin of every step is printed."""
import time

import numpy as np
import pytest

from conftest import TOL

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(1500)]


def test_full_size_greedy_ids_match_oracle_for_64_steps(moon, O, ctx):
    cfg = O.TEXT_CFG
    t0 = time.time()
    w = O.synth_text_weights(cfg, 0)  # same seed / streams as the device-side generator
    ids = O.fill_uniform_u32(768, 0, 50, cfg["vocab"])
    ref = O.TextModel(w, cfg)
    want, margins, ref_logits = ref.greedy(ids, 64)
    print(f"\noracle: weights + prefill 768 + 64 steps in {time.time() - t0:.1f} s; "
          f"min top-2 margin {min(margins):.5f} at step {int(np.argmin(margins))}", flush=True)

    dev = moon.text_model.TextModel(moon.text_model.default_config(), seed=0, std=0.02, ctx=ctx)  # weights generated on the device
    dev.forward(ids)
    first_logits = dev.logits()
    # The 1e-3 bar is per GEMM / attention call.  After 24 layers (about 150 f16 rounding points per token, each of
    # which can land one ulp apart when the f32 summation order differs) the two implementations drift apart like a
    # random walk; the end-to-end logits are held to 4x the per-op bar, and the token ids below to equality.
    err = O.rel_frobenius(first_logits.reshape(1, -1), ref_logits[0].reshape(1, -1))
    print(f"logits after prefill: rel-Frobenius {err:.2e}", flush=True)
    assert err <= 4 * TOL
    got = dev.greedy(64).tolist()
    for s, (a, b) in enumerate(zip(got, want)):
        assert a == b, f"step {s}: gpu {a} != oracle {b} (oracle top-2 margin {margins[s]:.5f})"
    # the three- and the two-kernels-per-layer loops give the same ids
    for mode in (2, 3):
        dev.reset()
        dev.set_decode_mode(mode)
        dev.forward(ids)
        assert dev.greedy(64).tolist() == want, f"decode mode {mode}"
    assert dev.position == 768 + 64
    dev.close()


def test_the_cache_filled_token_by_token_in_the_default_mode_matches_the_wait_free_mode(moon, O, ctx):
    """1,983 greedy tokens from a 64-token prompt, to the end of the 2048-entry cache: the default mode (one kernel per layer,
    whose workgroups hand the qkv rows, the fc1 vector and the attention output to each other inside the launch, the
    last two through the die's L2 and behind counters that exist in copies) against mode 2 (three kernels per layer,
    no exchange inside a launch).  One stale or early read of an exchanged vector anywhere in 47,592 layer launches
    would change the hidden state and with it the ids from there on."""
    dev = moon.text_model.TextModel(moon.text_model.default_config(), seed=0, std=0.02, ctx=ctx)
    ids = O.fill_uniform_u32(64, 0, 50, O.TEXT_CFG["vocab"])
    out = {}
    for mode in (0, 2):
        dev.set_decode_mode(mode)
        dev.reset()
        dev.forward(ids)
        out[mode] = dev.greedy(2047 - len(ids))
    dev.close()
    assert len(out[0]) == 1983
    differ = np.flatnonzero(out[0] != out[2])
    assert differ.size == 0, f"first difference at step {int(differ[0])} (position {64 + int(differ[0])})"
