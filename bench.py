#!/usr/bin/env python3
"""Benchmark of the FP16 matmul + attention hot path on one MI355X.

Workload (the configuration the headline metric is quoted on): the 24-layer Phi-1.5-style FP16 decoder with
random-init weights generated on the device (seed 0, N(0,0.02), LayerNorm gamma=1/beta=0): prefill of 768
uniform-random token ids, then greedy decoding at batch 1.  One "step" is one decoded token (LM head, arg-max,
embedding gather, 24 decoder layers over the KV cache).  `value` is tokens/s over exactly --steps tokens, wall
clock around the device loop with everything resident in HBM.

Beside it, in the same run:
  * roofline: the dominant kernel of a decode step, decode_layer_kernel (one whole decoder layer: LayerNorm, qkv,
    attention over the KV cache, fc1 + GELU, out_proj, fc2, residual adds; 100,769,792 bytes of weights and vectors
    plus the layer's K/V prefix per launch, 24 launches per token), timed per launch with HIP event pairs on the
    library's stream inside the same greedy loop, right after the timed steps;
  * extra: the same decoder driven from the host one token per call (the reference's own loop shape) and one decode token
    through the operator-level C ABI with registered weights; a plain read of one layer launch's bytes; config 1's stand-alone GEMV [1x2048].[2048x8192] (33,591,296 bytes per launch, rotating over 32 weight
    buffers = 1 GiB so the 256 MB last-level cache cannot serve them, with a plain read of the same bytes beside it), the vision fc1/fc2 GEMMs (729x1152x4304, 729x4304x1152), decode / prefill / vision attention and the
    full 27-block vision encoder, each with its own roofline fraction;
  * cpu_baseline: a CPU restatement of the reference's kernels (same blocking and threading as the Zig code; the
    Zig toolchain is not available) timed on this host on a bounded sample of the same decode workload.
"""
from __future__ import annotations

import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X dense FP16

# HBM bytes per launch of the dominant kernel (decode_layer_kernel) from rocprofv3 counters: FETCH_SIZE 52846.23 KiB x
# 1.99984 plus WRITE_SIZE 754.00 KiB x 1.0, the factors being what the same counters read for the 256 MiB copies of
# --calibrate-copy (profiles/decode_kernels_hbm_traffic_pmc.txt).  A measured constant, not a live reading; it belongs
# to the default decode mode.
TRAFFIC_BYTES_PER_LAUNCH = 108_992_459

PREFILL = 768
D, FFN, H, HD, L, V = 2048, 8192, 32, 64, 24, 51200


def event_time_us(ctx, launch, iters, warmup=3):
    """Average GPU duration of one launch, HIP events (recorded on the library's stream) around every launch."""
    for i in range(warmup):
        launch(i)
    ctx.sync()
    total = 0.0
    for i in range(iters):
        ctx.timer_start()
        launch(i)
        total += ctx.timer_stop()
    return total / iters * 1e3


def launch_time_us(ctx, launch, iters, warmup=3):
    """Two figures for one launch: `us`, from ONE event pair around `iters` back-to-back launches (no per-launch event
    handling inside; the figure a kernel trace's average duration is compared with), and `event_interval_us`, the average of
    an event pair around every single launch (which adds the command processor's handling of the two events)."""
    for i in range(warmup):
        launch(i)
    ctx.sync()
    ctx.timer_start()
    for i in range(iters):
        launch(i)
    batch = ctx.timer_stop() / iters * 1e3
    return batch, event_time_us(ctx, launch, iters, warmup=0)


COPY_BYTES = 256 * 2**20


def calibration_copies(ctx, n=8):
    """n launches of the plain copy kernel, each reading and writing exactly COPY_BYTES: the dispatches of known
    traffic that FETCH_SIZE / WRITE_SIZE readings of the other kernels in the same profiler run are scaled by."""
    src = ctx.alloc(COPY_BYTES)
    dst = ctx.alloc(COPY_BYTES)
    src.fill_normal(COPY_BYTES // 2, 0, 999, 1.0)
    for _ in range(n):
        dst.copy_from(src, COPY_BYTES)
    ctx.sync()
    src.free()
    dst.free()


def bench_decoder(moon, ctx, steps, warmup, decode_mode=None):
    cfg = moon.text_model.default_config()
    t0 = time.time()
    model = moon.text_model.TextModel(cfg, seed=0, std=0.02, ctx=ctx)
    if decode_mode is not None:
        model.set_decode_mode(decode_mode)
    ids_buf = ctx.alloc(PREFILL * 4)
    ids_buf.fill_uniform_u32(PREFILL, 0, 50, V)
    ids = ids_buf.to_host((PREFILL,), np.uint32)
    setup_s = time.time() - t0
    # the first prefill also pays for workspace allocation and the first use of every kernel: time a second one
    t0 = time.perf_counter()
    model.forward(ids)
    ctx.sync()
    prefill_first_s = time.perf_counter() - t0
    model.reset()
    ctx.sync()
    t0 = time.perf_counter()
    model.forward(ids)
    ctx.sync()
    prefill_samples = [time.perf_counter() - t0]
    # The timed region: exactly `steps` decoded tokens after `warmup` untimed ones, from the same cache length every time.
    # One such sample is only 10-15 ms long, so it is repeated REPEATS times (prefill again, warm up again, time the same
    # steps) and the median is reported; every repeat's figure is kept in the output.
    samples = []
    for rep in range(REPEATS):
        if rep:
            model.reset()
            ctx.sync()
            t0 = time.perf_counter()
            model.forward(ids)
            ctx.sync()
            prefill_samples.append(time.perf_counter() - t0)
        if warmup:
            model.greedy(warmup)
        ctx.sync()
        kv0 = model.position
        t0 = time.perf_counter()
        toks = model.greedy(steps)
        ctx.sync()
        samples.append(time.perf_counter() - t0)
    dt = sorted(samples)[len(samples) // 2]
    prefill_s = sorted(prefill_samples)[len(prefill_samples) // 2]  # (the first call of the session is reported apart)
    wbytes = model.weight_bytes_per_token
    # K and V of every layer are read once per token: 2 * L * H * HD * 2 bytes per cached position
    kv_bytes = sum(2 * L * H * HD * 2 * (kv0 + s + 1) for s in range(steps)) / steps
    res = dict(tokens_per_s=steps / dt, ms_per_token=dt / steps * 1e3, prefill_tokens=PREFILL, prefill_ms=prefill_s * 1e3, prefill_repeats_ms=[x * 1e3 for x in prefill_samples], prefill_first_call_ms=prefill_first_s * 1e3,
               setup_s=setup_s, kv_len_start=kv0, weight_bytes_per_token=wbytes, kv_bytes_per_token=kv_bytes,
               hbm_gbs=(wbytes + kv_bytes) / (dt / steps) / 1e9, first_tokens=toks[:8].tolist(),
               repeats_ms_per_token=[x / steps * 1e3 for x in samples], reported="median of the repeats")
    res["hbm_frac"] = res["hbm_gbs"] / HBM_PEAK_GBS
    model.bench_ids = ids
    return model, res


PROFILE_STEPS = 32
REPEATS = 5
SAMPLED_STEPS = 64


def bench_sampled_decode(moon, ctx, model):
    """The same loop with the reference CLI's default sampler (top_k 3 at temperature 0.5, moondream.zig:64-65, 198-202) in
    place of arg-max: LM head, sample_kernel, 24 layer kernels and the position bump per token, logits never leave HBM."""
    cfg = moon.sampling.sampling_config("top_k", temperature=0.5, top_k=3)
    u = np.random.default_rng(0).random(SAMPLED_STEPS).astype(np.float32)
    model.sample(cfg, u[:4])
    ctx.sync()
    kv0 = model.position
    t0 = time.perf_counter()
    toks = model.sample(cfg, u)
    ctx.sync()
    dt = time.perf_counter() - t0
    # the greedy loop over the next 64 positions, for a comparison at (nearly) the same cache length
    t0 = time.perf_counter()
    model.greedy(SAMPLED_STEPS)
    ctx.sync()
    dt_greedy = time.perf_counter() - t0
    return dict(method="top_k", top_k=3, temperature=0.5, steps=SAMPLED_STEPS, kv_len_start=kv0, tokens_per_s=SAMPLED_STEPS / dt,
                ms_per_token=dt / SAMPLED_STEPS * 1e3, greedy_ms_per_token_next_64=dt_greedy / SAMPLED_STEPS * 1e3,
                first_tokens=toks[:8].tolist())


def profile_decode_kernels(model, us_per_token, mode=None):
    """Per-launch HIP-event timing of the decode kernels over PROFILE_STEPS further tokens of the same loop.
    An event interval is the kernel plus the command processor's handling of the two events; that overhead is taken
    from the same run: (sum of all intervals of a token - the un-instrumented time per token) / launches per token,
    and subtracted from every interval."""
    _, prof = model.greedy_profile(PROFILE_STEPS)
    kv_mid = model.position - PROFILE_STEPS / 2
    # algorithmic bytes per launch: weights and biases once, activations in and out once
    nbytes = {
        "ln_qkv_fc1": 2 * ((3 * D + FFN) * D + (3 * D + FFN) + D + 2 * D + (3 * D + FFN)),
        "attention": 2 * (2 * H * HD * kv_mid + 3 * D + D + 2 * H * HD),
        "out_fc2_residual": 2 * (D * D + D * FFN + 2 * D + D + FFN + D + D),
        "lm_head": 2 * (V * D + V + D + 2 * D + V),
        "argmax": 2 * V + 8,
        "bump_pos": 8,
    }
    # in decode mode 0 the attention runs inside the front kernel: its K/V bytes belong to that launch
    if prof["attention"][1] == 0:
        nbytes["ln_qkv_fc1"] += nbytes["attention"]
    # ... and with one kernel per layer so do the out_proj / fc2 bytes
    if prof["out_fc2_residual"][1] == 0:
        nbytes["ln_qkv_fc1"] += nbytes["out_fc2_residual"]
    launches_per_token = sum(n for _, n in prof.values()) / PROFILE_STEPS
    interval_sum = sum(us * n for us, n in prof.values()) / PROFILE_STEPS
    overhead = max(0.0, (interval_sum - us_per_token) / launches_per_token)
    out = {"event_overhead_us": overhead, "launches_per_token": launches_per_token, "interval_sum_us_per_token": interval_sum}
    for k, (raw, n) in prof.items():
        if n == 0:  # this kernel does not run in the current decode mode
            continue
        us = raw - overhead
        out[k] = dict(us=us, event_interval_us=raw, launches=n, bytes=nbytes[k], gbs=nbytes[k] / us / 1e3,
                      frac=nbytes[k] / us / 1e3 / HBM_PEAK_GBS, us_per_token=us * n / PROFILE_STEPS)
    return out


def bench_layer_read(ctx, nbytes, iters=96):
    """The yardstick for the dominant kernel: a kernel that only reads as many bytes as one decoder-layer launch does
    (weights, vectors and the K/V prefix), rotating over 24 distinct buffers like the 24 layers do, so that the 256 MB
    last-level cache serves it no better than it serves the decoder."""
    nbytes = (int(nbytes) + 15) // 16 * 16
    ring = 24
    buf = ctx.alloc(ring * nbytes)
    buf.fill_normal(ring * nbytes // 2, 0, 77, 0.02)

    def read(i):
        ctx.check(ctx.lib.moon_dev_read(ctx.handle, buf.offset((i % ring) * nbytes), nbytes, None))

    us, us_ev = launch_time_us(ctx, read, iters, warmup=ring)
    buf.free()
    return dict(kernel="read16_kernel", bytes=nbytes, ring=ring, us=us, event_interval_us=us_ev, gbs=nbytes / us / 1e3,
                frac=nbytes / us / 1e3 / HBM_PEAK_GBS)


HOST_STEPS = 64


def bench_host_stepped(moon, ctx, model, ids):
    """The reference keeps its generation loop on the host (moondream.zig:323-368).  Two forms of that loop over the
    device-resident session, HOST_STEPS tokens each from the same prefill, wall clock:
      session_calls: next_token() (LM head + arg-max on the device, 4 bytes back) and forward([token]) per token;
      reference_signatures: the unchanged loop of moondream.zig:323-368 over the drop-ins: text_decoder (a row of embeddings
        up, the hidden row down), lm_head (100 KB of logits down), the cast to f32, sampling.sample (its drop-in sends the
        f32 row up again and brings the index back), text_encoder (the next row looked up on the device and brought down)."""
    out = {}
    model.reset()
    model.forward(ids)
    ctx.sync()
    one = np.zeros(1, dtype=np.uint32)
    for timed in (False, True):
        n = HOST_STEPS if timed else 4
        t0 = time.perf_counter()
        toks = []
        for _ in range(n):
            tok = model.next_token()
            toks.append(tok)
            one[0] = tok
            model.forward(one)
        dt = time.perf_counter() - t0
    out["session_calls"] = dict(calls_per_token=2, steps=HOST_STEPS, tokens_per_s=HOST_STEPS / dt, ms_per_token=dt / HOST_STEPS * 1e3,
                                kv_len_start=model.position - HOST_STEPS, first_tokens=toks[:4])
    model.reset()
    x = model.text_encoder(ids)
    model.text_decoder(x)
    x = model.text_encoder(one)
    for timed in (False, True):
        n = HOST_STEPS if timed else 4
        t0 = time.perf_counter()
        for _ in range(n):
            model.text_decoder(x)
            logits_f32 = model.lm_head().astype(np.float32)  # logits.castWithSimd(f32), moondream.zig:335
            one[0] = moon.sampling.argmax_f32(logits_f32, ctx=ctx)  # sampling.sample with the greedy method, through its drop-in
            x = model.text_encoder(one)
        dt = time.perf_counter() - t0
    out["reference_signatures"] = dict(calls_per_token=5, steps=HOST_STEPS, tokens_per_s=HOST_STEPS / dt, ms_per_token=dt / HOST_STEPS * 1e3,
                                       kv_len_start=model.position - HOST_STEPS,
                                       bytes_per_token=dict(up=2 * D + 4 * V + 4, down=2 * D + 2 * V + 2 * D + 8))
    return out


def bench_op_level_decode(moon, ctx, tokens=3, kv0=PREFILL):
    """One decode token through the operator-level C ABI (host pointers in, host pointers out, a blocking call per
    operator) in the reference's call order (text_model.zig:150-172, 182-300, 303-345), all 24 layers' weights registered
    as resident.  Per layer: layerNorm, Wqkv product + bias, head split, applyRotEmb on q and on k, cache update on the
    host, singleMaskedSDPA on the host-side cache prefix (6.3 MB up per layer at kv 769), out_proj, fc1 + gelu, fc2, the
    two adds; then the final layerNorm, the LM head and arg-max.  Every operator is a library call; the head split /
    merge and the cache update are numpy (the reference does them on the host too).  Wall clock, `tokens` tokens."""
    ops, hg, att, rope, samp = moon.ops, moon.hgemm_trans, moon.attention, moon.rope, moon.sampling
    S = 2048

    def synth(shape, stream, std=0.02):
        n = int(np.prod(shape))
        buf = ctx.alloc(n * 2)
        buf.fill_normal(n, 0, stream, std)
        a = buf.to_host(shape)
        buf.free()
        return a

    t0 = time.perf_counter()
    w = dict(qkv=synth((L, 3 * D, D), 1), out=synth((L, D, D), 2), fc1=synth((L, FFN, D), 3), fc2=synth((L, D, FFN), 4),
             lin=synth((V, D), 5), wte=synth((V, D), 6))
    b = dict(qkv=synth((L, 3 * D), 11), out=synth((L, D), 12), fc1=synth((L, FFN), 13), fc2=synth((L, D), 14), lin=synth((V,), 15))
    ones, zeros = np.ones(D, np.float16), np.zeros(D, np.float16)
    K = synth((L, H, S, HD), 20, 1.0)
    Vc = synth((L, H, S, HD), 21, 1.0)
    table = rope.precompute_freqs_cis(32, S, 10000.0)
    registered = []
    for name in ("qkv", "out", "fc1", "fc2"):
        for l in range(L):
            ctx.register_weight(w[name][l])
            registered.append(w[name][l])
    ctx.register_weight(w["lin"])
    registered.append(w["lin"])
    setup_s = time.perf_counter() - t0

    def token(hidden, pos):
        mask = np.ones((1, 1, pos + 1), dtype=bool)
        pid = np.array([pos], dtype=np.uint64)
        for l in range(L):
            ln = ops.layer_norm(hidden, ones, zeros, ctx=ctx)
            qkv = ops.broadcast_add_simd(hg.matmul(ln, w["qkv"][l], ctx=ctx), b["qkv"][l], ctx=ctx)
            q, k, v = (np.ascontiguousarray(qkv[0, i * D:(i + 1) * D].reshape(H, 1, HD)) for i in range(3))
            q = rope.apply_rot_emb(q, H, HD, table, pid, 32, ctx=ctx)
            k = rope.apply_rot_emb(k, H, HD, table, pid, 32, ctx=ctx)
            K[l][:, pos] = k[:, 0]
            Vc[l][:, pos] = v[:, 0]
            a = att.single_masked_sdpa(q, K[l][:, :pos + 1], Vc[l][:, :pos + 1], mask, ctx=ctx)
            a = ops.broadcast_add_simd(hg.matmul(a.reshape(1, D), w["out"][l], ctx=ctx), b["out"][l], ctx=ctx)
            m = ops.gelu(ops.broadcast_add_simd(hg.matmul(ln, w["fc1"][l], ctx=ctx), b["fc1"][l], ctx=ctx), ctx=ctx)
            m = ops.broadcast_add_simd(hg.matmul(m, w["fc2"][l], ctx=ctx), b["fc2"][l], ctx=ctx)
            hidden = ops.add(hidden, ops.add(a, m, ctx=ctx), ctx=ctx)
        logits = ops.broadcast_add_simd(hg.matmul(ops.layer_norm(hidden, ones, zeros, ctx=ctx), w["lin"], ctx=ctx), b["lin"], ctx=ctx)
        return samp.argmax(logits, ctx=ctx)

    hidden = w["wte"][7:8].copy()
    tok = token(hidden, kv0)  # untimed: first use of every kernel and of the staging buffers
    t0 = time.perf_counter()
    toks = []
    for i in range(tokens):
        tok = token(w["wte"][tok:tok + 1].copy(), kv0 + 1 + i)
        toks.append(tok)
    dt = time.perf_counter() - t0
    for a in registered:
        ctx.unregister_weight(a)
    return dict(tokens=tokens, kv_len_start=kv0 + 1, ms_per_token=dt / tokens * 1e3, tokens_per_s=tokens / dt, library_calls_per_token=L * 15 + 4,
                setup_s=setup_s, tokens_out=toks,
                note="host pointers and a blocking call per operator; weights resident, activations and the K/V prefix cross the bus every call")


def bench_gemv(moon, ctx, iters=256):
    """Config 1: y = f16(f16(x.W^T) + b), x [1,2048], W [8192,2048], rotating over 32 distinct weight buffers (1 GiB) so that
    the 256 MB last-level cache cannot serve them.  Beside it the plain-read kernel on the same buffers: what one launch
    that only streams 33.6 MB reaches on this device."""
    L_ = moon._lib
    N, K, ring = FFN, D, 32
    w = ctx.alloc(ring * N * K * 2)
    for i in range(ring):
        w.fill_normal(N * K, 0, 100 + i, 0.02, byte_offset=i * N * K * 2)
    x = ctx.alloc(K * 2)
    x.fill_normal(K, 0, 1, 1.0)
    b = ctx.alloc(N * 2)
    b.fill_normal(N, 0, 2, 0.02)
    y = ctx.alloc(N * 2)

    def launch(i):
        ctx.check(ctx.lib.moon_dev_linear(ctx.handle, x.ptr, 1, K, w.offset((i % ring) * N * K * 2), N, L_.B_NK, b.ptr,
                                          L_.EPI_BIAS, y.ptr))

    def read(i):
        ctx.check(ctx.lib.moon_dev_read(ctx.handle, w.offset((i % ring) * N * K * 2), N * K * 2, None))

    us, us_ev = launch_time_us(ctx, launch, iters)
    kernel = ctx.last_kernel()
    us_read, us_read_ev = launch_time_us(ctx, read, iters)
    alg_bytes = N * K * 2 + K * 2 + N * 2 + N * 2
    for buf in (w, x, b, y):
        buf.free()
    return dict(kernel=kernel, shape="[1x2048].[2048x8192]^T + bias", us=us, event_interval_us=us_ev, bytes=alg_bytes, gbs=alg_bytes / us / 1e3,
                frac=alg_bytes / us / 1e3 / HBM_PEAK_GBS, ring_mib=ring * N * K * 2 / 2**20,
                plain_read_same_bytes=dict(kernel="read16_kernel", us=us_read, event_interval_us=us_read_ev, gbs=N * K * 2 / us_read / 1e3,
                                           frac=N * K * 2 / us_read / 1e3 / HBM_PEAK_GBS))


def bench_gemm(moon, ctx, M, K, N, iters=50, b_kn=False):
    """b_kn: the second operand as hgemm.zig takes it, [K, N]; otherwise the resident form [N, K] (the sessions transpose the
    vision weights once at load time)."""
    L_ = moon._lib
    a = ctx.alloc(M * K * 2)
    a.fill_normal(M * K, 0, 0, 1.0)
    wt = ctx.alloc(N * K * 2)
    wt.fill_normal(N * K, 0, 1, 0.02)
    b = ctx.alloc(N * 2)
    b.fill_normal(N, 0, 2, 0.02)
    c = ctx.alloc(M * N * 2)
    layout = L_.B_KN if b_kn else L_.B_NK

    def launch(i):
        ctx.check(ctx.lib.moon_dev_linear(ctx.handle, a.ptr, M, K, wt.ptr, N, layout, b.ptr, L_.EPI_BIAS, c.ptr))

    us, us_ev = launch_time_us(ctx, launch, iters)
    kernel = ctx.last_kernel()
    flops = 2.0 * M * N * K
    for buf in (a, wt, b, c):
        buf.free()
    return dict(shape=[M, K, N], kernel=kernel, us=us, event_interval_us=us_ev, tflops=flops / us / 1e6, frac=flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS)


def bench_attention(moon, ctx):
    out = {}
    # decode: 32 x 64, kv = 1024, fused rope + append, rotating over 24 caches
    S, pos, ring = 2048, 1023, 24
    ck = ctx.alloc(ring * H * S * HD * 2)
    cv = ctx.alloc(ring * H * S * HD * 2)
    ck.fill_normal(ring * H * S * HD, 0, 1, 1.0)
    cv.fill_normal(ring * H * S * HD, 0, 2, 1.0)
    qkv = ctx.alloc(3 * H * HD * 2)
    qkv.fill_normal(3 * H * HD, 0, 3, 1.0)
    rope = importlib.import_module("moondream-zig_amd").rope
    tab = ctx.to_device(rope.precompute_freqs_cis(32, S, 10000.0))
    o = ctx.alloc(H * HD * 2)

    def launch(i):
        off = (i % ring) * H * S * HD * 2
        ctx.check(ctx.lib.moon_dev_decode_attention(ctx.handle, qkv.ptr, ck.offset(off), cv.offset(off), tab.ptr, o.ptr, H, HD, 32, S, pos))

    us, us_ev = launch_time_us(ctx, launch, 100)
    nbytes = 2 * H * (pos + 1) * HD * 2 + 2 * 3 * H * HD * 2
    out["decode_32x64_kv1024"] = dict(kernel=ctx.last_kernel(), us=us, event_interval_us=us_ev, bytes=nbytes, gbs=nbytes / us / 1e3,
                                      frac=nbytes / us / 1e3 / HBM_PEAK_GBS)
    for buf in (ck, cv, qkv, o, tab):
        buf.free()

    def sdpa(Hh, Lq, Dd, causal):
        q = ctx.alloc(Hh * Lq * Dd * 2)
        k = ctx.alloc(Hh * Lq * Dd * 2)
        v = ctx.alloc(Hh * Lq * Dd * 2)
        oo = ctx.alloc(Hh * Lq * Dd * 2)
        for j, bb in enumerate((q, k, v)):
            bb.fill_normal(Hh * Lq * Dd, 0, 10 + j, 1.0)

        def launch(i):
            ctx.check(ctx.lib.moon_dev_sdpa(ctx.handle, q.ptr, k.ptr, v.ptr, oo.ptr, Hh, Lq, Lq, Dd, 0 if causal else -1, None, 0))

        t, t_ev = launch_time_us(ctx, launch, 50)
        kernel = ctx.last_kernel()
        pairs = Lq * (Lq + 1) // 2 if causal else Lq * Lq
        flops = 4.0 * Hh * Dd * pairs
        for bb in (q, k, v, oo):
            bb.free()
        return dict(kernel=kernel, us=t, event_interval_us=t_ev, useful_tflops=flops / t / 1e6, frac=flops / t / 1e6 / MFMA_F16_PEAK_TFLOPS)

    out["prefill_causal_32x768x64"] = sdpa(32, 768, 64, True)
    out["vision_16x729x72"] = sdpa(16, 729, 72, False)
    return out


def bench_vision(moon, ctx, iters=3):
    cfg = moon.vision_model.default_config()
    vm = moon.vision_model.VisionModel(cfg, seed=0, std=0.02, ctx=ctx)
    T, d = 729, 1152
    x = ctx.alloc(T * d * 2)
    x.fill_normal(T * d, 0, 200, 1.0)
    o = ctx.alloc(T * d * 2)
    vm.encode_dev(x, T, o)
    ctx.sync()
    ctx.timer_start()
    for _ in range(iters):
        vm.encode_dev(x, T, o)
    ms = ctx.timer_stop() / iters
    flops = 27 * (2.0 * T * d * (3 * d + d + 2 * 4304) + 4.0 * 16 * T * T * 72)
    finite = bool(np.isfinite(o.to_host((T, d)).astype(np.float32)).all())
    res = dict(ms=ms, tflops=flops / ms / 1e9, frac=flops / ms / 1e9 / MFMA_F16_PEAK_TFLOPS, output_finite=finite)
    # the whole encode_image as the reference runs it: two crops (1458 rows as one sequence), patch + positional embedding
    # in front, concatenation and the projection MLP behind
    vm.attach_io(seed=0, std=0.02)
    K, Hp, O = 588, 8192, 2048
    patches = ctx.alloc(2 * T * K * 2)
    patches.fill_normal(2 * T * K, 0, 300, 1.0)
    img = ctx.alloc(T * O * 2)
    vm.encode_image_dev(patches, img)
    ctx.sync()
    ctx.timer_start()
    for _ in range(iters):
        vm.encode_image_dev(patches, img)
    ms2 = ctx.timer_stop() / iters
    R = 2 * T
    flops2 = 27 * (2.0 * R * d * (3 * d + d + 2 * 4304) + 4.0 * 16 * R * R * 72) + 2.0 * R * K * d + 2.0 * T * (2 * d * Hp + Hp * O)
    finite2 = bool(np.isfinite(img.to_host((T, O)).astype(np.float32)).all())
    res["encode_image_two_crops"] = dict(ms=ms2, tflops=flops2 / ms2 / 1e9, frac=flops2 / ms2 / 1e9 / MFMA_F16_PEAK_TFLOPS, output_finite=finite2)
    # from the resized 378 x 378 x 3 image in host memory to the features in host memory (428 KB up, 3 MB down,
    # the normalise-and-patchify kernel, then the same path): wall clock of the blocking call
    pixels = np.random.default_rng(0).integers(0, 256, size=(378, 378, 3), dtype=np.uint8)
    vm.encode_image_u8(pixels)
    t0 = time.perf_counter()
    for _ in range(iters):
        vm.encode_image_u8(pixels)
    res["encode_image_from_resized_u8_host_to_host_ms"] = (time.perf_counter() - t0) / iters * 1e3
    vm.close()
    for b in (x, o, patches, img):
        b.free()
    return res


def cpu_baseline(budget_s=5.0):
    """Reference-style CPU kernels (oracle/moon_oracle.c: 32-output GEMV chunks, per-head attention, one thread per
    core spawned per call like the Zig code) on a bounded sample: LAYERS_S of the 24 decoder layers plus the LM
    head, a few decode steps at kv_len 769, extrapolated to 24 layers."""
    sys.path.insert(0, os.path.join(ROOT, "oracle"))
    O = importlib.import_module("moon_oracle")
    threads = O.host_threads()
    layers_s = 6  # 600 MB of layer weights + 210 MB LM head: beyond any CPU cache
    w = {k: O.fill_normal_f16(s, 0, i, 0.02) for i, (k, s) in enumerate(
        dict(qkv=(layers_s, 3 * D, D), out=(layers_s, D, D), fc1=(layers_s, FFN, D), fc2=(layers_s, D, FFN), lin=(V, D)).items())}
    bias = {k: O.fill_normal_f16((v.shape[-2],), 0, 20 + i, 0.02) for i, (k, v) in enumerate(w.items())}
    ones, zeros = np.ones(D, np.float16), np.zeros(D, np.float16)
    kv = 769
    K = O.fill_normal_f16((layers_s, H, kv, HD), 0, 30, 1.0)
    Vv = O.fill_normal_f16((layers_s, H, kv, HD), 0, 31, 1.0)
    hidden = O.fill_normal_f16((1, D), 0, 32, 1.0)

    def layer(l, hidden):
        ln = O.layernorm(hidden, ones, zeros)
        qkv = O.bias_add(O.refstyle_hgemm(ln, w["qkv"][l], True, threads), bias["qkv"])
        q = O.split_heads(qkv, 0, H, HD)
        a = O.merge_heads(O.refstyle_sdpa_single(q, K[l], Vv[l], threads))
        a = O.bias_add(O.refstyle_hgemm(a, w["out"][l], True, threads), bias["out"])
        m = O.gelu(O.bias_add(O.refstyle_hgemm(ln, w["fc1"][l], True, threads), bias["fc1"]))
        m = O.bias_add(O.refstyle_hgemm(m, w["fc2"][l], True, threads), bias["fc2"])
        return O.add(hidden, O.add(a, m))

    def head(hidden):
        return O.argmax(O.bias_add(O.refstyle_hgemm(O.layernorm(hidden, ones, zeros), w["lin"], True, threads), bias["lin"]))

    for l in range(layers_s):  # warm-up (bench.zig:187-252 does one warm-up run)
        layer(l, hidden)
    head(hidden)
    t_layer, t_head, reps = 0.0, 0.0, 0
    t_begin = time.perf_counter()
    while reps < 5 or (time.perf_counter() - t_begin < budget_s and reps < 2000):
        t0 = time.perf_counter()
        for l in range(layers_s):
            hidden = layer(l, hidden)
        t1 = time.perf_counter()
        head(hidden)
        t2 = time.perf_counter()
        t_layer += (t1 - t0) / layers_s
        t_head += t2 - t1
        reps += 1
    per_token = L * t_layer / reps + t_head / reps
    return dict(value=1.0 / per_token, unit="tokens/s", cores=threads, kind="port",
                sample=f"{layers_s} of 24 decoder layers + LM head, {reps} decode steps at kv_len {kv}, per-layer time x24; "
                       "C restatement of the reference's AVX2 kernels and per-call thread spawning, not the Zig binary")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--no-extra", action="store_true", help="skip the GEMM / attention / vision side measurements")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only-gemm", action="store_true",
                    help="only the stand-alone GEMM / attention / vision legs, printed as their own JSON line (what a counter run profiles)")
    ap.add_argument("--only-host-loops", action="store_true", help="only the host-stepped and operator-level decode legs")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="first run 8 plain 256 MiB copies (copy16_kernel) as the known-traffic yardstick for a counter run")
    ap.add_argument("--decode-mode", type=int, default=None,
                    help="0: one kernel per layer (default), 2: three kernels per layer, 3: two kernels per layer")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives or sharding exist); use --gpus 1")
    if PREFILL + args.warmup + args.steps + PROFILE_STEPS + 2 * SAMPLED_STEPS + 4 > 2048:
        sys.exit("bench.py: prefill 768 + warmup + steps + 32 profiled + 132 further steps must stay within the 2048-token KV cache")

    moon = importlib.import_module("moondream-zig_amd")
    ctx = moon.Context(0)
    if args.calibrate_copy:
        calibration_copies(ctx)
    if args.only_gemm:
        out = {"gemm_vision_fc1": bench_gemm(moon, ctx, 729, 1152, 4304), "gemm_vision_fc2": bench_gemm(moon, ctx, 729, 4304, 1152),
               "gemm_vision_fc1_kn_operand": bench_gemm(moon, ctx, 729, 1152, 4304, b_kn=True),
               "gemm_vision_fc2_kn_operand": bench_gemm(moon, ctx, 729, 4304, 1152, b_kn=True),
               "gemm_vision_qkv": bench_gemm(moon, ctx, 729, 1152, 3456), "gemm_vision_fc1_m1458": bench_gemm(moon, ctx, 1458, 1152, 4304),
               "gemm_prefill_fc1": bench_gemm(moon, ctx, 768, 2048, 8192), "gemm_prefill_fc2": bench_gemm(moon, ctx, 768, 8192, 2048),
               "gemm_4096": bench_gemm(moon, ctx, 4096, 4096, 4096, iters=20), "attention": bench_attention(moon, ctx),
               "vision_encoder_27_blocks": bench_vision(moon, ctx)}
        ctx.close()
        print(json.dumps(out))
        return
    if args.only_host_loops:
        model, _ = bench_decoder(moon, ctx, 8, 0)
        out = {"host_stepped_decode": bench_host_stepped(moon, ctx, model, model.bench_ids)}
        model.close()
        out["op_level_decode_registered_weights"] = bench_op_level_decode(moon, ctx)
        ctx.close()
        print(json.dumps(out))
        return
    model, dec = bench_decoder(moon, ctx, args.steps, args.warmup, args.decode_mode)
    kern = profile_decode_kernels(model, dec["ms_per_token"] * 1e3, args.decode_mode)
    sampled = None if args.no_extra else bench_sampled_decode(moon, ctx, model)
    host_loop = None if args.no_extra else bench_host_stepped(moon, ctx, model, model.bench_ids)
    model.close()
    yardstick = bench_layer_read(ctx, kern["ln_qkv_fc1"]["bytes"])
    gemv = bench_gemv(moon, ctx)
    extra = {"decoder": dec, "decode_kernels": kern, "plain_read_of_one_layer_launch": yardstick, "gemv_config1": gemv}
    if sampled:
        extra["sampled_decode_top_k"] = sampled
    if not args.no_extra:
        extra["host_stepped_decode"] = host_loop
        extra["op_level_decode_registered_weights"] = bench_op_level_decode(moon, ctx)
        extra["gemm_vision_fc1"] = bench_gemm(moon, ctx, 729, 1152, 4304)
        extra["gemm_vision_fc2"] = bench_gemm(moon, ctx, 729, 4304, 1152)
        extra["gemm_vision_fc1_kn_operand"] = bench_gemm(moon, ctx, 729, 1152, 4304, b_kn=True)  # hgemm.zig's own operand layout
        extra["gemm_vision_fc1_m1458"] = bench_gemm(moon, ctx, 1458, 1152, 4304)
        extra["attention"] = bench_attention(moon, ctx)
        extra["vision_encoder_27_blocks"] = bench_vision(moon, ctx)
    ctx.close()
    cpu = None if args.no_cpu else cpu_baseline()

    dom = kern["ln_qkv_fc1"]
    if "out_fc2_residual" not in kern:
        dom_name = "decode_layer_kernel<4, 16> (a whole decoder layer, 24 launches per token)"
    elif "attention" not in kern:
        dom_name = "decode_front_kernel<4> (LayerNorm + qkv + fc1 + attention, 24 launches per token)"
    else:
        dom_name = "decode_ln_gemv_kernel<4, true> (LayerNorm + qkv + fc1, 24 launches per token)"
    line = {
        "metric": "decode tokens/s (24-layer FP16 decoder); GEMV HBM GB/s; GEMM MFMA TFLOPS",
        "value": dec["tokens_per_s"], "unit": "tokens/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": dec["ms_per_token"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 (f32 accumulate)", "data": "synthetic",
        "config": {"workload": "Phi-1.5-style decoder, 24 layers, d=2048, 32x64 heads, MLP 8192, vocab 51200, random-init FP16 "
                               "weights N(0,0.02) seed 0; prefill 768 ids then greedy decode at batch 1; step = one decoded token",
                   "prefill": PREFILL, "batch": 1},
        "roofline": {"bound": "hbm", "achieved": dom["gbs"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": dom["frac"],
                     "traffic": TRAFFIC_BYTES_PER_LAUNCH if "out_fc2_residual" not in kern else None, "kernel": dom_name,
                     "bytes_per_launch": dom["bytes"], "us_per_launch": dom["us"], "event_interval_us": dom["event_interval_us"],
                     "event_overhead_us": kern["event_overhead_us"], "launches_timed": dom["launches"],
                     "plain_read_same_bytes": {"us": yardstick["us"], "gbs": yardstick["gbs"], "frac": yardstick["frac"]}},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
