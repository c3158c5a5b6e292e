"""Mirror of the reference's sampling module (src/utils/sampling.zig): argmax (:257-273) and sample (:353-389) with
its SamplingConfig (:248-254).  The reference draws one number per call from its PRNG (rng.float(f32)); here that
number is the argument ``u`` and the generator stays with the caller."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib as L
from .context import Context, default_context, f16, ptr

METHODS = {"greedy": L.SAMPLE_GREEDY, "multinomial": L.SAMPLE_MULTINOMIAL, "top_k": L.SAMPLE_TOP_K, "min_p": L.SAMPLE_MIN_P}


def sampling_config(method: str = "greedy", temperature: float = 0.5, top_k: int = 3, min_p: float = 0.05) -> L.SamplingConfig:
    """SamplingConfig with the reference's defaults (sampling.zig:250-252)."""
    return L.SamplingConfig(METHODS[method], temperature, top_k, min_p)


def argmax(logits, ctx: Context | None = None) -> int:
    ctx = ctx or default_context()
    logits = f16(logits).reshape(-1)
    if logits.size == 0:
        raise ValueError("EmptyTensor (sampling.zig:258)")
    idx = C.c_size_t()
    ctx.check(ctx.lib.moon_argmax(ctx.handle, ptr(logits), logits.size, C.byref(idx)))
    return int(idx.value)


def sample(logits, config: L.SamplingConfig, u: float = 0.0, ctx: Context | None = None) -> int:
    """sampling.sample on one row of f16 logits (host memory)."""
    ctx = ctx or default_context()
    logits = f16(logits).reshape(-1)
    idx = C.c_size_t()
    ctx.check(ctx.lib.moon_sample(ctx.handle, ptr(logits), logits.size, C.byref(config), u, C.byref(idx)))
    return int(idx.value)


def sample_f32(logits, config: L.SamplingConfig, u: float = 0.0, ctx: Context | None = None) -> int:
    """sampling.sample(tensor: *Tensor(f32), config, rng, allocator) (sampling.zig:353-389) on the f32 row the reference
    hands it (moondream.zig:335-337)."""
    ctx = ctx or default_context()
    logits = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
    idx = C.c_size_t()
    ctx.check(ctx.lib.moon_sample_f32(ctx.handle, logits.ctypes.data_as(C.c_void_p), logits.size, C.byref(config), u, C.byref(idx)))
    return int(idx.value)


def argmax_f32(logits, ctx: Context | None = None) -> int:
    """sampling.argmax(f32, tensor) (sampling.zig:257-273)."""
    ctx = ctx or default_context()
    logits = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
    idx = C.c_size_t()
    ctx.check(ctx.lib.moon_argmax_f32(ctx.handle, logits.ctypes.data_as(C.c_void_p), logits.size, C.byref(idx)))
    return int(idx.value)


def sample_dev(logits_dev: int, n: int, config: L.SamplingConfig, u: float = 0.0, ctx: Context | None = None) -> int:
    """sampling.sample on n f16 logits that already sit in device memory (a device address)."""
    ctx = ctx or default_context()
    idx = C.c_size_t()
    ctx.check(ctx.lib.moon_dev_sample(ctx.handle, logits_dev, n, C.byref(config), u, C.byref(idx)))
    return int(idx.value)
