"""Mirror of src/core/rope.zig."""
from __future__ import annotations

import numpy as np

from .context import Context, InvalidTensorDimension, default_context, f16, ptr


def precompute_freqs_cis(dim: int, end: int, theta: float = 10000.0) -> np.ndarray:
    """precomputeFreqsCis (rope.zig:32-128): f32 [end, dim/2, 2] (cos, sin). Computed on the host
    in f32 steps like the reference (the table is an input of applyRotEmb, not a kernel)."""
    if dim <= 0 or dim % 2 or end <= 0 or theta <= 0:
        raise ValueError("DimensionTooSmall / DimensionNotEven / EndTooSmall / ThetaTooSmall")
    i = np.arange(dim // 2, dtype=np.float32)
    power = (i * np.float32(2.0)) / np.float32(dim)
    inv = np.float32(1.0) / np.power(np.float32(theta), power, dtype=np.float32)
    ang = np.arange(end, dtype=np.float32)[:, None] * inv[None, :]
    return np.stack([np.cos(ang, dtype=np.float32), np.sin(ang, dtype=np.float32)], axis=-1).astype(np.float32)


def precompute_freqs_cis_device(dim: int, end: int, theta: float = 10000.0, ctx: Context | None = None) -> np.ndarray:
    """The same table built by the device kernel the text session uses for its own copy (rope.zig:32-128)."""
    ctx = ctx or default_context()
    if end <= 0 or theta <= 0:
        raise ValueError("EndTooSmall / ThetaTooSmall")
    buf = ctx.alloc(max(1, (dim // 2) * end * 2 * 4))
    ctx.check(ctx.lib.moon_dev_rope_table(ctx.handle, buf.ptr, dim, end, theta))
    ctx.sync()
    out = buf.to_host((end, dim // 2, 2), dtype=np.float32)
    buf.free()
    return out


def apply_rot_emb(x, n_heads: int, head_dim: int, freqs_cis: np.ndarray, position_ids, rot_dim: int,
                  ctx: Context | None = None) -> np.ndarray:
    """applyRotEmb (rope.zig:130-272): x [n_heads, seq_len, head_dim]."""
    ctx = ctx or default_context()
    x = f16(x)
    if x.ndim != 3:
        raise InvalidTensorDimension("InvalidInputDimensions (rope.zig:140)")
    table = np.ascontiguousarray(freqs_cis, dtype=np.float32)
    pos = np.ascontiguousarray(position_ids, dtype=np.uint64)
    out = np.empty_like(x)
    ctx.check(ctx.lib.moon_rope_apply(ctx.handle, ptr(x), ptr(out), x.shape[0], x.shape[1], x.shape[2], ptr(table),
                                      table.shape[0], table.shape[-2], ptr(pos), rot_dim))
    return out
