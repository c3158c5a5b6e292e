"""Device-resident mirror of TextModel + KVCache (src/model/text_model.zig)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib as L
from .context import InvalidTensorDimension, Context, default_context, ptr


def default_config() -> L.TextConfig:
    cfg = L.TextConfig()
    L.load().moon_text_config_default(C.byref(cfg))
    return cfg


def make_config(**kw) -> L.TextConfig:
    cfg = default_config()
    for k, v in kw.items():
        setattr(cfg, k, v)
    return cfg


# TextWeights field -> short name used by the synthetic-weight dictionaries
_SHORT = {"word_token_embedding": "wte", "t_ln_w": "ln_w", "t_ln_b": "ln_b", "t_Wqkv_w": "Wqkv_w", "t_Wqkv_b": "Wqkv_b",
          "t_out_proj_w": "out_proj_w", "t_out_proj_b": "out_proj_b", "t_fc1_w": "fc1_w", "t_fc1_b": "fc1_b", "t_fc2_w": "fc2_w",
          "t_fc2_b": "fc2_b", "t_linear_w": "linear_w", "t_linear_b": "linear_b", "t_ln_out_w": "ln_out_w", "t_ln_out_b": "ln_out_b"}


class TextModel:
    def __init__(self, cfg: L.TextConfig, weights: dict | None = None, seed: int | None = None, std: float = 0.02,
                 ctx: Context | None = None):
        self.ctx = ctx or default_context()
        self.cfg = cfg
        h = C.c_void_p()
        if hasattr(weights, "text_weights"):  # a weights.BinFile: upload straight from the mapped moondream.bin
            w = weights.text_weights(cfg)
            self.ctx.check(self.ctx.lib.moon_text_model_create(self.ctx.handle, C.byref(cfg), C.byref(w), C.byref(h)))
        elif weights is not None:
            w = L.TextWeights()
            keep = []
            for field in L.TEXT_WEIGHT_FIELDS:
                a = np.ascontiguousarray(weights[_SHORT[field]], dtype=np.float16)
                keep.append(a)
                setattr(w, field, a.ctypes.data)
            self.ctx.check(self.ctx.lib.moon_text_model_create(self.ctx.handle, C.byref(cfg), C.byref(w), C.byref(h)))
        else:
            self.ctx.check(self.ctx.lib.moon_text_model_create_synthetic(self.ctx.handle, C.byref(cfg), seed or 0, std, C.byref(h)))
        self.handle = h

    def close(self):
        if getattr(self, "handle", None) and self.ctx.handle:
            self.ctx.lib.moon_text_model_destroy(self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def reset(self):
        self.ctx.check(self.ctx.lib.moon_text_reset(self.handle))

    def set_decode_mode(self, mode: int):
        """0 (default): one fused kernel per layer; 2: three kernels per layer (no waits inside kernels); 3: two per layer."""
        self.ctx.check(self.ctx.lib.moon_text_set_decode_mode(self.handle, mode))

    @property
    def position(self) -> int:
        return int(self.ctx.lib.moon_text_position(self.handle))

    def forward(self, ids):
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        self.ctx.check(self.ctx.lib.moon_text_forward(self.handle, ptr(ids), ids.size))

    # ---- the reference's own three calls (text_model.zig:106, 139, 325), for a host that keeps its loop
    def text_encoder(self, ids) -> np.ndarray:
        """Rows of the embedding table, [n, dim] (text_model.zig:106-137)."""
        ids = np.ascontiguousarray(ids, dtype=np.uint32).reshape(-1)
        out = np.empty((ids.size, self.cfg.dim), dtype=np.float16)
        self.ctx.check(self.ctx.lib.moon_text_embed(self.handle, ptr(ids), ids.size, ptr(out)))
        return out

    def text_decoder(self, input_embeds) -> np.ndarray:
        """Appends the rows to the session's cache and returns the decoder's output for them (text_model.zig:139-180)."""
        e = np.ascontiguousarray(input_embeds, dtype=np.float16)
        if e.ndim != 2 or e.shape[1] != self.cfg.dim:
            raise InvalidTensorDimension(f"embeddings of shape {e.shape}")
        self.ctx.check(self.ctx.lib.moon_text_forward_embeds(self.handle, ptr(e), e.shape[0]))
        return self.hidden(e.shape[0])

    def lm_head(self) -> np.ndarray:
        """Logits [1, vocab] of the last row of the latest text_decoder / forward call (text_model.zig:325-345)."""
        return self.logits().reshape(1, -1)

    def hidden(self, n_rows: int) -> np.ndarray:
        out = np.empty((n_rows, self.cfg.dim), dtype=np.float16)
        self.ctx.check(self.ctx.lib.moon_text_hidden(self.handle, ptr(out), n_rows))
        return out

    def logits(self) -> np.ndarray:
        out = np.empty(self.cfg.vocab, dtype=np.float16)
        self.ctx.check(self.ctx.lib.moon_text_logits(self.handle, ptr(out)))
        return out

    def greedy(self, n_steps: int) -> np.ndarray:
        out = np.empty(n_steps, dtype=np.uint32)
        self.ctx.check(self.ctx.lib.moon_text_greedy(self.handle, n_steps, ptr(out)))
        return out

    def sample(self, config, u) -> np.ndarray:
        """The generation loop with sampling.sample in place of argmax (moondream.zig:323-368): one token per entry
        of ``u`` (the numbers the reference would draw from its PRNG), logits stay on the device."""
        u = np.ascontiguousarray(u, dtype=np.float32).reshape(-1)
        out = np.empty(u.size, dtype=np.uint32)
        self.ctx.check(self.ctx.lib.moon_text_sample(self.handle, C.byref(config), ptr(u), u.size, ptr(out)))
        return out

    def generate(self, max_tokens: int, eos_token: int, config=None, u=None) -> np.ndarray:
        """The reference's whole generation loop on the device (moondream.zig:323-368): stops at the end-of-sequence token
        (not part of the result) or at the last cache position.  config None: arg-max."""
        out = np.empty(max_tokens, dtype=np.uint32)
        n = C.c_size_t(0)
        if u is not None:
            u = np.ascontiguousarray(u, dtype=np.float32).reshape(-1)
            if u.size < max_tokens:
                raise ValueError("one random number per step is needed")
        self.ctx.check(self.ctx.lib.moon_text_generate(self.handle, C.byref(config) if config is not None else None,
                                                       ptr(u) if u is not None else None, max_tokens, eos_token, ptr(out), C.byref(n)))
        return out[: n.value].copy()

    def next_token(self, config=None, u: float = 0.0) -> int:
        """lm_head + sampling.sample on the last position (moondream.zig:333-337); the logits stay on the device."""
        tok = C.c_uint32(0)
        self.ctx.check(self.ctx.lib.moon_text_next_token(self.handle, C.byref(config) if config is not None else None, u, C.byref(tok)))
        return int(tok.value)

    PROFILE_KERNELS = ("ln_qkv_fc1", "attention", "out_fc2_residual", "lm_head", "argmax", "bump_pos")

    def greedy_profile(self, n_steps: int):
        """greedy() with a HIP event pair around every kernel launch (decode mode 0 only).  Returns
        (ids, {kernel: (average event interval in microseconds, launches)})."""
        out = np.empty(n_steps, dtype=np.uint32)
        us = np.zeros(6, dtype=np.float32)
        launches = np.zeros(6, dtype=np.uint64)
        self.ctx.check(self.ctx.lib.moon_text_greedy_profile(self.handle, n_steps, ptr(out), ptr(us), ptr(launches)))
        return out, {k: (float(us[i]), int(launches[i])) for i, k in enumerate(self.PROFILE_KERNELS)}

    @property
    def weight_bytes_per_token(self) -> int:
        return int(self.ctx.lib.moon_text_weight_bytes_per_token(self.handle))
