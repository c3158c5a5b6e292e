"""Device-resident mirror of VisionModel: the encoder blocks (src/model/vision_model.zig:231-364) and, once attached, the
patch / positional embedding in front and the projection MLP behind (vision_model.zig:186-229, 366-387)."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib as L
from .context import Context, DeviceBuffer, default_context, f16, ptr


def default_config() -> L.VisionConfig:
    cfg = L.VisionConfig()
    L.load().moon_vision_config_default(C.byref(cfg))
    return cfg


def default_io_config() -> L.VisionIoConfig:
    cfg = L.VisionIoConfig()
    L.load().moon_vision_io_config_default(C.byref(cfg))
    return cfg


def make_io_config(**kw) -> L.VisionIoConfig:
    cfg = default_io_config()
    for k, v in kw.items():
        setattr(cfg, k, v)
    return cfg


def make_config(**kw) -> L.VisionConfig:
    cfg = default_config()
    for k, v in kw.items():
        setattr(cfg, k, v)
    return cfg


def image_patches(image, patch_size: int = 14, ctx: Context | None = None) -> np.ndarray:
    """What encode_image does to the resized image before the encoder (vision_model.zig:129-184, reshape_handler.zig:5-129):
    image[H, W, C] uint8 -> normalised f16 patches [2, (H/p)*(W/p), C*p*p]."""
    ctx = ctx or default_context()
    image = np.ascontiguousarray(image)
    if image.dtype != np.uint8 or image.ndim != 3:
        raise TypeError("expected a uint8 array [H, W, C]")
    H, W, Cn = image.shape
    out = np.empty((2, (H // patch_size) * (W // patch_size) if patch_size else 0, Cn * patch_size * patch_size), dtype=np.float16)
    ctx.check(ctx.lib.moon_image_patches(ctx.handle, ptr(image), H, W, Cn, patch_size, ptr(out)))
    return out


class VisionModel:
    def __init__(self, cfg: L.VisionConfig, weights: dict | None = None, seed: int | None = None, std: float = 0.02,
                 ctx: Context | None = None):
        self.ctx = ctx or default_context()
        self.cfg = cfg
        h = C.c_void_p()
        if hasattr(weights, "vision_weights"):  # a weights.BinFile
            w = weights.vision_weights(cfg)
            self.ctx.check(self.ctx.lib.moon_vision_model_create(self.ctx.handle, C.byref(cfg), C.byref(w), C.byref(h)))
        elif weights is not None:
            w = L.VisionWeights()
            keep = []
            for field in L.VISION_WEIGHT_FIELDS:
                a = np.ascontiguousarray(weights[field[2:]], dtype=np.float16)
                keep.append(a)
                setattr(w, field, a.ctypes.data)
            self.ctx.check(self.ctx.lib.moon_vision_model_create(self.ctx.handle, C.byref(cfg), C.byref(w), C.byref(h)))
        else:
            self.ctx.check(self.ctx.lib.moon_vision_model_create_synthetic(self.ctx.handle, C.byref(cfg), seed or 0, std, C.byref(h)))
        self.handle = h

    def close(self):
        if getattr(self, "handle", None) and self.ctx.handle:
            self.ctx.lib.moon_vision_model_destroy(self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def encode(self, x) -> np.ndarray:
        x = f16(x)
        out = np.empty_like(x)
        self.ctx.check(self.ctx.lib.moon_vision_encode(self.handle, ptr(x), x.shape[0], ptr(out)))
        return out

    # ---- encode_image: patch embedding + positional embedding, encoder, concat of the two crops, projection MLP
    def attach_io(self, io_cfg: L.VisionIoConfig | None = None, weights=None, seed: int | None = None, std: float = 0.02):
        """weights: dict with the VISION_IO_WEIGHT_FIELDS names (without the v_ prefix) in the file layout, a weights.BinFile, or
        None for seeded synthetic weights."""
        self.io_cfg = io_cfg or default_io_config()
        if hasattr(weights, "vision_io_weights"):
            w = weights.vision_io_weights(self.cfg, self.io_cfg)
            self.ctx.check(self.ctx.lib.moon_vision_io_attach(self.handle, C.byref(self.io_cfg), C.byref(w)))
        elif weights is not None:
            w = L.VisionIoWeights()
            keep = []
            for field in L.VISION_IO_WEIGHT_FIELDS:
                a = np.ascontiguousarray(weights[field[2:]], dtype=np.float16)
                keep.append(a)
                setattr(w, field, a.ctypes.data)
            self.ctx.check(self.ctx.lib.moon_vision_io_attach(self.handle, C.byref(self.io_cfg), C.byref(w)))
        else:
            self.ctx.check(self.ctx.lib.moon_vision_io_attach_synthetic(self.handle, C.byref(self.io_cfg), seed or 0, std))

    def encode_image(self, patches) -> np.ndarray:
        """patches[2 * tokens, patch_dim] -> [tokens, out_dim] (VisionModel.encode_image after the rearrangement into patches)."""
        patches = f16(patches)
        io = getattr(self, "io_cfg", None) or default_io_config()  # (nothing attached: the library reports it)
        out = np.empty((io.tokens, io.out_dim), dtype=np.float16)
        self.ctx.check(self.ctx.lib.moon_vision_encode_image(self.handle, ptr(patches), ptr(out)))
        return out

    def vision_encoder(self, patches) -> np.ndarray:
        """patches[2 * tokens, patch_dim] -> [2, tokens, dim]: VisionModel.vision_encoder (vision_model.zig:204-271) after its
        rearrangement into patches: patch embedding, positional embedding, the blocks, the final LayerNorm."""
        patches = f16(patches)
        io = getattr(self, "io_cfg", None) or default_io_config()
        out = np.empty((2, io.tokens, self.cfg.dim), dtype=np.float16)
        self.ctx.check(self.ctx.lib.moon_vision_encoder(self.handle, ptr(patches), ptr(out)))
        return out

    def encode_image_u8(self, image) -> np.ndarray:
        """VisionModel.encode_image from the resized image on: image[side, side, 3] uint8 -> [tokens, out_dim]."""
        image = np.ascontiguousarray(image)
        if image.dtype != np.uint8:
            raise TypeError(f"expected uint8, got {image.dtype}")
        io = getattr(self, "io_cfg", None) or default_io_config()
        side = int(round(io.tokens ** 0.5)) * int(round((io.patch_dim / 3) ** 0.5))
        if getattr(self, "io_cfg", None) is not None and image.shape != (side, side, 3):
            raise ValueError(f"expected a {side} x {side} x 3 image, got {image.shape}")
        out = np.empty((io.tokens, io.out_dim), dtype=np.float16)
        self.ctx.check(self.ctx.lib.moon_vision_encode_image_u8(self.handle, ptr(image), ptr(out)))
        return out

    def encode_image_dev(self, patches: DeviceBuffer, out: DeviceBuffer):
        self.ctx.check(self.ctx.lib.moon_vision_encode_image_dev(self.handle, patches.ptr, out.ptr))

    def encode_dev(self, x: DeviceBuffer, tokens: int, out: DeviceBuffer):
        self.ctx.check(self.ctx.lib.moon_vision_encode_dev(self.handle, x.ptr, tokens, out.ptr))
