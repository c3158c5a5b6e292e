"""Context, error mapping and device buffers on top of the C ABI."""
from __future__ import annotations

import ctypes as C

import numpy as np

from . import _lib as L


class MoonError(RuntimeError):
    code = -1


class InvalidTensorDimension(MoonError):  # hgemm.zig:369-372
    code = L.EINVAL_DIM


class IncompatibleTensorShapes(MoonError):  # hgemm.zig:378-381
    code = L.ESHAPE


class SequenceTooLong(MoonError):  # attention.zig:769
    code = L.ESEQ_TOO_LONG


class OutOfMemory(MoonError):
    code = L.ENOMEM


class HipError(MoonError):
    code = L.EHIP


class InvalidArgument(MoonError):
    code = L.EINVAL


class InvalidRotationDimension(MoonError):  # rope.zig:141-143
    code = L.EROT_DIM


class TokenIdOutOfBounds(MoonError):  # text_model.zig:125-128
    code = L.ETOKEN


class InvalidEpsilon(MoonError):  # ops.zig:1174-1176
    code = L.EEPS


class InvalidTemperature(MoonError):  # sampling.zig:343-345
    code = L.ETEMPERATURE


class NoDevice(MoonError):
    code = L.ENODEVICE


_BY_CODE = {c.code: c for c in (InvalidTensorDimension, IncompatibleTensorShapes, SequenceTooLong, OutOfMemory, HipError,
                                InvalidArgument, InvalidRotationDimension, TokenIdOutOfBounds, InvalidEpsilon, NoDevice, InvalidTemperature)}


def f16(a) -> np.ndarray:
    """C-contiguous float16 view/copy of a (the layout Zig's Tensor(f16).data has)."""
    a = np.ascontiguousarray(a)
    if a.dtype != np.float16:
        raise TypeError(f"expected float16, got {a.dtype}")
    return a


def ptr(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


class Context:
    """One moon_ctx: a HIP stream, staging buffers, workspaces and the resident-weight registry."""

    def __init__(self, device: int = 0):
        self.lib = L.load()
        h = C.c_void_p()
        rc = self.lib.moon_ctx_create(device, C.byref(h))
        if rc != L.OK:
            msg = self.lib.moon_last_error(None).decode()
            raise _BY_CODE.get(rc, MoonError)(msg)
        self.handle = h

    def check(self, rc: int):
        if rc != L.OK:
            raise _BY_CODE.get(rc, MoonError)(self.lib.moon_last_error(self.handle).decode())

    def close(self):
        if getattr(self, "handle", None):
            self.lib.moon_ctx_destroy(self.handle)
            self.handle = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def sync(self):
        self.check(self.lib.moon_sync(self.handle))

    def cleanup(self):
        self.lib.moon_cleanup(self.handle)

    def set_gemm_kernel(self, name: str = ""):
        """Measurement / test knob: the matrix-product kernel to take where the shape allows it ("" = by shape)."""
        self.check(self.lib.moon_set_gemm_kernel(self.handle, name.encode()))

    def last_kernel(self) -> str:
        """What the latest product / attention call dispatched (kernel name, grid, k split)."""
        return self.lib.moon_last_kernel(self.handle).decode()

    # ---- resident weights
    def register_weight(self, w: np.ndarray):
        self.check(self.lib.moon_weight_register(self.handle, ptr(w), w.size))

    def unregister_weight(self, w: np.ndarray):
        self.check(self.lib.moon_weight_unregister(self.handle, ptr(w)))

    # ---- device memory
    def alloc(self, nbytes: int) -> "DeviceBuffer":
        return DeviceBuffer(self, nbytes)

    def to_device(self, a: np.ndarray) -> "DeviceBuffer":
        a = np.ascontiguousarray(a)
        buf = DeviceBuffer(self, a.nbytes)
        self.check(self.lib.moon_dev_upload(self.handle, buf.ptr, ptr(a), a.nbytes))
        return buf

    def timer_start(self):
        self.check(self.lib.moon_timer_start(self.handle))

    def timer_stop(self) -> float:
        ms = C.c_float()
        self.check(self.lib.moon_timer_stop(self.handle, C.byref(ms)))
        return float(ms.value)


class DeviceBuffer:
    def __init__(self, ctx: Context, nbytes: int):
        self.ctx, self.nbytes = ctx, int(nbytes)
        p = C.c_void_p()
        ctx.check(ctx.lib.moon_dev_alloc(ctx.handle, self.nbytes, C.byref(p)))
        self.ptr = p

    def offset(self, nbytes: int) -> C.c_void_p:
        return C.c_void_p(self.ptr.value + int(nbytes))

    def to_host(self, shape, dtype=np.float16) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        self.ctx.check(self.ctx.lib.moon_dev_download(self.ctx.handle, ptr(out), self.ptr, out.nbytes))
        return out

    def copy_from(self, src: "DeviceBuffer", nbytes: int):
        """Device-to-device copy by the library's plain copy kernel (16-byte granules)."""
        assert nbytes <= self.nbytes and nbytes <= src.nbytes
        self.ctx.check(self.ctx.lib.moon_dev_copy(self.ctx.handle, self.ptr, src.ptr, nbytes))

    def fill_normal(self, n: int, seed: int, stream: int, std: float, byte_offset: int = 0):
        self.ctx.check(self.ctx.lib.moon_dev_fill_normal_f16(self.ctx.handle, self.offset(byte_offset), n, seed, stream, std))

    def fill_const(self, n: int, value: float):
        self.ctx.check(self.ctx.lib.moon_dev_fill_const_f16(self.ctx.handle, self.ptr, n, value))

    def fill_uniform_u32(self, n: int, seed: int, stream: int, modulo: int):
        self.ctx.check(self.ctx.lib.moon_dev_fill_uniform_u32(self.ctx.handle, self.ptr, n, seed, stream, modulo))

    def free(self):
        if self.ptr is not None and self.ctx.handle:
            self.ctx.check(self.ctx.lib.moon_dev_free(self.ctx.handle, self.ptr))
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


_default: Context | None = None


def default_context() -> Context:
    """Process-wide context, created on first use (the reference's ops likewise lean on lazily
    initialised global state: the attention thread pool, attention.zig:752-774)."""
    global _default
    if _default is None or _default.handle is None:
        _default = Context(0)
    return _default
