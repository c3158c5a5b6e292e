"""ctypes front end of the CPU oracle -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Only tests, the smoke check and the benchmark's CPU-baseline leg import this.
The C functions restate moondream-zig's arithmetic (citations in moon_oracle.h);
the model-level functions below compose them exactly the way the reference's
text_model.zig / vision_model.zig compose the core ops.  f16 tensors are numpy
float16 arrays (C-contiguous).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmoon_oracle.so")

EPS_F16 = float(np.float32(np.float16(1e-5)))  # text_model.zig:28,154-160: eps is passed typed f16


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-B", "-C", _HERE, "libmoon_oracle.so"])
    return _SO


def _load():
    lib = C.CDLL(build())
    sz, vp, f32, u64, u32 = C.c_size_t, C.c_void_p, C.c_float, C.c_uint64, C.c_uint32
    sig = {
        "orc_fill_normal_f16": (None, [vp, sz, u64, u64, f32]),
        "orc_fill_uniform_u32": (None, [vp, sz, u64, u64, u32]),
        "orc_hgemm_nn": (None, [vp, vp, vp, sz, sz, sz]),
        "orc_hgemm_nt": (None, [vp, vp, vp, sz, sz, sz]),
        "orc_hgemm_nn_f64": (None, [vp, vp, vp, sz, sz, sz]),
        "orc_hgemm_nt_f64": (None, [vp, vp, vp, sz, sz, sz]),
        "orc_sgemm": (None, [vp, vp, vp, sz, sz, sz]),
        "orc_bias_add": (None, [vp, vp, sz, sz]),
        "orc_add": (None, [vp, vp, sz]),
        "orc_gelu": (None, [vp, sz]),
        "orc_layernorm": (C.c_int, [vp, vp, vp, vp, sz, sz, f32]),
        "orc_softmax_rows": (None, [vp, sz, sz]),
        "orc_rope_table": (None, [vp, sz, sz, f32]),
        "orc_rope_apply": (None, [vp, vp, sz, sz, sz, vp, vp, sz]),
        "orc_attention_mask": (None, [vp, sz, sz]),
        "orc_sdpa_multi": (None, [vp, vp, vp, vp, sz, vp, sz, sz, sz, sz]),
        "orc_sdpa_single": (C.c_int, [vp, vp, vp, vp, vp, sz, sz, sz]),
        "orc_sdpa_f64": (None, [vp, vp, vp, vp, sz, vp, sz, sz, sz, sz]),
        "orc_kv_update": (C.c_int, [vp, vp, vp, vp, vp, sz, sz, sz, sz]),
        "orc_kv_active": (None, [vp, vp, sz, sz, sz, sz]),
        "orc_split_heads": (None, [vp, sz, sz, vp, sz, sz, sz]),
        "orc_merge_heads": (None, [vp, vp, sz, sz, sz]),
        "orc_argmax_f16": (sz, [vp, sz]),
        "orc_sample_f16": (C.c_int, [vp, sz, C.c_int, f32, sz, f32, f32, C.POINTER(sz)]),
        "orc_sample_f32": (C.c_int, [vp, sz, C.c_int, f32, sz, f32, f32, C.POINTER(sz)]),
        "orc_sampling_expf": (None, [vp, vp, sz]),
        "orc_rel_frobenius": (C.c_double, [vp, vp, sz]),
        "orc_refstyle_gemv_nt": (None, [vp, vp, vp, sz, sz, C.c_int]),
        "orc_refstyle_hgemm": (None, [vp, vp, vp, sz, sz, sz, C.c_int, C.c_int]),
        "orc_refstyle_sdpa_single": (None, [vp, vp, vp, vp, sz, sz, sz, C.c_int]),
        "orc_host_threads": (C.c_int, []),
        "orc_h2f": (f32, [C.c_uint16]),
        "orc_f2h": (C.c_uint16, [f32]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype, fn.argtypes = res, args
    return lib


_lib = _load()


def _p(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"], "oracle needs C-contiguous arrays"
    return a.ctypes.data_as(C.c_void_p)


def _h(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    assert a.dtype == np.float16, a.dtype
    return a


# ---------------------------------------------------------------- data
def fill_normal_f16(shape, seed: int, stream: int, std: float) -> np.ndarray:
    out = np.empty(shape, dtype=np.float16)
    _lib.orc_fill_normal_f16(_p(out), out.size, seed, stream, std)
    return out


def fill_uniform_u32(n: int, seed: int, stream: int, modulo: int) -> np.ndarray:
    out = np.empty(n, dtype=np.uint32)
    _lib.orc_fill_uniform_u32(_p(out), n, seed, stream, modulo)
    return out


def f2h(x: float) -> int:
    return _lib.orc_f2h(x)


def h2f(bits: int) -> float:
    return _lib.orc_h2f(bits)


# ---------------------------------------------------------------- core ops
class IncompatibleTensorShapes(ValueError):
    """hgemm.zig:378-381 / hgemm_trans.zig:417-420."""


class InvalidTensorDimension(ValueError):
    """hgemm.zig:369-372 / hgemm_trans.zig:408-411."""


class SequenceTooLong(ValueError):
    """attention.zig:769 / text_model.zig:478."""


def hgemm(a, b, f64: bool = False) -> np.ndarray:
    """hgemm.matmul(a[M,K], b[K,N]) (hgemm.zig:362)."""
    a, b = _h(a), _h(b)
    if a.ndim != 2 or b.ndim != 2:
        raise InvalidTensorDimension((a.shape, b.shape))
    if b.shape[0] != a.shape[1]:
        raise IncompatibleTensorShapes((a.shape, b.shape))
    M, K = a.shape
    N = b.shape[1]
    c = np.empty((M, N), dtype=np.float16)
    (_lib.orc_hgemm_nn_f64 if f64 else _lib.orc_hgemm_nn)(_p(a), _p(b), _p(c), M, N, K)
    return c


def hgemm_trans(a, b_t, f64: bool = False) -> np.ndarray:
    """hgemm_trans.matmul(a[M,K], b_t[N,K]) (hgemm_trans.zig:400)."""
    a, b_t = _h(a), _h(b_t)
    if a.ndim != 2 or b_t.ndim != 2:
        raise InvalidTensorDimension((a.shape, b_t.shape))
    if b_t.shape[1] != a.shape[1]:
        raise IncompatibleTensorShapes((a.shape, b_t.shape))
    M, K = a.shape
    N = b_t.shape[0]
    c = np.empty((M, N), dtype=np.float16)
    (_lib.orc_hgemm_nt_f64 if f64 else _lib.orc_hgemm_nt)(_p(a), _p(b_t), _p(c), M, N, K)
    return c


def sgemm(a: np.ndarray, b: np.ndarray) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    c = np.empty((a.shape[0], b.shape[1]), dtype=np.float32)
    _lib.orc_sgemm(_p(a), _p(b), _p(c), a.shape[0], b.shape[1], a.shape[1])
    return c


def bias_add(a, b) -> np.ndarray:
    out = _h(a).copy()
    b = _h(b)
    assert b.ndim == 1 and b.shape[0] == out.shape[-1]
    _lib.orc_bias_add(_p(out), _p(b), out.size // out.shape[-1], out.shape[-1])
    return out


def add(a, b) -> np.ndarray:
    out = _h(a).copy()
    b = _h(b)
    assert out.shape == b.shape
    _lib.orc_add(_p(out), _p(b), out.size)
    return out


def gelu(x) -> np.ndarray:
    out = _h(x).copy()
    _lib.orc_gelu(_p(out), out.size)
    return out


def layernorm(x, gamma, beta, eps: float = EPS_F16) -> np.ndarray:
    x, gamma, beta = _h(x), _h(gamma), _h(beta)
    y = np.empty_like(x)
    rc = _lib.orc_layernorm(_p(x), _p(gamma), _p(beta), _p(y), x.size // x.shape[-1], x.shape[-1], eps)
    if rc != 0:
        raise ValueError("InvalidEpsilon")
    return y


def softmax_rows(s: np.ndarray) -> np.ndarray:
    out = np.ascontiguousarray(s, dtype=np.float32).copy()
    _lib.orc_softmax_rows(_p(out), out.size // out.shape[-1], out.shape[-1])
    return out


def rope_table(dim: int, end: int, theta: float = 10000.0) -> np.ndarray:
    t = np.empty((end, dim // 2, 2), dtype=np.float32)
    _lib.orc_rope_table(_p(t), dim, end, theta)
    return t


def rope_apply(x, table: np.ndarray, position_ids, rot_dim: int) -> np.ndarray:
    x = _h(x)
    H, S, D = x.shape
    pos = np.ascontiguousarray(position_ids, dtype=np.uint64)
    assert pos.shape == (S,)
    assert table.shape[-2] * 2 == rot_dim, "InvalidRotationDimension (rope.zig:141)"
    out = np.empty_like(x)
    _lib.orc_rope_apply(_p(x), _p(out), H, S, D, _p(np.ascontiguousarray(table)), _p(pos), rot_dim)
    return out


def attention_mask(pos: int, seq_len: int) -> np.ndarray:
    m = np.zeros((1, seq_len, pos + seq_len), dtype=np.uint8)
    _lib.orc_attention_mask(_p(m), pos, seq_len)
    return m.astype(bool)


def _mask_u8(mask):
    if mask is None:
        return None, 0, None
    m = np.ascontiguousarray(mask).astype(np.uint8)
    return m, m.shape[-1], _p(m)


def sdpa_multi(q, k, v, mask=None) -> np.ndarray:
    q, k, v = _h(q), _h(k), _h(v)
    H, Lq, D = q.shape
    Lk = k.shape[1]
    m, stride, mp = _mask_u8(mask)
    out = np.empty_like(q)
    _lib.orc_sdpa_multi(_p(q), _p(k), _p(v), mp, stride, _p(out), H, Lq, Lk, D)
    return out


def sdpa_single(q, k, v, mask=None) -> np.ndarray:
    q, k, v = _h(q), _h(k), _h(v)
    H, one, D = q.shape
    assert one == 1
    Lk = k.shape[1]
    m, _, mp = _mask_u8(mask)
    out = np.empty_like(q)
    rc = _lib.orc_sdpa_single(_p(q), _p(k), _p(v), mp, _p(out), H, Lk, D)
    if rc == -3:
        raise SequenceTooLong(Lk)
    return out


def sdpa_f64(q, k, v, mask=None) -> np.ndarray:
    q, k, v = _h(q), _h(k), _h(v)
    H, Lq, D = q.shape
    m, stride, mp = _mask_u8(mask)
    out = np.empty(q.shape, dtype=np.float64)
    _lib.orc_sdpa_f64(_p(q), _p(k), _p(v), mp, stride, _p(out), H, Lq, k.shape[1], D)
    return out


def split_heads(qkv, which: int, n_heads: int, head_dim: int) -> np.ndarray:
    qkv = _h(qkv)
    S, W = qkv.shape
    out = np.empty((n_heads, S, head_dim), dtype=np.float16)
    _lib.orc_split_heads(_p(qkv), W, which * n_heads * head_dim, _p(out), S, n_heads, head_dim)
    return out


def merge_heads(x) -> np.ndarray:
    x = _h(x)
    H, S, D = x.shape
    out = np.empty((S, H * D), dtype=np.float16)
    _lib.orc_merge_heads(_p(x), _p(out), S, H, D)
    return out


def argmax(logits) -> int:
    logits = _h(logits).reshape(-1)
    return int(_lib.orc_argmax_f16(_p(logits), logits.size))


SAMPLING_METHODS = {"greedy": 0, "multinomial": 1, "top_k": 2, "min_p": 3}


def sample(logits, method: str, u: float, temperature: float = 0.5, top_k: int = 3, min_p: float = 0.05) -> int:
    """sampling.sample (sampling.zig:353-389) on one row of f16 logits; ``u`` is the number the reference draws
    from its PRNG (rng.float(f32)).  Defaults are SamplingConfig's (sampling.zig:248-254)."""
    logits = _h(logits).reshape(-1)
    idx = C.c_size_t(0)
    rc = _lib.orc_sample_f16(_p(logits), logits.size, SAMPLING_METHODS[method], temperature, top_k, min_p, u, C.byref(idx))
    if rc:
        raise ValueError({1: "InvalidTemperature", 2: "top_k of 0", 3: "empty input or unknown method"}[rc])
    return int(idx.value)


def sample_f32(logits, method: str, u: float, temperature: float = 0.5, top_k: int = 3, min_p: float = 0.05) -> int:
    """sampling.sample on the f32 row it takes in the reference (sampling.zig:353-358)."""
    logits = np.ascontiguousarray(logits, dtype=np.float32).reshape(-1)
    idx = C.c_size_t(0)
    rc = _lib.orc_sample_f32(_p(logits), logits.size, SAMPLING_METHODS[method], temperature, top_k, min_p, u, C.byref(idx))
    if rc:
        raise ValueError({1: "InvalidTemperature", 2: "top_k of 0", 3: "empty input or unknown method"}[rc])
    return int(idx.value)


def sampling_expf(x):
    """The exp the sampling paths use (one definition shared with the device), element-wise on f32."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    y = np.empty_like(x)
    _lib.orc_sampling_expf(_p(x), _p(y), x.size)
    return y


def rel_frobenius(a, b) -> float:
    a, b = _h(a), _h(b)
    assert a.shape == b.shape, (a.shape, b.shape)
    return float(_lib.orc_rel_frobenius(_p(a), _p(b), a.size))


def host_threads() -> int:
    return int(_lib.orc_host_threads())


def refstyle_hgemm(a, b, b_transposed: bool, threads: int | None = None) -> np.ndarray:
    a, b = _h(a), _h(b)
    M, K = a.shape
    N = b.shape[0] if b_transposed else b.shape[1]
    c = np.empty((M, N), dtype=np.float16)
    _lib.orc_refstyle_hgemm(_p(a), _p(b), _p(c), M, N, K, int(b_transposed), threads or host_threads())
    return c


def refstyle_sdpa_single(q, k, v, threads: int | None = None) -> np.ndarray:
    q, k, v = _h(q), _h(k), _h(v)
    H, _, D = q.shape
    out = np.empty_like(q)
    _lib.orc_refstyle_sdpa_single(_p(q), _p(k), _p(v), _p(out), H, k.shape[1], D, threads or host_threads())
    return out


# ---------------------------------------------------------------- KV cache (text_model.zig:349-539)
class KVCache:
    def __init__(self, n_layers: int, n_heads: int, head_dim: int, max_seq: int = 2048):
        self.n_layers, self.n_heads, self.head_dim, self.max_seq = n_layers, n_heads, head_dim, max_seq
        self.k = np.zeros((n_layers, n_heads, max_seq, head_dim), dtype=np.float16)
        self.v = np.zeros_like(self.k)
        self.len = [0] * n_layers

    def update(self, layer: int, kr, v):
        kr, v = _h(kr), _h(v)
        cur = C.c_size_t(self.len[layer])
        rc = _lib.orc_kv_update(_p(self.k[layer]), _p(self.v[layer]), C.byref(cur), _p(kr), _p(v),
                                self.n_heads, kr.shape[1], self.head_dim, self.max_seq)
        if rc == -3:
            raise SequenceTooLong(self.len[layer] + kr.shape[1])
        self.len[layer] = cur.value

    def active(self, layer: int):
        n = self.len[layer]
        ko = np.empty((self.n_heads, n, self.head_dim), dtype=np.float16)
        vo = np.empty_like(ko)
        _lib.orc_kv_active(_p(self.k[layer]), _p(ko), self.n_heads, n, self.head_dim, self.max_seq)
        _lib.orc_kv_active(_p(self.v[layer]), _p(vo), self.n_heads, n, self.head_dim, self.max_seq)
        return ko, vo


# ---------------------------------------------------------------- synthetic weights
TEXT_STREAMS = ["wte", "ln_w", "ln_b", "Wqkv_w", "Wqkv_b", "out_proj_w", "out_proj_b", "fc1_w", "fc1_b",
                "fc2_w", "fc2_b", "linear_w", "linear_b", "ln_out_w", "ln_out_b"]


def text_weight_shapes(cfg: dict) -> dict:
    """Tensor shapes of the text model in the moondream.bin layout (weights.zig:439-454)."""
    L, d, ffn, V = cfg["n_layers"], cfg["dim"], cfg["hidden_dim"], cfg["vocab"]
    return {"wte": (V, d), "ln_w": (L, d), "ln_b": (L, d), "Wqkv_w": (L, 3 * d, d), "Wqkv_b": (L, 3 * d),
            "out_proj_w": (L, d, d), "out_proj_b": (L, d), "fc1_w": (L, ffn, d), "fc1_b": (L, ffn),
            "fc2_w": (L, d, ffn), "fc2_b": (L, d), "linear_w": (V, d), "linear_b": (V,),
            "ln_out_w": (d,), "ln_out_b": (d,)}


def synth_text_weights(cfg: dict, seed: int, std: float = 0.02) -> dict:
    """Random-init decoder: every matrix/bias/embedding ~N(0,std), LayerNorm gamma=1, beta=0.
    Stream numbers follow TEXT_STREAMS order, so the device-side generator fills identical bytes."""
    w = {}
    for stream, name in enumerate(TEXT_STREAMS):
        shape = text_weight_shapes(cfg)[name]
        if name in ("ln_w", "ln_out_w"):
            w[name] = np.ones(shape, dtype=np.float16)
        elif name in ("ln_b", "ln_out_b"):
            w[name] = np.zeros(shape, dtype=np.float16)
        else:
            w[name] = fill_normal_f16(shape, seed, stream, std)
    return w


VISION_STREAMS = ["Wqkv_w", "Wqkv_b", "out_proj_w", "out_proj_b", "fc1_w", "fc1_b", "fc2_w", "fc2_b",
                  "norm1_w", "norm1_b", "norm2_w", "norm2_b", "norm_out_w", "norm_out_b"]


def vision_weight_shapes(cfg: dict) -> dict:
    """Encoder-block tensor shapes, [L, in, out] layout (weights.zig:459-474)."""
    L, d, ffn = cfg["n_layers"], cfg["dim"], cfg["hidden_dim"]
    return {"Wqkv_w": (L, d, 3 * d), "Wqkv_b": (L, 3 * d), "out_proj_w": (L, d, d), "out_proj_b": (L, d),
            "fc1_w": (L, d, ffn), "fc1_b": (L, ffn), "fc2_w": (L, ffn, d), "fc2_b": (L, d),
            "norm1_w": (L, d), "norm1_b": (L, d), "norm2_w": (L, d), "norm2_b": (L, d),
            "norm_out_w": (d,), "norm_out_b": (d,)}


def synth_vision_weights(cfg: dict, seed: int, std: float = 0.02) -> dict:
    w = {}
    for stream, name in enumerate(VISION_STREAMS):
        shape = vision_weight_shapes(cfg)[name]
        if name.startswith("norm") and name.endswith("_w"):
            w[name] = np.ones(shape, dtype=np.float16)
        elif name.startswith("norm") and name.endswith("_b"):
            w[name] = np.zeros(shape, dtype=np.float16)
        else:
            w[name] = fill_normal_f16(shape, seed, 100 + stream, std)
    return w


TEXT_CFG = dict(vocab=51200, dim=2048, hidden_dim=8192, n_layers=24, n_heads=32, head_dim=64,
                rot_dim=32, theta=10000.0, max_seq=2048)  # config.zig:3-14
VISION_CFG = dict(dim=1152, hidden_dim=4304, n_layers=27, n_heads=16, head_dim=72)  # config.zig:16-26


# ---------------------------------------------------------------- text model (text_model.zig:106-345)
class TextModel:
    def __init__(self, weights: dict, cfg: dict):
        self.w, self.cfg = weights, cfg
        # text_model.zig:88 passes (dim=n_heads, end=config.dim); equivalent to (rot_dim, max_seq)
        # for the shipped config. The table has rot_dim/2 frequency pairs per position.
        self.freqs = rope_table(cfg["rot_dim"], cfg["max_seq"], cfg["theta"])

    def new_cache(self) -> KVCache:
        c = self.cfg
        return KVCache(c["n_layers"], c["n_heads"], c["head_dim"], c["max_seq"])

    def text_encoder(self, ids) -> np.ndarray:
        ids = np.asarray(ids)
        if ids.ndim != 1:
            raise ValueError("InvalidInputShape")
        if ids.shape[0] > self.cfg["max_seq"]:
            raise SequenceTooLong(ids.shape[0])
        if (ids >= self.cfg["vocab"]).any():
            raise IndexError("TokenIdOutOfBounds")
        return np.ascontiguousarray(self.w["wte"][ids])

    def attention_block(self, x, layer: int, cache: KVCache) -> np.ndarray:
        c, w = self.cfg, self.w
        H, D = c["n_heads"], c["head_dim"]
        S = x.shape[0]
        pos = cache.len[layer]
        qkv = bias_add(hgemm_trans(x, w["Wqkv_w"][layer]), w["Wqkv_b"][layer])      # :193-196
        q, k, v = (split_heads(qkv, i, H, D) for i in range(3))                       # :198-226
        position_ids = np.arange(pos, pos + S, dtype=np.uint64)                       # :228-233
        qr = rope_apply(q, self.freqs, position_ids, c["rot_dim"])                    # :235-244
        kr = rope_apply(k, self.freqs, position_ids, c["rot_dim"])                    # :246-254
        cache.update(layer, kr, v)                                                    # :261
        kf, vf = cache.active(layer)                                                  # :262
        mask = attention_mask(pos, S)                                                 # :279
        if S == 1:
            o = sdpa_single(qr, kf, vf, mask)                                         # :286
        else:
            o = sdpa_multi(qr, kf, vf, mask)                                          # :289
        o = merge_heads(o)                                                            # :293-294
        return bias_add(hgemm_trans(o, w["out_proj_w"][layer]), w["out_proj_b"][layer])  # :296-299

    def mlp(self, x, layer: int) -> np.ndarray:
        w = self.w
        h = gelu(bias_add(hgemm_trans(x, w["fc1_w"][layer]), w["fc1_b"][layer]))      # :310-315
        return bias_add(hgemm_trans(h, w["fc2_w"][layer]), w["fc2_b"][layer])         # :317-320

    def text_decoder(self, embeds, cache: KVCache) -> np.ndarray:
        hidden = _h(embeds).copy()
        for layer in range(self.cfg["n_layers"]):
            ln_in = layernorm(hidden, self.w["ln_w"][layer], self.w["ln_b"][layer])   # :154-160
            attn = self.attention_block(ln_in, layer, cache)                          # :164
            mlp = self.mlp(ln_in, layer)                                              # :167
            attn = add(attn, mlp)                                                     # :170
            hidden = add(hidden, attn)                                                # :171
        return hidden

    def lm_head(self, hidden) -> np.ndarray:
        last = _h(hidden)[-1:]                                                        # :331
        n = layernorm(last, self.w["ln_out_w"], self.w["ln_out_b"])                   # :334
        return bias_add(hgemm_trans(n, self.w["linear_w"]), self.w["linear_b"])       # :339-342

    def greedy(self, ids, n_steps: int):
        """Prefill + n_steps of greedy decoding (moondream.zig:323-368 loop shape).
        Returns (token ids, per-step top-2 logit margin, logits of every step)."""
        cache = self.new_cache()
        hidden = self.text_decoder(self.text_encoder(ids), cache)
        out, margins, all_logits = [], [], []
        for _ in range(n_steps):
            logits = self.lm_head(hidden)
            tok = argmax(logits)
            lf = logits.astype(np.float32).reshape(-1)
            top2 = np.partition(lf, -2)[-2:]
            margins.append(float(top2[1] - top2[0]))
            all_logits.append(logits.reshape(-1))
            out.append(tok)
            hidden = self.text_decoder(self.text_encoder(np.array([tok])), cache)
        return out, margins, all_logits


# ---------------------------------------------------------------- vision encoder (vision_model.zig:231-364)
class VisionEncoder:
    def __init__(self, weights: dict, cfg: dict):
        self.w, self.cfg = weights, cfg

    def attention_block(self, x, layer: int) -> np.ndarray:
        c, w = self.cfg, self.w
        H, D = c["n_heads"], c["head_dim"]
        qkv = bias_add(hgemm(x, w["Wqkv_w"][layer]), w["Wqkv_b"][layer])              # :279-282
        q, k, v = (split_heads(qkv, i, H, D) for i in range(3))                       # :285-314
        o = merge_heads(sdpa_multi(q, k, v, None))                                    # :316-329
        return bias_add(hgemm(o, w["out_proj_w"][layer]), w["out_proj_b"][layer])     # :337-340

    def mlp(self, x, layer: int) -> np.ndarray:
        w = self.w
        h = gelu(bias_add(hgemm(x, w["fc1_w"][layer]), w["fc1_b"][layer]))            # :351-356
        return bias_add(hgemm(h, w["fc2_w"][layer]), w["fc2_b"][layer])               # :358-361

    def block(self, x, layer: int) -> np.ndarray:
        w = self.w
        x = add(x, self.attention_block(layernorm(x, w["norm1_w"][layer], w["norm1_b"][layer]), layer))  # :239-248
        x = add(x, self.mlp(layernorm(x, w["norm2_w"][layer], w["norm2_b"][layer]), layer))              # :253-262
        return x

    def encode(self, x, n_layers: int | None = None) -> np.ndarray:
        x = _h(x).copy()
        for layer in range(self.cfg["n_layers"] if n_layers is None else n_layers):
            x = self.block(x, layer)
        return layernorm(x, self.w["norm_out_w"], self.w["norm_out_b"])               # :266


# ---------------------------------------------------------------- encode_image around the encoder (vision_model.zig:186-229, 366-387)
VISION_IO_STREAMS = ["patch_embedding_linear_w", "patch_embedding_linear_b", "pos_embedding", "proj_fc1_w", "proj_fc1_b",
                     "proj_fc2_w", "proj_fc2_b"]
VISION_IO_CFG = dict(patch_dim=588, tokens=729, proj_hidden=8192, out_dim=2048)  # config.zig:16-26, 3-14


def vision_io_weight_shapes(cfg: dict, io: dict) -> dict:
    """[in, out] layout (weights.zig:456-458, 476-479)."""
    d, K, T, Hp, O = cfg["dim"], io["patch_dim"], io["tokens"], io["proj_hidden"], io["out_dim"]
    return {"patch_embedding_linear_w": (K, d), "patch_embedding_linear_b": (d,), "pos_embedding": (1, T, d),
            "proj_fc1_w": (2 * d, Hp), "proj_fc1_b": (Hp,), "proj_fc2_w": (Hp, O), "proj_fc2_b": (O,)}


def synth_vision_io_weights(cfg: dict, io: dict, seed: int, std: float = 0.02) -> dict:
    shapes = vision_io_weight_shapes(cfg, io)
    return {name: fill_normal_f16(shapes[name], seed, 120 + stream, std) for stream, name in enumerate(VISION_IO_STREAMS)}


def image_patches(image, patch_size: int = 14) -> np.ndarray:
    """The steps of VisionModel.createPatches / encode_image between the resize and the encoder, each in f16 as the
    reference's Tensor(f16) arithmetic is: u8 -> f16 in both crops (vision_model.zig:137-157), BHWC -> BCHW
    (reshape_handler.zig:98-129), /= 255 (vision_model.zig:167-169), (x - 0.5) / 0.5 (reshape_handler.zig:67-96), and
    rearrangeBCHWtoBTC (reshape_handler.zig:5-65).  image[H, W, C] uint8 -> [2, (H/p)*(W/p), C*p*p] float16."""
    image = np.asarray(image)
    if image.dtype != np.uint8 or image.ndim != 3:
        raise TypeError("expected a uint8 array [H, W, C]")
    H, W, Cn = image.shape
    p = patch_size
    if H % p or W % p:
        raise ValueError("InvalidPatchSize")
    x = np.stack([image, image]).astype(np.float16)          # both crops hold the same pixels
    x = np.ascontiguousarray(x.transpose(0, 3, 1, 2))         # BHWC -> BCHW
    x = x / np.float16(255.0)
    x = (x - np.float16(0.5)) / np.float16(0.5)
    assert x.dtype == np.float16
    x = x.reshape(2, Cn, H // p, p, W // p, p).transpose(0, 2, 4, 1, 3, 5)   # b c (h p1) (w p2) -> b (h w) (c p1 p2)
    return np.ascontiguousarray(x).reshape(2, (H // p) * (W // p), Cn * p * p)


class VisionModel:
    """encode_image after the rearrangement into patches: patches[2 * tokens, patch_dim] -> [tokens, out_dim]."""

    def __init__(self, weights: dict, io_weights: dict, cfg: dict, io: dict):
        self.enc, self.w, self.cfg, self.io = VisionEncoder(weights, cfg), io_weights, cfg, io

    def embed(self, patches) -> np.ndarray:
        w, T, d = self.w, self.io["tokens"], self.cfg["dim"]
        x = bias_add(hgemm(patches, w["patch_embedding_linear_w"]), w["patch_embedding_linear_b"])   # :220-222
        x = x.reshape(2, T * d)
        pos = _h(w["pos_embedding"]).reshape(T * d)
        return np.stack([add(x[0], pos), add(x[1], pos)]).reshape(2 * T, d)                            # :226-227

    def project(self, enc_out) -> np.ndarray:
        w, T = self.w, self.io["tokens"]
        cat = np.ascontiguousarray(np.concatenate([enc_out[:T], enc_out[T:]], axis=1))                 # :189-196
        h = gelu(bias_add(hgemm(cat, w["proj_fc1_w"]), w["proj_fc1_b"]))                               # :372-379
        return bias_add(hgemm(h, w["proj_fc2_w"]), w["proj_fc2_b"])                                    # :381-384

    def encode_image(self, patches, n_layers: int | None = None) -> np.ndarray:
        return self.project(self.enc.encode(self.embed(patches), n_layers))                            # all 2T rows as one sequence (:273-329)


# ---------------------------------------------------------------- moondream.bin (weights.zig:62-204, weights.py:106-125,161)
# An independent restatement of the file layout for the tests of the library's reader: u32 magic "MOON", u32 version 2,
# then per tensor {u32 name length, u32 number of dims, u32 element count}, name bytes, dims as u64, binary16 data.
BIN_MAGIC, BIN_VERSION = 0x4D4F4F4E, 2
TEXT_BIN_NAMES = {"wte": "word_token_embedding", "ln_w": "t_ln_w", "ln_b": "t_ln_b", "Wqkv_w": "t_Wqkv_w", "Wqkv_b": "t_Wqkv_b",
                  "out_proj_w": "t_out_proj_w", "out_proj_b": "t_out_proj_bias", "fc1_w": "t_fc1_w", "fc1_b": "t_fc1_b",
                  "fc2_w": "t_fc2_w", "fc2_b": "t_fc2_b", "linear_w": "t_linear_w", "linear_b": "t_linear_b",
                  "ln_out_w": "t_ln_out_w", "ln_out_b": "t_ln_out_b"}  # storeTensor's names (weights.zig:236-267)


def bin_record(name: str, arr: np.ndarray) -> bytes:
    a = np.ascontiguousarray(arr, dtype=np.float16)
    nb = name.encode()
    out = len(nb).to_bytes(4, "little") + a.ndim.to_bytes(4, "little") + (a.size & 0xFFFFFFFF).to_bytes(4, "little") + nb
    for d in a.shape:
        out += int(d).to_bytes(8, "little")
    return out + a.tobytes()


def write_moondream_bin(path: str, tensors: dict) -> None:
    with open(path, "wb") as f:
        f.write(BIN_MAGIC.to_bytes(4, "little") + BIN_VERSION.to_bytes(4, "little"))
        for name, arr in tensors.items():
            f.write(bin_record(name, arr))


def read_moondream_bin(path: str) -> dict:
    raw = open(path, "rb").read()
    if int.from_bytes(raw[0:4], "little") != BIN_MAGIC:
        raise ValueError("InvalidMagicNumber")
    if int.from_bytes(raw[4:8], "little") != BIN_VERSION:
        raise ValueError("InvalidVersion")
    pos, out = 8, {}
    while pos < len(raw):
        name_len, ndim = int.from_bytes(raw[pos:pos + 4], "little"), int.from_bytes(raw[pos + 4:pos + 8], "little")
        pos += 12
        name = raw[pos:pos + name_len].decode()
        pos += name_len
        shape = tuple(int.from_bytes(raw[pos + 8 * i:pos + 8 * i + 8], "little") for i in range(ndim))
        pos += 8 * ndim
        n = int(np.prod(shape)) if shape else 1
        out[name] = np.frombuffer(raw, dtype=np.float16, count=n, offset=pos).reshape(shape)
        pos += 2 * n
    return out


def text_bin_tensors(w: dict) -> dict:
    return {TEXT_BIN_NAMES[k]: v for k, v in w.items()}


def vision_bin_tensors(w: dict) -> dict:
    return {"v_" + k: v for k, v in w.items()}
