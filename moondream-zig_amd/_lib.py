"""ctypes binding of libmoonhip.so (the C ABI declared in include/moonhip.h).

The library is loaded from this directory only.  There is no fallback: if the
shared object is missing, or no gfx950 GPU is present, loading / context
creation raises.
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmoonhip.so")
CSRC_DIR = os.path.join(_HERE, "csrc")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "moonhip.h")

# error codes (moonhip.h)
OK, EINVAL_DIM, ESHAPE, ESEQ_TOO_LONG, ENOMEM, EHIP, EINVAL, EROT_DIM, ETOKEN, EEPS, ENODEVICE, EFORMAT, ETEMPERATURE = range(13)
SAMPLE_GREEDY, SAMPLE_MULTINOMIAL, SAMPLE_TOP_K, SAMPLE_MIN_P = range(4)
EPI_NONE, EPI_BIAS, EPI_BIAS_GELU = 0, 1, 2
B_KN, B_NK = 0, 1


class TextConfig(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in ("vocab", "dim", "hidden_dim", "n_layers", "n_heads", "head_dim", "rot_dim", "max_seq")] + [
        ("rope_theta", C.c_float), ("ln_eps", C.c_float)]


TEXT_WEIGHT_FIELDS = ["word_token_embedding", "t_ln_w", "t_ln_b", "t_Wqkv_w", "t_Wqkv_b", "t_out_proj_w", "t_out_proj_b",
                      "t_fc1_w", "t_fc1_b", "t_fc2_w", "t_fc2_b", "t_linear_w", "t_linear_b", "t_ln_out_w", "t_ln_out_b"]


class TextWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in TEXT_WEIGHT_FIELDS]


class SamplingConfig(C.Structure):
    _fields_ = [("method", C.c_int), ("temperature", C.c_float), ("top_k", C.c_size_t), ("min_p", C.c_float)]


class VisionConfig(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in ("dim", "hidden_dim", "n_layers", "n_heads", "head_dim")] + [("ln_eps", C.c_float)]


VISION_WEIGHT_FIELDS = ["v_Wqkv_w", "v_Wqkv_b", "v_out_proj_w", "v_out_proj_b", "v_fc1_w", "v_fc1_b", "v_fc2_w", "v_fc2_b",
                        "v_norm1_w", "v_norm1_b", "v_norm2_w", "v_norm2_b", "v_norm_out_w", "v_norm_out_b"]


class VisionWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in VISION_WEIGHT_FIELDS]


class VisionIoConfig(C.Structure):
    _fields_ = [(n, C.c_size_t) for n in ("patch_dim", "tokens", "proj_hidden", "out_dim")]


VISION_IO_WEIGHT_FIELDS = ["v_patch_embedding_linear_w", "v_patch_embedding_linear_b", "v_pos_embedding", "v_proj_fc1_w", "v_proj_fc1_b",
                           "v_proj_fc2_w", "v_proj_fc2_b"]


class VisionIoWeights(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in VISION_IO_WEIGHT_FIELDS]


_sz, _vp, _i, _f, _u64, _u32, _l = C.c_size_t, C.c_void_p, C.c_int, C.c_float, C.c_uint64, C.c_uint32, C.c_long
_pp = C.POINTER(C.c_void_p)

# name -> (restype, argtypes); one entry per function declared in moonhip.h
SIGNATURES = {
    "moon_ctx_create": (_i, [_i, _pp]),
    "moon_ctx_destroy": (None, [_vp]),
    "moon_last_error": (C.c_char_p, [_vp]),
    "moon_sync": (_i, [_vp]),
    "moon_cleanup": (None, [_vp]),
    "moon_set_gemm_kernel": (_i, [_vp, C.c_char_p]),
    "moon_last_kernel": (C.c_char_p, [_vp]),
    "moon_hgemm": (_i, [_vp, _vp, _sz, _sz, _vp, _sz, _sz, _vp]),
    "moon_hgemm_trans": (_i, [_vp, _vp, _sz, _sz, _vp, _sz, _sz, _vp]),
    "moon_linear": (_i, [_vp, _vp, _sz, _sz, _vp, _sz, _i, _vp, _i, _vp]),
    "moon_weight_register": (_i, [_vp, _vp, _sz]),
    "moon_weight_unregister": (_i, [_vp, _vp]),
    "moon_sdpa_maskless": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz]),
    "moon_sdpa_masked": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _vp, _sz, _sz, _sz, _sz]),
    "moon_sdpa_single": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz]),
    "moon_rope_apply": (_i, [_vp, _vp, _vp, _sz, _sz, _sz, _vp, _sz, _sz, _vp, _sz]),
    "moon_layernorm": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _f]),
    "moon_gelu": (_i, [_vp, _vp, _sz]),
    "moon_bias_add": (_i, [_vp, _vp, _vp, _sz, _sz]),
    "moon_add": (_i, [_vp, _vp, _vp, _sz]),
    "moon_argmax": (_i, [_vp, _vp, _sz, C.POINTER(_sz)]),
    "moon_image_patches": (_i, [_vp, _vp, _sz, _sz, _sz, _sz, _vp]),
    "moon_sampling_config_default": (None, [_vp]),
    "moon_sample": (_i, [_vp, _vp, _sz, _vp, _f, C.POINTER(_sz)]),
    "moon_sample_f32": (_i, [_vp, _vp, _sz, _vp, _f, C.POINTER(_sz)]),
    "moon_argmax_f32": (_i, [_vp, _vp, _sz, C.POINTER(_sz)]),
    "moon_dev_sample": (_i, [_vp, _vp, _sz, _vp, _f, C.POINTER(_sz)]),
    "moon_dev_alloc": (_i, [_vp, _sz, _pp]),
    "moon_dev_free": (_i, [_vp, _vp]),
    "moon_dev_upload": (_i, [_vp, _vp, _vp, _sz]),
    "moon_dev_download": (_i, [_vp, _vp, _vp, _sz]),
    "moon_dev_copy": (_i, [_vp, _vp, _vp, _sz]),
    "moon_dev_read": (_i, [_vp, _vp, _sz, _vp]),
    "moon_dev_fill_normal_f16": (_i, [_vp, _vp, _sz, _u64, _u64, _f]),
    "moon_dev_fill_const_f16": (_i, [_vp, _vp, _sz, _f]),
    "moon_dev_fill_uniform_u32": (_i, [_vp, _vp, _sz, _u64, _u64, _u32]),
    "moon_dev_linear": (_i, [_vp, _vp, _sz, _sz, _vp, _sz, _i, _vp, _i, _vp]),
    "moon_dev_sdpa": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _l, _vp, _sz]),
    "moon_dev_decode_attention": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz]),
    "moon_dev_decode_attention_noalloc": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _sz, _sz, _sz, _sz, _sz]),
    "moon_dev_rope_table": (_i, [_vp, _vp, _sz, _sz, _f]),
    "moon_dev_layernorm": (_i, [_vp, _vp, _vp, _vp, _vp, _sz, _sz, _f]),
    "moon_timer_start": (_i, [_vp]),
    "moon_timer_stop": (_i, [_vp, C.POINTER(_f)]),
    "moon_text_config_default": (None, [C.POINTER(TextConfig)]),
    "moon_text_model_create": (_i, [_vp, C.POINTER(TextConfig), C.POINTER(TextWeights), _pp]),
    "moon_text_model_create_synthetic": (_i, [_vp, C.POINTER(TextConfig), _u64, _f, _pp]),
    "moon_text_model_destroy": (None, [_vp]),
    "moon_text_reset": (_i, [_vp]),
    "moon_text_forward": (_i, [_vp, _vp, _sz]),
    "moon_text_logits": (_i, [_vp, _vp]),
    "moon_text_greedy": (_i, [_vp, _sz, _vp]),
    "moon_text_sample": (_i, [_vp, _vp, _vp, _sz, _vp]),
    "moon_text_forward_embeds": (_i, [_vp, _vp, _sz]),
    "moon_text_embed": (_i, [_vp, _vp, _sz, _vp]),
    "moon_text_generate": (_i, [_vp, _vp, _vp, _sz, _u32, _vp, C.POINTER(_sz)]),
    "moon_text_next_token": (_i, [_vp, _vp, _f, C.POINTER(_u32)]),
    "moon_text_greedy_profile": (_i, [_vp, _sz, _vp, _vp, _vp]),
    "moon_text_set_decode_mode": (_i, [_vp, _i]),
    "moon_text_debug_raise_wait_error": (_i, [_vp]),
    "moon_text_position": (_sz, [_vp]),
    "moon_text_hidden": (_i, [_vp, _vp, _sz]),
    "moon_text_weight_bytes_per_token": (_sz, [_vp]),
    "moon_vision_config_default": (None, [C.POINTER(VisionConfig)]),
    "moon_vision_model_create": (_i, [_vp, C.POINTER(VisionConfig), C.POINTER(VisionWeights), _pp]),
    "moon_vision_model_create_synthetic": (_i, [_vp, C.POINTER(VisionConfig), _u64, _f, _pp]),
    "moon_vision_model_destroy": (None, [_vp]),
    "moon_vision_encode": (_i, [_vp, _vp, _sz, _vp]),
    "moon_vision_encode_dev": (_i, [_vp, _vp, _sz, _vp]),
    "moon_vision_io_config_default": (None, [C.POINTER(VisionIoConfig)]),
    "moon_vision_io_attach": (_i, [_vp, C.POINTER(VisionIoConfig), C.POINTER(VisionIoWeights)]),
    "moon_vision_io_attach_synthetic": (_i, [_vp, C.POINTER(VisionIoConfig), _u64, _f]),
    "moon_vision_encode_image": (_i, [_vp, _vp, _vp]),
    "moon_vision_encoder": (_i, [_vp, _vp, _vp]),
    "moon_vision_encode_image_dev": (_i, [_vp, _vp, _vp]),
    "moon_vision_encode_image_u8": (_i, [_vp, _vp, _vp]),
    "moon_bin_open": (_i, [C.c_char_p, _pp, C.c_char_p, _sz]),
    "moon_bin_close": (None, [_vp]),
    "moon_bin_tensor_count": (_sz, [_vp]),
    "moon_bin_tensor": (_i, [_vp, _sz, C.POINTER(C.c_char_p), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t * 4), C.POINTER(C.c_void_p)]),
    "moon_bin_find": (_i, [_vp, C.c_char_p, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t * 4), C.POINTER(C.c_void_p)]),
    "moon_bin_text_weights": (_i, [_vp, C.POINTER(TextConfig), C.POINTER(TextWeights), C.c_char_p, _sz]),
    "moon_bin_vision_weights": (_i, [_vp, C.POINTER(VisionConfig), C.POINTER(VisionWeights), C.c_char_p, _sz]),
    "moon_bin_vision_io_weights": (_i, [_vp, C.POINTER(VisionConfig), C.POINTER(VisionIoConfig), C.POINTER(VisionIoWeights), C.c_char_p, _sz]),
}

_lib = None


def load() -> C.CDLL:
    """Load libmoonhip.so built in-tree (python __graft_entry__.py build, or make -C csrc)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` (hipcc, gfx950). "
                "There is no CPU implementation to fall back to.")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib
