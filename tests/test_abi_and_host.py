"""No-GPU checks: the C-ABI library loads and exports every function include/moonhip.h declares, the ctypes table
covers them, context creation fails loudly without a device, and the host-side helpers agree with the oracle."""
import ctypes as C
import os
import re

import numpy as np
import pytest


def _declared_functions(header_path):
    text = open(header_path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moon_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(moon):
    lib = moon._lib.load()
    names = _declared_functions(moon._lib.HEADER_PATH)
    assert len(names) >= 45
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in moonhip.h but not exported: {missing}"
    unbound = [n for n in names if n not in moon._lib.SIGNATURES]
    assert not unbound, f"no ctypes signature for: {unbound}"
    extra = [n for n in moon._lib.SIGNATURES if n not in names]
    assert not extra, f"bound but not declared: {extra}"


def test_header_cites_the_reference_for_each_drop_in(moon):
    text = open(moon._lib.HEADER_PATH).read()
    for needle in ["hgemm.zig:362", "hgemm_trans.zig:400", "attention.zig:125", "attention.zig:416", "attention.zig:759",
                   "rope.zig:130", "ops.zig:1063", "ops.zig:1635", "sampling.zig:257", "text_model.zig", "vision_model.zig"]:
        assert needle in text, needle


def test_header_compiles_as_c(moon, tmp_path):
    import subprocess
    src = tmp_path / "t.c"
    src.write_text('#include "moonhip.h"\nint main(void){ moon_text_config c; moon_text_config_default(&c); return (int)c.dim == 0; }\n')
    inc = os.path.dirname(moon._lib.HEADER_PATH)
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", inc, "-c", str(src), "-o", str(tmp_path / "t.o")])


def test_no_device_is_a_loud_error(moon):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    with pytest.raises(moon.NoDevice) as e:
        moon.Context(0)
    assert "no CPU path" in str(e.value)
    lib = moon._lib.load()
    h = C.c_void_p()
    assert lib.moon_ctx_create(0, C.byref(h)) == moon._lib.ENODEVICE and not h.value
    assert lib.moon_sync(None) == moon._lib.EINVAL  # null ctx is rejected, not dereferenced


def test_config_defaults_match_the_reference(moon):
    t = moon.text_model.default_config()  # config.zig:3-14
    assert (t.vocab, t.dim, t.hidden_dim, t.n_layers, t.n_heads, t.head_dim, t.rot_dim, t.max_seq) == (51200, 2048, 8192, 24, 32, 64, 32, 2048)
    assert abs(t.rope_theta - 10000.0) < 1e-6 and abs(t.ln_eps - 1.00135803e-5) < 1e-11
    v = moon.vision_model.default_config()  # config.zig:16-26
    assert (v.dim, v.hidden_dim, v.n_layers, v.n_heads, v.head_dim) == (1152, 4304, 27, 16, 72)


def test_host_mask_and_rope_table_match_oracle(moon, O):
    for pos, seq in [(0, 1), (0, 7), (5, 1), (729, 39)]:
        assert np.array_equal(moon.attention.create_attention_mask(pos, seq), O.attention_mask(pos, seq))
    a = moon.rope.precompute_freqs_cis(32, 2048, 10000.0)
    b = O.rope_table(32, 2048, 10000.0)
    assert a.shape == b.shape == (2048, 16, 2) and a.dtype == np.float32
    assert np.abs(a - b).max() < 2e-4  # powf / cosf / sinf implementations differ in the last bits at large angles
    with pytest.raises(ValueError):
        moon.rope.precompute_freqs_cis(31, 10)


def test_python_mirror_rejects_bad_ranks_before_calling_c(moon):
    with pytest.raises((moon.InvalidTensorDimension, moon.NoDevice)):
        moon.hgemm.matmul(np.zeros((2, 2, 2), np.float16), np.zeros((2, 2), np.float16))
    with pytest.raises(TypeError):
        moon.context.f16(np.zeros(4, np.float32))
    assert np.array_equal(moon.hgemm_trans.transpose(np.arange(6, dtype=np.float16).reshape(2, 3)),
                          np.arange(6, dtype=np.float16).reshape(2, 3).T)


def test_sequential_sum_maps_equal_the_float_loop():
    """The sampler evaluates the reference's sequential f32 sums (ops.zig:1585-1592, sampling.zig:139-147, 281-294) by composing
    per-term integer maps (csrc/seq_sum.hpp).  The host program checks that arithmetic against the plain loop on 20,000 term
    lists (ties at half an ulp, whole ulps, subnormals, terms rounded away one by one, terms as large as the sum) and the
    composition's associativity; it needs no GPU."""
    import subprocess
    here = os.path.dirname(os.path.abspath(__file__))
    exe = os.path.join(here, "cxx", "seq_sum_check")
    src = os.path.join(here, "cxx", "seq_sum_check.cpp")
    hdr = os.path.join(here, "..", "moondream-zig_amd", "csrc", "seq_sum.hpp")
    if not os.path.exists(exe) or os.path.getmtime(exe) < max(os.path.getmtime(src), os.path.getmtime(hdr)):
        subprocess.check_call(["make", "-C", os.path.join(here, "cxx"), "seq_sum_check"])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=100)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert " 0 failures" in r.stdout
