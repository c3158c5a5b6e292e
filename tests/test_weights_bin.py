"""moondream.bin reader (host side of the C ABI, no device call) against an independent restatement of the layout
(weights.zig:62-204, weights.py:106-125,161), and the reference's rejection cases."""
import ctypes as C
import struct

import numpy as np
import pytest

SMALL = dict(vocab=96, dim=64, hidden_dim=128, n_layers=2, n_heads=2, head_dim=32, rot_dim=16, theta=10000.0, max_seq=32)
SMALL_V = dict(dim=64, hidden_dim=96, n_layers=2, n_heads=2, head_dim=32)


def _cfg(moon, d):
    return moon.text_model.make_config(**{k: v for k, v in d.items() if k != "theta"})


def test_record_layout_is_the_closed_form(O):
    a = np.arange(6, dtype=np.float16).reshape(2, 3)
    rec = O.bin_record("t_ln_w", a)
    assert rec == struct.pack("<III", 6, 2, 6) + b"t_ln_w" + struct.pack("<2Q", 2, 3) + a.tobytes()
    assert len(rec) == 12 + 6 + 16 + 12


def test_reader_returns_what_the_restated_writer_wrote(moon, O, tmp_path):
    w = O.text_bin_tensors(O.synth_text_weights(SMALL, 3))
    w.update(O.vision_bin_tensors(O.synth_vision_weights(SMALL_V, 4)))
    io = dict(patch_dim=12, tokens=9, proj_hidden=48, out_dim=SMALL["dim"])
    w.update(O.vision_bin_tensors(O.synth_vision_io_weights(SMALL_V, io, 7)))  # includes the 3-d v_pos_embedding
    path = str(tmp_path / "moondream.bin")
    O.write_moondream_bin(path, w)
    ref = O.read_moondream_bin(path)
    with moon.weights.BinFile(path) as f:
        assert len(f) == len(w)
        got = list(f.tensors())
        assert [n for n, _ in got] == list(w.keys())  # file order
        for name, arr in got:
            assert arr.shape == ref[name].shape == w[name].shape
            assert np.array_equal(arr.view(np.uint16), np.asarray(w[name]).view(np.uint16))
        assert np.array_equal(f["t_fc1_b"].view(np.uint16), w["t_fc1_b"].view(np.uint16))
        with pytest.raises(KeyError):
            f["t_nothing"]
        tw = f.text_weights(_cfg(moon, SMALL))
        assert tw.t_Wqkv_w and tw.t_ln_out_b
        vw = f.vision_weights(moon.vision_model.make_config(**SMALL_V))
        assert vw.v_fc2_w and vw.v_norm_out_b
        iw = f.vision_io_weights(moon.vision_model.make_config(**SMALL_V), moon.vision_model.make_io_config(**io))
        assert iw.v_patch_embedding_linear_w and iw.v_pos_embedding and iw.v_proj_fc2_b
        with pytest.raises(moon.IncompatibleTensorShapes):  # a shape that disagrees with the configuration (error.ShapeMismatch)
            f.vision_io_weights(moon.vision_model.make_config(**SMALL_V), moon.vision_model.make_io_config(**dict(io, tokens=10)))


def test_package_writer_equals_restated_writer(moon, O, tmp_path):
    w = O.text_bin_tensors(O.synth_text_weights(SMALL, 1))
    a, b = str(tmp_path / "a.bin"), str(tmp_path / "b.bin")
    O.write_moondream_bin(a, w)
    moon.weights.write_bin(b, w)
    assert open(a, "rb").read() == open(b, "rb").read()


def _write(path, payload):
    with open(path, "wb") as f:
        f.write(payload)
    return str(path)


HDR = struct.pack("<II", 0x4D4F4F4E, 2)


@pytest.mark.parametrize("payload,text", [
    (struct.pack("<II", 0x4D4F4F4F, 2), "InvalidMagicNumber"),
    (struct.pack("<II", 0x4D4F4F4E, 3), "InvalidVersion"),
    (HDR + b"\x01\x00\x00", "InvalidHeader"),
    (HDR + struct.pack("<III", 257, 1, 1), "InvalidNameLength"),
    (HDR + struct.pack("<III", 6, 5, 1), "InvalidShapeLength"),
    (HDR + struct.pack("<III", 6, 1, 4) + b"t_ln_w" + struct.pack("<Q", 4) + b"\x00" * 6, "InvalidRead"),
    (HDR + struct.pack("<III", 5, 1, 1) + b"bogus" + struct.pack("<Q", 1) + b"\x00\x00", "UnknownTensorName"),
    (b"MOO", "InvalidRead"),
    # the record's element count disagrees with its dimensions
    (HDR + struct.pack("<III", 6, 1, 3) + b"t_ln_w" + struct.pack("<Q", 4) + b"\x00" * 8, "InvalidHeader"),
    # four dimensions whose product wraps 64 bits to a small number (2^20 each: 2^80 -> 0 elements, "fits" any file)
    (HDR + struct.pack("<III", 6, 4, 0) + b"t_ln_w" + struct.pack("<4Q", 1 << 20, 1 << 20, 1 << 20, 1 << 20) + b"\x00" * 64, "InvalidRead"),
])
def test_malformed_files_are_rejected_like_the_reference(moon, tmp_path, payload, text):
    path = _write(tmp_path / "bad.bin", payload)
    with pytest.raises(moon.weights.WeightFormatError, match=text):
        moon.weights.BinFile(path)


def test_missing_file(moon, tmp_path):
    with pytest.raises(moon.weights.WeightFormatError, match="cannot open"):
        moon.weights.BinFile(str(tmp_path / "nope.bin"))


def test_shape_mismatch_and_missing_tensor(moon, O, tmp_path):
    w = O.text_bin_tensors(O.synth_text_weights(SMALL, 3))
    path = str(tmp_path / "m.bin")
    O.write_moondream_bin(path, w)
    with moon.weights.BinFile(path) as f:
        other = dict(SMALL, hidden_dim=256)
        with pytest.raises(moon.IncompatibleTensorShapes, match="t_fc1_w.*ShapeMismatch"):  # weights.zig:177-181
            f.text_weights(_cfg(moon, other))
        with pytest.raises(moon.weights.WeightFormatError, match="v_Wqkv_w.*missing"):
            f.vision_weights(moon.vision_model.make_config(**SMALL_V))


def test_empty_tensor_list_is_a_valid_file(moon, tmp_path):
    with moon.weights.BinFile(_write(tmp_path / "e.bin", HDR)) as f:
        assert len(f) == 0
