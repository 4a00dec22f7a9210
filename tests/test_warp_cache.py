"""The `.warp` container (crates/loader/src/warp_cache.rs:1-21) on the CPU: the byte layout against a file
assembled by hand, round trips, and the reader's error behaviour."""
import struct

import numpy as np
import pytest

from tensorwarp_amd import warp_cache as W


def test_byte_layout_matches_the_format_description(tmp_path):
    data = bytes(range(12))
    path = tmp_path / "model.warp"
    W.save_warp_cache(path, '{"a":1}', [("w.q", W.DTYPE_U8, (3, 4), data)])
    want = (b"WARP0001" + struct.pack("<I", 7) + b'{"a":1}' + struct.pack("<I", 1) +
            struct.pack("<I", 3) + b"w.q" + struct.pack("<I", 2) + struct.pack("<I", 2) +
            struct.pack("<QQ", 3, 4) + struct.pack("<Q", 12) + data)
    assert path.read_bytes() == want
    assert W.has_warp_cache(str(tmp_path)) and W.warp_cache_path(str(tmp_path)) == str(path)


def test_round_trip_of_mixed_tensors(tmp_path):
    rng = np.random.default_rng(5)
    f32 = rng.standard_normal((4, 5)).astype(np.float32)
    f16 = rng.standard_normal(9).astype(np.float16).view(np.uint16)
    u8 = rng.integers(0, 256, 1000, dtype=np.uint8)
    path = tmp_path / "m.warp"
    W.save_warp_cache(path, "{}", [("norm", W.DTYPE_F32, f32.shape, f32), ("scales", W.DTYPE_F16, f16.shape, f16),
                                   ("blob", W.DTYPE_U8, u8.shape, u8), ("empty", W.DTYPE_U8, (0,), b"")])
    cfg, tensors = W.load_warp_cache(path)
    assert cfg == "{}" and [t.name for t in tensors] == ["norm", "scales", "blob", "empty"]
    assert np.array_equal(tensors[0].array(), f32) and tensors[0].shape == (4, 5)
    assert np.array_equal(tensors[1].array(), f16)
    assert np.array_equal(tensors[2].array(), u8)
    assert tensors[3].array().size == 0


def test_reader_rejects_foreign_and_truncated_files(tmp_path):
    bad = tmp_path / "x.warp"
    bad.write_bytes(b"WARP0002" + b"\0" * 16)
    with pytest.raises(ValueError):
        W.load_warp_cache(bad)
    good = tmp_path / "g.warp"
    W.save_warp_cache(good, "{}", [("t", W.DTYPE_U8, (64,), bytes(64))])
    cut = tmp_path / "c.warp"
    cut.write_bytes(good.read_bytes()[:-10])
    with pytest.raises(EOFError):
        W.load_warp_cache(cut)
    assert not W.has_warp_cache(str(tmp_path / "nowhere"))
