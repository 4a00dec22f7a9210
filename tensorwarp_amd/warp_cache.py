"""Reader and writer of the reference's `.warp` pre-quantized weight cache container
(crates/loader/src/warp_cache.rs:1-21 for the byte format, :27-62 writer, :73-138 reader), used here
to persist repacked weights (MarlinWeight.export_blob) as U8 tensors so that a later load is one
host-to-device copy per projection.

File, all integers little-endian:
    8 bytes  b"WARP0001"
    u32      length of the config JSON, then the JSON (UTF-8)
    u32      number of tensors, then per tensor:
        u32 name length, name (UTF-8); u32 dtype (0 = F32, 1 = F16, 2 = U8/Q4); u32 ndims;
        ndims x u64 shape; u64 data length; data
"""
import os
import struct

import numpy as np

MAGIC = b"WARP0001"
DTYPE_F32, DTYPE_F16, DTYPE_U8 = 0, 1, 2
_NP_OF = {DTYPE_F32: np.float32, DTYPE_F16: np.uint16, DTYPE_U8: np.uint8}


class WarpTensor:
    """warp_cache.rs:65-70: one entry of a `.warp` file; f16 data stay raw uint16 bit patterns."""

    def __init__(self, name, dtype, shape, data):
        self.name, self.dtype, self.shape, self.data = name, int(dtype), tuple(int(d) for d in shape), data

    def array(self):
        if self.dtype not in _NP_OF:
            raise ValueError("tensor %r has unknown dtype %d" % (self.name, self.dtype))
        return np.frombuffer(self.data, _NP_OF[self.dtype]).reshape(self.shape)


def save_warp_cache(path, config_json, tensors):
    """tensors: iterable of (name, dtype, shape, data) with data bytes-like or a numpy array."""
    tensors = list(tensors)
    tmp = str(path) + ".tmp"
    with open(tmp, "wb") as f:
        f.write(MAGIC)
        cfg = config_json.encode("utf-8")
        f.write(struct.pack("<I", len(cfg)))
        f.write(cfg)
        f.write(struct.pack("<I", len(tensors)))
        for name, dtype, shape, data in tensors:
            raw = memoryview(np.ascontiguousarray(data)).cast("B") if isinstance(data, np.ndarray) else memoryview(data)
            nb = name.encode("utf-8")
            f.write(struct.pack("<I", len(nb)))
            f.write(nb)
            f.write(struct.pack("<II", int(dtype), len(shape)))
            for d in shape:
                f.write(struct.pack("<Q", int(d)))
            f.write(struct.pack("<Q", raw.nbytes))
            f.write(raw)
    os.replace(tmp, path)   # a reader never sees a half-written cache


def _read_exact(f, n):
    b = f.read(n)
    if len(b) != n:
        raise EOFError("truncated .warp file: wanted %d bytes, got %d" % (n, len(b)))
    return b


def load_warp_cache(path):
    """Returns (config_json, [WarpTensor]); raises ValueError on a wrong magic, EOFError on truncation."""
    with open(path, "rb") as f:
        magic = f.read(8)
        if magic != MAGIC:
            raise ValueError("not a .warp file (magic: %r)" % (magic,))
        (cfg_len,) = struct.unpack("<I", _read_exact(f, 4))
        config_json = _read_exact(f, cfg_len).decode("utf-8", errors="replace")
        (count,) = struct.unpack("<I", _read_exact(f, 4))
        tensors = []
        for _ in range(count):
            (name_len,) = struct.unpack("<I", _read_exact(f, 4))
            name = _read_exact(f, name_len).decode("utf-8", errors="replace")
            dtype, ndims = struct.unpack("<II", _read_exact(f, 8))
            shape = struct.unpack("<%dQ" % ndims, _read_exact(f, 8 * ndims)) if ndims else ()
            (data_len,) = struct.unpack("<Q", _read_exact(f, 8))
            tensors.append(WarpTensor(name, dtype, shape, _read_exact(f, data_len)))
    return config_json, tensors


def warp_cache_path(model_dir):
    """warp_cache.rs:141-143"""
    return os.path.join(model_dir, "model.warp")


def has_warp_cache(model_dir):
    """warp_cache.rs:146-159: the file exists and starts with the magic."""
    try:
        with open(warp_cache_path(model_dir), "rb") as f:
            return f.read(8) == MAGIC
    except OSError:
        return False
