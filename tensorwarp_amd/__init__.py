"""tensorwarp_amd: MI355X (gfx950) implementation of TensorWarp's TW-Marlin W4A16
quantized-linear path.  The product is libtwmarlin_hip.so (C ABI in include/twmarlin.h);
this package is the thin Python mirror of the reference's Rust interface used by tests
and the benchmark."""
from . import _lib  # noqa: F401
from .quantize import *  # noqa: F401,F403
from .quantize import (DeviceError, ExpertBank, GpuTensor, GraphCapture, MarlinWeight, TWMarlinWeights,  # noqa: F401
                       WarpDevice)

__version__ = "0.1.0"
