"""MI355X (gfx950) quantized-weight matmuls for oxinfer: Python binding of liboxinfer_hip.so.

The product is the shared library (C ABI in include/oxhip.h); this package loads it for tests and
measurement and mirrors the reference's `gpu::Backend` surface (src/gpu.rs:151-294) in `HipBackend`.
There is no CPU fallback here: without the built library, or without a gfx950 device, it raises.
"""
from .hip import HipBackend, DeviceWeight, QAct, library_path, load_library  # noqa: F401
