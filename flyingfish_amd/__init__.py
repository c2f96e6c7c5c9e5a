"""flyingfish_amd: MI355X-native kernels for flyingfish's quantized MoE expert-FFN path.

The product is ``libffmoe.so`` (hand-written HIP for gfx950 behind the C ABI of ``include/ffmoe.h``).
This package is the host-side harness over it: ctypes bindings (``capi``), operator objects that
mirror the reference's Rust operator structs (``ops``), and seeded synthetic inputs (``synth``).
PyTorch is used only to own device memory and streams.
"""
from . import capi  # noqa: F401

__all__ = ["capi"]
