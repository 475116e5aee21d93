"""guffin_amd — MI355X (gfx950) backend of Guffin's H1 speculative decode step.

The compute lives in libguffin_hip.so (hand-written HIP kernels behind a C ABI, see
include/guffin_hip.h).  This package only loads that library and passes device pointers
to it; PyTorch is used for device memory and streams, nothing else.  There is no CPU
fallback: importing `guffin_amd.hip` without the built library, or calling it without a
gfx950 device, raises.
"""
__all__ = ["hip", "synth", "build"]
