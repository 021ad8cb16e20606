"""zigrad_amd: an MI355X (gfx950) device backend for Zigrad's device-op hot path.

The product is the C-ABI shared library declared in include/zg_hip.h (hand-written HIP kernels);
this package is the thin host side above it: `HipDevice` mirrors the reference's DeviceReference
interface and `trainers` issues the reference's op sequences for the benchmark configurations.
"""
from .device import DevBuf, Event, HipDevice  # noqa: F401
from ._lib import Library, ZgHipError, lib  # noqa: F401
