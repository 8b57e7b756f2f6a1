"""MI355X (gfx950) implementations of the per-layer CPU ops of the maderix/ANE training loops.

The product is the C-ABI shared library ``libmi355_ops.so`` (see ``include/mi355_bridge.h``);
``ane_amd.bridge`` is its ctypes binding.
"""
from . import bridge  # noqa: F401

__all__ = ["bridge"]
