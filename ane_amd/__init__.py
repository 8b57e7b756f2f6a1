"""MI355X (gfx950) implementations of the per-layer CPU ops of the maderix/ANE training loops.

The product is the C-ABI shared library ``libmi355_ops.so`` (see ``include/mi355_bridge.h``);
``ane_amd.bridge`` is its ctypes binding.  The binding is loaded on first use, so that ``ane_amd.build`` can
run when the library is absent or older than the header.
"""
import importlib

__all__ = ["bridge", "build"]


def __getattr__(name):
    if name in __all__:
        return importlib.import_module("." + name, __name__)
    raise AttributeError("module %r has no attribute %r" % (__name__, name))
