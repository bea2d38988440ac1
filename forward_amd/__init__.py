"""forward_amd -- MI355X (gfx950) implementation of Tencent/Forward's embedding-side plugin path.

The product is ``libfwdmi.so`` (hand-written HIP kernels, a C ABI and C++ plugin classes; sources
under ``csrc/``, declarations under ``include/``).  This package is the Python host side above
that ABI: a ctypes binding (``lib``), tensor-level wrappers of the kernel launchers (``ops``) and
a mirror of the plugin/creator/registry objects (``plugin``).  PyTorch is used only to own device
memory and streams.  There is no CPU fallback: every op raises if the library or a GPU is missing.
"""
from . import lib  # noqa: F401
