"""tidaldecode_amd -- MI355X (gfx950) implementation of TidalDecode's decode-attention path.

Layout mirrors the reference's ``tidal`` package where it is part of that path:

* ``tidaldecode_amd._kernels``   <->  ``tidal._kernels`` (PyBind operator module)
* ``tidaldecode_amd.utils``      <->  ``tidal.utils`` (operator wrappers, controller, KV cache)
* ``tidaldecode_amd.enable_tidal`` <-> ``src/enable_tidal.py`` (model patching)

Everything executes in ``libtidal_hip.so`` (hand-written HIP kernels behind a C ABI); importing
the package fails if the library has not been built.
"""
from . import _lib  # noqa: F401  (raises if libtidal_hip.so is missing)
from . import _kernels  # noqa: F401

__all__ = ["_kernels", "utils"]
__version__ = "0.1.0"
