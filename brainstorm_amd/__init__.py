"""brainstorm_amd: an MI355X (gfx950) compute handler for the brainstorm neural-network library.

``HipHandler`` implements brainstorm's ``Handler`` interface on top of
``libbship.so``, a C-ABI library of hand-written HIP kernels (see
``include/bship.h``). ``DeviceArray`` is the array type it works on.
"""
from .device_array import DeviceArray
from .handler_api import HANDLER_METHODS, Handler

__all__ = ["DeviceArray", "Handler", "HipHandler", "HANDLER_METHODS"]
__version__ = "0.1.0"


def __getattr__(name):
    # HipHandler loads libbship.so on import; keep `import brainstorm_amd` itself light so that
    # host-only tools (the build script, the array type) work before the library is built.
    if name == "HipHandler":
        from .hip_handler import HipHandler
        return HipHandler
    raise AttributeError("module 'brainstorm_amd' has no attribute %r" % name)
