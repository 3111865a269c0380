"""nesgpu_amd: MI355X-native population-batched binary layer forward path.

Python host layer over libnesbin.so (hand-written gfx950 kernels behind a C ABI).  The sub-packages
mirror the reference's layout: ``extensions.booleanOperations`` (op functions), ``extensions.boolop_cuda``
/ ``extensions.boolutil_cuda`` (torch-extension namespaces) and ``modules.binary`` (perturbed layers).
"""
import sys as _sys

__version__ = "0.1.0"


def install_as_reference_modules():
    """Register this package under the reference's import names so that unmodified reference code
    (`from extensions import booleanOperations`, `from modules import binary`) picks it up."""
    from . import extensions, modules
    from .extensions import booleanOperations, boolop_cuda, boolutil_cuda
    from .modules import base, binary
    _sys.modules.setdefault("extensions", extensions)
    _sys.modules.setdefault("extensions.booleanOperations", booleanOperations)
    _sys.modules.setdefault("boolop_cuda", boolop_cuda)
    _sys.modules.setdefault("boolutil_cuda", boolutil_cuda)
    _sys.modules.setdefault("modules", modules)
    _sys.modules.setdefault("modules.base", base)
    _sys.modules.setdefault("modules.binary", binary)
