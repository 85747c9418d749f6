"""`frisk`: the Python front end of the Frisk IR builder, with the same names as the
reference package (python/frisk/__init__.py:1-4): everything in `frisk_ffi.ir`, plus
`FriskHelper`, `create_context`, `create_session`; and `runtime`, which executes a
tiled-GEMM kernel on gfx950 through libfrisk_hip.so."""
import os as _os

from .frisk_ffi.ir import *  # noqa: F401,F403
from .frisk_ffi import ir, runtime  # noqa: F401
from .common.utils import FriskHelper, create_context, create_session  # noqa: F401

runtime.set_library(_os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "lib", "libfrisk_hip.so"))

__all__ = [name for name in globals().keys() if not name.startswith("_")]
