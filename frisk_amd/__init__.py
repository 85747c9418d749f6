"""frisk_amd: gfx950 (MI355X) execution path for the tiled GEMM of the Frisk dialect.

  frisk_amd.runtime   ctypes binding of libfrisk_hip.so (include/frisk_hip.h)
  frisk_amd.frisk     the `frisk` Python package (IR builder + runtime), importable as `import frisk`
                      once frisk_amd has been imported
  frisk_amd.build     builds the HIP library and the builder extension in-tree
"""
import os as _os
import sys as _sys

_HERE = _os.path.dirname(_os.path.abspath(__file__))
if _HERE not in _sys.path:
    _sys.path.insert(0, _HERE)  # makes `import frisk` resolve to frisk_amd/frisk, the drop-in package name

from . import runtime  # noqa: E402,F401
