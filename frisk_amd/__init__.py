"""frisk_amd: gfx950 (MI355X) execution path for the tiled GEMM of the Frisk dialect.

  frisk_amd.runtime   ctypes binding of libfrisk_hip.so (include/frisk_hip.h)
  frisk_amd.build     builds the library in-tree with hipcc
"""
from . import runtime  # noqa: F401
