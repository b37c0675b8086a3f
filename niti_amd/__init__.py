"""niti_amd: MI355X (gfx950) implementation of NITI's int8 training hot path.

  niti_amd.ops        tensor-level front end of the C ABI (include/niti_gfx950.h)
  niti_amd.shims      modules named like the reference's four CUDA extensions
  niti_amd.ti_torch   layer library with the reference's ti_torch API
  niti_amd.ti_net / ti_vgg / ti_loss   network container, VGG configs, integer loss gradient
"""
from . import _lib


def library_path() -> str:
    return _lib.SO_PATH


def require_library():
    """Loads libniti_gfx950.so or raises ImportError (there is no fallback path)."""
    return _lib.lib()
