"""Python modules with the names, signatures and return conventions of the reference's four
pybind11 CUDA extensions (cutlassconv_cuda, int8mm_cuda, int8conv_cuda, int8pool_cuda), backed
by libniti_gfx950.so.  ``install()`` registers them in ``sys.modules`` under the reference's
names so the reference's unmodified ``ti_torch.py`` (which does ``import cutlassconv_cuda`` ...)
runs on an MI355X."""
import sys

from . import cutlassconv_cuda, int8conv_cuda, int8mm_cuda, int8pool_cuda

_NAMES = ("cutlassconv_cuda", "int8mm_cuda", "int8conv_cuda", "int8pool_cuda")


def install(overwrite: bool = False) -> None:
    for name in _NAMES:
        if overwrite or name not in sys.modules:
            sys.modules[name] = globals()[name]


def check_input(t, name):
    """CHECK_INPUT of the reference bindings (e.g. cutlassconv.cpp:43-45)."""
    if not t.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not t.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
