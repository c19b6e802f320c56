"""homura_amd: a gfx950 (MI355X) implementation of homura's tensor elementwise, broadcast and
reduction path behind homura's own C ABI.

  homura_amd.capi    ctypes binding of include/homura_rocm.h (libhomura_rocm.so)
  homura_amd._host   the C++ host layer (Tensor, type promotion, broadcasting, dispatch), bound
                     with pybind11

Both are compiled in-tree by `__graft_entry__.build()`. There is no Python or CPU fallback for
the kernels: importing either module without its shared library raises ImportError.
"""
import os as _os

_HERE = _os.path.dirname(_os.path.abspath(__file__))
LIB_DIR = _os.path.join(_HERE, "lib")


def _require(path):
    if not _os.path.exists(path):
        raise ImportError(
            f"{path} is missing. Build the native libraries first: "
            "python -c 'import __graft_entry__ as g; g.build()'")


def load_host():
    """Imports the pybind11 host module (fails loudly if it has not been built)."""
    _require(_os.path.join(LIB_DIR, "libhomura_rocm.so"))
    from . import _host  # noqa: PLC0415
    return _host
