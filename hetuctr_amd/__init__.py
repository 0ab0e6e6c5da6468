"""MI355X-native embedding hot path of HetuCTR: HIP kernels behind a C ABI, plus python mirrors of the
reference's table interface.

``hetuctr_amd.capi``   ctypes binding of the C ABI (include/hetuctr_hip.h)
``hetuctr_amd.hetuCTR`` the pybind11 module with the reference's python surface (also importable as a
                        top-level ``hetuCTR`` after ``hetuctr_amd.install_as_hetuCTR()``)
"""
import importlib
import os
import sys

__all__ = ["capi", "load_hetuCTR", "install_as_hetuCTR"]
LIBDIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib")


def load_hetuCTR():
    """Imports the compiled `hetuCTR` module from hetuctr_amd/lib (it must have been built)."""
    if "hetuCTR" in sys.modules:
        return sys.modules["hetuCTR"]
    if LIBDIR not in sys.path:
        sys.path.insert(0, LIBDIR)
    try:
        return importlib.import_module("hetuCTR")
    except ImportError as e:
        raise ImportError("the hetuCTR extension is not built: run `python -m hetuctr_amd.build` (%s)" % e)


install_as_hetuCTR = load_hetuCTR
