"""MI355X-native embedding hot path of HetuCTR: HIP kernels behind a C ABI, plus python mirrors of the
reference's table interface.

``hetuctr_amd.capi``   ctypes binding of the C ABI (include/hetuctr_hip.h)
``hetuctr_amd.hetuCTR`` the pybind11 module with the reference's python surface (also importable as a
                        top-level ``hetuCTR`` after ``hetuctr_amd.install_as_hetuCTR()``)
``hetuctr_amd.partition`` the offline partitioner with the surface of the reference's ``hetuCTR_partition`` module
                        (importable under that name after ``hetuctr_amd.install_as_hetuCTR_partition()``)
"""
import importlib
import os
import sys

__all__ = ["capi", "load_hetuCTR", "install_as_hetuCTR", "install_as_hetuCTR_partition"]
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


def install_as_hetuCTR_partition():
    """Makes `import hetuCTR_partition` (as in the reference's experimental/partition.py:7) find hetuctr_amd.partition."""
    from . import partition
    sys.modules.setdefault("hetuCTR_partition", partition)
    return sys.modules["hetuCTR_partition"]
