"""The drop-in boundary without a GPU: the C-ABI library loads and exports exactly what include/*.h declares; the
python module `hetuCTR` has the reference's surface (csrc/pybind/pybind.cu:42-79); host-side argument checks."""
import ctypes
import glob
import inspect
import os
import re

import numpy as np
import pytest

import hetuctr_amd
from hetuctr_amd import capi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = []
    for h in glob.glob(os.path.join(ROOT, "include", "*.h")):
        text = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        names += re.findall(r"\b(hctr_[a-z_0-9]+)\s*\(", text)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(capi.LIB_PATH)
    declared = declared_symbols()
    assert len(declared) >= 14
    for name in declared:
        assert hasattr(lib, name), "include/*.h declares %s but the library does not export it" % name
    assert sorted(capi.SYMBOLS) == declared, "capi.SYMBOLS and the header disagree"
    lib.hctr_version.restype = ctypes.c_char_p
    assert b"gfx950" in lib.hctr_version()
    lib.hctr_stage_name.restype = ctypes.c_char_p
    names = [lib.hctr_stage_name(i).decode() for i in range(lib.hctr_stage_count())]
    assert "segment_sum_apply" in names and "gather" in names and "radix_sort" in names


def test_no_torch_or_cxx_types_in_the_header():
    text = open(os.path.join(ROOT, "include", "hetuctr_hip.h")).read()
    code = re.sub(r"/\*.*?\*/", "", text, flags=re.S)   # declarations only, comments stripped
    for bad in ("torch", "at::", "std::", "pybind", "template", "class ", "&"):
        assert bad not in code


def test_python_module_surface():
    m = hetuctr_amd.load_hetuCTR()
    assert {"HetuTable", "Initializer", "InitType", "seed", "_waittype"} <= set(dir(m))
    assert [n for n in m.InitType.__members__] == ["Zero", "Normal", "TruncatedNormal", "Uniform"]
    for meth in ("preprocess", "push_pull", "async_preprocess", "async_push_pull", "debug", "__repr__"):
        assert hasattr(m.HetuTable, meth)
    assert hasattr(m._waittype, "wait")
    doc = m.HetuTable.__init__.__doc__
    order = ["rank", "nrank", "device_id", "ip", "port", "length", "width", "pull_bound", "push_bound", "root_arr",
             "storage_arr", "init", "learning_rate", "verbose"]
    pos = [doc.index(k + ":") for k in order]
    assert pos == sorted(pos), "keyword order differs from csrc/pybind/pybind.cu:63-69"
    m.seed(3)  # accepted without a device
    m.seed(0)


def _no_gpu():
    import torch
    return not torch.cuda.is_available()


def test_constructor_argument_errors_are_runtime_errors():
    m = hetuctr_amd.load_hetuCTR()
    init = m.Initializer(m.InitType.Zero, 0, 0)
    kw = dict(rank=0, nrank=1, device_id=0, ip="127.0.0.1", port=1, length=8, width=4, pull_bound=0, push_bound=0,
              init=init, learning_rate=0.1, verbose=0)
    # a non-contiguous view is rejected like csrc/pybind/pybind.h:51-56 does when the dtype already matches
    with pytest.raises(RuntimeError, match="Array not continuous in C: storage_id_arr"):
        m.HetuTable(root_arr=np.zeros(8, np.uint8), storage_arr=np.arange(16, dtype=np.int64)[::2], **kw)
    with pytest.raises(RuntimeError, match="Array not continuous in C: root_id_arr"):
        m.HetuTable(root_arr=np.zeros(16, np.uint8)[::2], storage_arr=np.arange(8, dtype=np.int64), **kw)
    with pytest.raises(RuntimeError, match="length"):
        m.HetuTable(root_arr=np.zeros(7, np.uint8), storage_arr=np.arange(8, dtype=np.int64), **kw)
    with pytest.raises(TypeError):   # learning_rate has no default (csrc/pybind/pybind.cu:69)
        bad = dict(kw); bad.pop("learning_rate")
        m.HetuTable(root_arr=np.zeros(8, np.uint8), storage_arr=np.arange(8, dtype=np.int64), **bad)
    if _no_gpu():
        with pytest.raises(RuntimeError):  # loud failure, no CPU fallback
            m.HetuTable(root_arr=np.zeros(8, np.int64), storage_arr=np.arange(8), **kw)
        with pytest.raises(RuntimeError):
            capi.Table(0, 1, 0, "", 0, 8, 4, 0, 0, np.zeros(8, np.uint8), np.arange(8), ("Zero", 0, 0), 0.1)


def test_product_never_touches_the_oracle():
    """Nothing under hetuctr_amd/, include/ or bench.py's GPU path may import or link the CPU oracle."""
    for path in glob.glob(os.path.join(ROOT, "hetuctr_amd", "**", "*"), recursive=True):
        if os.path.isfile(path) and path.endswith((".py", ".hip", ".h", ".cpp")):
            text = open(path).read().lower()
            assert "oracle" not in text and "liborc" not in text, path


def test_bench_refuses_more_than_one_gpu():
    # the build runs on one GPU; asking for more must end with a message and a non-zero status, before any GPU work
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2", "--steps", "1"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "ONE GPU" in r.stderr and r.stdout.strip() == ""


def test_workload_byte_accounting():
    # algorithmic bytes per step: 4W(2N + 3U) + 41N + 81U, split into the stages bench.py reports
    from hetuctr_amd import workloads
    n, u, w = 1_703_936, 314_800, 128
    total = workloads.algorithmic_bytes(n, u, w)
    assert total == 4 * w * (2 * n + 3 * u) + 41 * n + 81 * u
    assert workloads.stage_bytes("segment_sum_apply", n, u, n, u, w) == 4 * w * n + 8 * w * u + 8 * n + 32 * u
    assert workloads.stage_bytes("gather", n, u, n, u, w) == 4 * w * n + 4 * w * u + 8 * n + 8 * u
    # the partitioner's cache-candidate kernels: 68 B per embedding for the keys at 8 parts, 76 B per (embedding, part)
    # for the four sort passes, 8 B per kept candidate
    assert workloads.cache_list_bytes(1000, 8, 100) == 1000 * 68 + 8 * 1000 * 76 + 8 * 100 * 8
