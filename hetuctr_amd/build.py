"""Builds the native parts in-tree: libhetuctr_hip.so (HIP kernels + C ABI, gfx950) and the pybind11 module
`hetuCTR` that mirrors the reference's python surface (csrc/pybind/pybind.cu:42-79) on top of the C ABI.

    python -m hetuctr_amd.build            # build what is missing or out of date
    python -m hetuctr_amd.build --force    # rebuild everything
"""
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(CSRC, "build")
LIBDIR = os.path.join(HERE, "lib")
HIP_SOURCES = ["radix_sort.hip", "tile_sort.hip", "preprocess.hip", "push.hip", "pull.hip", "init.hip", "table.hip", "checkpoint.hip", "loader.hip", "partition.hip", "host_copy.hip", "c_api.hip"]
HEADERS = ["common.h", "host_copy.h", "kernels.h", "radix_sort.h", "tile_sort.h", "run_lists.h", "table.h", "partition.h", os.path.join("..", "..", "include", "hetuctr_hip.h")]
# packed-fp32 instruction selection is switched off for all device code; no fused multiply-add contraction, so
# that "sum * -lr" then "row + that" rounds twice like the CPU restatement it is checked against (fused
# operations are written explicitly where they are meant)
HIPFLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off", "-fvisibility=hidden", "-Wall", "-Wno-unused-function",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# host code of the partitioner's sweeps: AVX2 (no fused multiply-add is formed: contraction is off above)
EXTRA_FLAGS = {"partition.hip": ["-Xarch_host", "-march=x86-64-v3"], "host_copy.hip": ["-Xarch_host", "-march=x86-64-v3"]}
LIB = os.path.join(LIBDIR, "libhetuctr_hip.so")
PYMOD = os.path.join(LIBDIR, "hetuCTR" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def _newer(target, deps):
    if not os.path.exists(target):
        return False
    t = os.path.getmtime(target)
    return all(os.path.getmtime(d) <= t for d in deps if os.path.exists(d))


def _run(cmd):
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in p.stdout.splitlines() if "packed-fp32-ops" not in l)
    if p.returncode != 0:
        raise RuntimeError("command failed: %s\n%s" % (" ".join(cmd), out))
    return out


def build_hip(force=False, verbose=True):
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(LIBDIR, exist_ok=True)
    hdrs = [os.path.join(CSRC, h) for h in HEADERS]
    jobs = []
    objs = []
    for src in HIP_SOURCES:
        s = os.path.join(CSRC, src)
        o = os.path.join(OBJ, src + ".o")
        objs.append(o)
        if force or not _newer(o, [s] + hdrs):
            jobs.append(["hipcc"] + HIPFLAGS + EXTRA_FLAGS.get(src, []) + ["-c", s, "-o", o])
    if jobs:
        if verbose:
            print("hipcc: compiling %d file(s) for gfx950" % len(jobs), flush=True)
        with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
            for out in ex.map(_run, jobs):
                if out.strip() and verbose:
                    print(out)
    if jobs or force or not _newer(LIB, objs):
        _run(["hipcc", "--offload-arch=gfx950", "-shared", "-o", LIB] + objs)
        if verbose:
            print("linked", LIB, flush=True)
    return LIB


def build_pymod(force=False, verbose=True):
    src = os.path.join(CSRC, "pybind_module.cpp")
    if not os.path.exists(src):
        return None
    deps = [src, os.path.join(HERE, "..", "include", "hetuctr_hip.h")]
    if force or not _newer(PYMOD, deps):
        import pybind11
        inc = ["-I" + sysconfig.get_paths()["include"], "-I" + pybind11.get_include(), "-I" + os.path.join(HERE, "..", "include")]
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-Wall"] + inc +
             [src, "-o", PYMOD, "-L" + LIBDIR, "-lhetuctr_hip", "-Wl,-rpath,$ORIGIN", "-pthread"])
        if verbose:
            print("built", PYMOD, flush=True)
    return PYMOD


def build_all(force=False, verbose=True):
    build_hip(force, verbose)
    build_pymod(force, verbose)


if __name__ == "__main__":
    build_all(force="--force" in sys.argv)
