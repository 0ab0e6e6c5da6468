"""ctypes front-end of the CPU oracle (``liborc.so``).  TEST INFRASTRUCTURE ONLY.

Imported by the test-suite, the smoke entry and the cpu_baseline leg of the benchmark; the product
never imports it.  ``Oracle`` steps R logical ranks in lock-step the way R reference processes would
(csrc/core/hetu_gpu_table.cu:9-65 per rank, csrc/core/all2all.cu between the stages).
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
INIT = {"Zero": 0, "Normal": 1, "Uniform": 2, "TruncatedNormal": 3}

# items of orc_fetch / hctr_debug_fetch (same numbering on both sides)
UNIQUE, SORTED_ARG, RUN_START, IDX_MAP, ROOT, OFFSET, SEND_CNT, RECV_CNT = range(8)
NEED_UPDATE, UPDATE_PREFIX, PUSH_CNT, PUSHRECV_CNT, OUTDATED, GOT, VERSION, UPDATES = range(8, 16)
EMBEDDING, PENDING, STORE_IDS, STATS, SIZES, KEYS = range(16, 22)
FLOAT_ITEMS = (EMBEDDING, PENDING)


def build(force=False):
    so = os.path.join(_HERE, "liborc.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "liborc.so"] + (["-B"] if force else []))
    return so


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = C.CDLL(build())
        _lib.orc_create.restype = C.c_void_p
        _lib.orc_create.argtypes = [C.c_int, C.c_size_t, C.c_size_t, C.c_longlong, C.c_longlong, C.c_void_p,
                                    C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_float, C.c_float, C.c_uint]
        _lib.orc_destroy.argtypes = [C.c_void_p]
        _lib.orc_set_parallel.argtypes = [C.c_void_p, C.c_int]
        _lib.orc_preprocess.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        _lib.orc_push_pull.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        _lib.orc_fetch.restype = C.c_longlong
        _lib.orc_fetch.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_size_t]
        _lib.orc_last_error.restype = C.c_char_p
        _lib.orc_num_threads.restype = C.c_int
        _lib.orc_init_values.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_float, C.c_float, C.c_uint]
    return _lib


def init_values(n, kind, a, b, seed=0):
    out = np.empty(n, dtype=np.float32)
    lib().orc_init_values(out.ctypes.data, n, INIT[kind], a, b, seed)
    return out


def ref_lib():
    """The reference's own initializer.cu compiled against the image's thrust, or None if not built."""
    so = os.path.join(_HERE, "_ref", "libref_initializer.so")
    if not os.path.exists(so):
        return None
    l = C.CDLL(so)
    l.ref_initialize_host.argtypes = [C.c_void_p, C.c_ulong, C.c_int, C.c_float, C.c_float, C.c_uint]
    return l


def _ptr_array(arrs):
    return (C.c_void_p * len(arrs))(*[a.ctypes.data if a is not None else None for a in arrs])


class Oracle:
    def __init__(self, nrank, length, width, pull_bound, push_bound, root_arr, storage_arrs,
                 init=("Zero", 0.0, 0.0), learning_rate=0.1, seed=0):
        self.R, self.length, self.W = nrank, length, width
        root = np.ascontiguousarray(root_arr, dtype=np.uint8)
        assert root.shape[0] == length
        st = [np.ascontiguousarray(s, dtype=np.int64) for s in storage_arrs]
        assert len(st) == nrank
        sizes = (C.c_size_t * nrank)(*[s.shape[0] for s in st])
        self._h = lib().orc_create(nrank, length, width, pull_bound, push_bound, root.ctypes.data,
                                   _ptr_array(st), sizes, INIT[init[0]], init[1], init[2], learning_rate, seed)
        if not self._h:
            raise RuntimeError(lib().orc_last_error().decode())

    def set_parallel(self, on):
        lib().orc_set_parallel(self._h, int(on))

    def preprocess(self, keys):
        """keys: list of R int64 arrays (one batch per rank)."""
        ks = [np.ascontiguousarray(k, dtype=np.int64) for k in keys]
        ns = (C.c_size_t * self.R)(*[k.shape[0] for k in ks])
        if lib().orc_preprocess(self._h, _ptr_array(ks), ns):
            raise RuntimeError(lib().orc_last_error().decode())
        self._n = [k.shape[0] for k in ks]

    def push_pull(self, grads):
        """grads: list of R float32 [Nprev, W] arrays or None (inference).  Returns list of dst arrays."""
        gs = [None if g is None else np.ascontiguousarray(g, dtype=np.float32) for g in grads]
        dsts = [np.zeros((n, self.W), dtype=np.float32) for n in self._n]
        if lib().orc_push_pull(self._h, _ptr_array(gs), _ptr_array(dsts)):
            raise RuntimeError(lib().orc_last_error().decode())
        return dsts

    def push_pull_pooled(self, grads_pooled, bag):
        """Sum-pooled bags of `bag` consecutive keys (no counterpart in the reference's API, which has no pooling:
        its drivers flatten a multi-hot sample into more keys, tests/benchmark.py:19-23, and pool outside).  Defined
        through the reference's own step: every key of a bag receives the bag's gradient row, and a bag's output is
        the sum of its keys' pulled rows in key order, one fp32 addition at a time, starting from the first row.
        grads_pooled: list of R float32 [Nprev / bag, W] arrays or None.  Returns R arrays [N / bag, W].
        Pinned by tests/test_oracle_update.py::test_pooled_* (bag 1 is the plain step; exact occurrence counts)."""
        gs = [None if g is None else np.repeat(np.ascontiguousarray(g, dtype=np.float32), bag, axis=0)
              for g in grads_pooled]
        out = []
        for d in self.push_pull(gs):
            assert d.shape[0] % bag == 0
            v = d.reshape(-1, bag, self.W)
            acc = v[:, 0, :].copy()
            for h in range(1, bag):
                acc = acc + v[:, h, :]          # elementwise float32 additions, in key order
            out.append(acc)
        return out

    def push_pull_into(self, grads, dsts):
        """Like push_pull with caller-provided float32 C-contiguous arrays (no allocation, no copies)."""
        if lib().orc_push_pull(self._h, _ptr_array(grads), _ptr_array(dsts)):
            raise RuntimeError(lib().orc_last_error().decode())

    def preprocess_raw(self, keys):
        """Like preprocess for int64 C-contiguous arrays, without conversions."""
        ns = (C.c_size_t * self.R)(*[k.shape[0] for k in keys])
        if lib().orc_preprocess(self._h, _ptr_array(keys), ns):
            raise RuntimeError(lib().orc_last_error().decode())
        self._n = [k.shape[0] for k in keys]

    def num_threads(self):
        return lib().orc_num_threads()

    def fetch(self, rank, which):
        n = lib().orc_fetch(self._h, rank, which, None, 0)
        dt = np.float32 if which in FLOAT_ITEMS else np.int64
        out = np.empty(max(n, 0), dtype=dt)
        lib().orc_fetch(self._h, rank, which, out.ctypes.data, n)
        return out

    def close(self):
        if self._h:
            lib().orc_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
