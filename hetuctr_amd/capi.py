"""ctypes binding of the C ABI (include/hetuctr_hip.h).  No fallback: if libhetuctr_hip.so is missing or does
not load, importing a table fails loudly."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# HETUCTR_LIB points at another build of the same library (kernel tuning experiments)
LIB_PATH = os.environ.get("HETUCTR_LIB") or os.path.join(_HERE, "lib", "libhetuctr_hip.so")
INIT = {"Zero": 0, "Normal": 1, "Uniform": 2, "TruncatedNormal": 3}
SYMBOLS = ["hctr_create", "hctr_destroy", "hctr_preprocess", "hctr_preprocess_noalloc", "hctr_push_pull", "hctr_push_pull_pooled",
           "hctr_group_preprocess", "hctr_group_push_pull", "hctr_group_push_pull_pooled", "hctr_seed", "hctr_repr", "hctr_debug", "hctr_last_error", "hctr_debug_fetch", "hctr_save", "hctr_load",
           "hctr_stream", "hctr_call_timing", "hctr_last_times", "hctr_last_push_ms", "hctr_defer_index", "hctr_stage_timing", "hctr_stage_count", "hctr_stage_name",
           "hctr_stage_times", "hctr_copy_probe", "hctr_sample_rows", "hctr_version", "hctr_part_create", "hctr_part_destroy",
           "hctr_part_sizes", "hctr_part_refine_data", "hctr_part_refine_embed", "hctr_part_get_communication",
           "hctr_part_get_priority", "hctr_part_get_result", "hctr_part_get_counts", "hctr_part_cache_lists"]

# items of hctr_debug_fetch (HCTR_F_*)
UNIQUE, SORTED_ARG, RUN_START, IDX_MAP, ROOT, OFFSET, SEND_CNT, RECV_CNT = range(8)
NEED_UPDATE, UPDATE_PREFIX, PUSH_CNT, PUSHRECV_CNT, OUTDATED, GOT, VERSION, UPDATES = range(8, 16)
EMBEDDING, PENDING, STORE_IDS, STATS, SIZES, KEYS = range(16, 22)
FLOAT_ITEMS = (EMBEDDING, PENDING)
NOALLOC_MAX_KEYS = 262144


class Config(C.Structure):
    _fields_ = [("rank", C.c_int), ("nrank", C.c_int), ("device_id", C.c_int), ("ip", C.c_char_p), ("port", C.c_int),
                ("length", C.c_size_t), ("width", C.c_size_t), ("pull_bound", C.c_longlong),
                ("push_bound", C.c_longlong), ("init_type", C.c_int), ("init_a", C.c_float), ("init_b", C.c_float),
                ("learning_rate", C.c_float), ("verbose", C.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libhetuctr_hip.so is not built: run `python -m hetuctr_amd.build`")
        l = C.CDLL(LIB_PATH)
        l.hctr_create.argtypes = [C.POINTER(Config), C.c_void_p, C.c_void_p, C.c_size_t, C.POINTER(C.c_void_p)]
        l.hctr_destroy.argtypes = [C.c_void_p]
        l.hctr_preprocess.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        l.hctr_preprocess_noalloc.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t]
        l.hctr_push_pull.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        l.hctr_push_pull_pooled.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        l.hctr_group_push_pull_pooled.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_size_t]
        l.hctr_group_preprocess.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        l.hctr_group_push_pull.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_void_p]
        l.hctr_seed.argtypes = [C.c_ulong]
        l.hctr_seed.restype = None
        l.hctr_repr.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t]
        l.hctr_debug.argtypes = [C.c_void_p, C.c_char_p, C.c_size_t]
        l.hctr_last_error.restype = C.c_char_p
        l.hctr_version.restype = C.c_char_p
        l.hctr_debug_fetch.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_size_t, C.POINTER(C.c_size_t)]
        l.hctr_save.argtypes = [C.c_void_p, C.c_char_p]
        l.hctr_load.argtypes = [C.c_void_p, C.c_char_p]
        l.hctr_stream.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
        l.hctr_call_timing.argtypes = [C.c_void_p, C.c_int]
        l.hctr_last_times.argtypes = [C.c_void_p, C.POINTER(C.c_float), C.POINTER(C.c_float)]
        l.hctr_last_push_ms.argtypes = [C.c_void_p, C.POINTER(C.c_float)]
        l.hctr_defer_index.argtypes = [C.c_void_p, C.c_int]
        l.hctr_stage_timing.argtypes = [C.c_void_p, C.c_int]
        l.hctr_stage_name.argtypes = [C.c_int]
        l.hctr_stage_name.restype = C.c_char_p
        l.hctr_stage_times.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int]
        l.hctr_copy_probe.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p]
        l.hctr_sample_rows.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]
        l.hctr_part_create.argtypes = [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_int, C.c_int, C.c_uint,
                                       C.POINTER(C.c_void_p)]
        l.hctr_part_sizes.argtypes = [C.c_void_p, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_int)]
        for name in ("destroy", "refine_data", "refine_embed"):
            getattr(l, "hctr_part_" + name).argtypes = [C.c_void_p]
        l.hctr_part_get_communication.argtypes = [C.c_void_p, C.c_void_p]
        l.hctr_part_get_priority.argtypes = [C.c_void_p, C.c_void_p]
        l.hctr_part_get_result.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        l.hctr_part_get_counts.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p]
        l.hctr_part_cache_lists.argtypes = [C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]
        _lib = l
    return _lib


def _check(rc):
    if rc != 0:
        raise RuntimeError(lib().hctr_last_error().decode())


def seed(n):
    lib().hctr_seed(int(n))


def copy_probe(dst_ptr, src_ptr, nbytes, repeats=5):
    """Average ms of a plain device copy of nbytes (read nbytes + write nbytes per launch)."""
    ms = C.c_float(0)
    _check(lib().hctr_copy_probe(dst_ptr, src_ptr, nbytes, repeats, C.byref(ms)))
    return ms.value


def sample_rows(log_ptr, n_samples, n_fields, rows_ptr, n_rows, out_ptr):
    """out[r * n_fields + f] = log[rows[r] * n_fields + f] on the device (all pointers device memory)."""
    _check(lib().hctr_sample_rows(log_ptr, n_samples, n_fields, rows_ptr, n_rows, out_ptr))


class Table:
    """One shard.  Arguments as hetuCTR.HetuTable (csrc/pybind/pybind.cu:63-69); `init` is (kind, a, b)."""

    def __init__(self, rank, nrank, device_id, ip, port, length, width, pull_bound, push_bound, root_arr,
                 storage_arr, init, learning_rate, verbose=0):
        root = np.ascontiguousarray(root_arr).astype(np.uint8, copy=False)
        storage = np.ascontiguousarray(storage_arr, dtype=np.int64)
        if root.shape[0] != length:
            raise RuntimeError("root_arr must hold `length` entries")
        kind = INIT[init[0]] if isinstance(init[0], str) else int(init[0])
        cfg = Config(rank, nrank, device_id, (ip or "").encode(), port, length, width, pull_bound, push_bound, kind,
                     float(init[1]), float(init[2]), float(learning_rate), verbose)
        h = C.c_void_p()
        _check(lib().hctr_create(C.byref(cfg), root.ctypes.data, storage.ctypes.data, storage.shape[0], C.byref(h)))
        self._h = h
        self.rank, self.nrank, self.width, self.length = rank, nrank, width, length

    def preprocess(self, ptr, n):
        _check(lib().hctr_preprocess(self._h, C.c_void_p(int(ptr)), n))

    def preprocess_noalloc(self, ptr, n):
        """preprocess that allocates nothing (device ids, at most NOALLOC_MAX_KEYS, buffers sized by earlier calls)."""
        _check(lib().hctr_preprocess_noalloc(self._h, C.c_void_p(int(ptr)), n))

    def push_pull(self, grad_ptr, dst_ptr):
        _check(lib().hctr_push_pull(self._h, C.c_void_p(int(grad_ptr) or None), C.c_void_p(int(dst_ptr) or None)))

    def push_pull_pooled(self, grad_ptr, dst_ptr, bag):
        """push_pull with sum-pooled bags of `bag` consecutive keys: one gradient / output row per bag."""
        _check(lib().hctr_push_pull_pooled(self._h, C.c_void_p(int(grad_ptr) or None),
                                           C.c_void_p(int(dst_ptr) or None), bag))

    def fetch(self, which):
        n = C.c_size_t()
        _check(lib().hctr_debug_fetch(self._h, which, None, 0, C.byref(n)))
        out = np.empty(n.value, dtype=np.float32 if which in FLOAT_ITEMS else np.int64)
        _check(lib().hctr_debug_fetch(self._h, which, out.ctypes.data, n.value, C.byref(n)))
        return out

    def save(self, path):
        """Rows, versions, pending gradients and update counters of this shard to one file."""
        _check(lib().hctr_save(self._h, os.fsencode(path)))

    def load(self, path):
        """Restores what save() wrote into a table of the same configuration; its batches start empty."""
        _check(lib().hctr_load(self._h, os.fsencode(path)))

    def stream(self):
        s = C.c_void_p()
        _check(lib().hctr_stream(self._h, C.byref(s)))
        return s.value

    def call_timing(self, on):
        """Switches the HIP events around the two calls on or off (last_times / last_push_ms need them on)."""
        _check(lib().hctr_call_timing(self._h, int(on)))

    def last_times(self):
        a, b = C.c_float(), C.c_float()
        _check(lib().hctr_last_times(self._h, C.byref(a), C.byref(b)))
        return a.value, b.value

    def last_push_ms(self):
        """Device time of the push stage of the last push_pull call (ms)."""
        a = C.c_float()
        _check(lib().hctr_last_push_ms(self._h, C.byref(a)))
        return a.value

    def defer_index(self, on):
        """False: preprocess returns only when all of its work is done (the reference's contract)."""
        _check(lib().hctr_defer_index(self._h, int(on)))

    def stage_timing(self, on):
        """Switches per-stage HIP-event timing on (resetting the accumulators) or off."""
        _check(lib().hctr_stage_timing(self._h, int(on)))

    def stage_times(self):
        """{stage name: (accumulated ms, bracketed intervals)} since stage_timing(True)."""
        n = lib().hctr_stage_count()
        ms = (C.c_double * n)()
        calls = (C.c_longlong * n)()
        _check(lib().hctr_stage_times(self._h, ms, calls, n))
        return {lib().hctr_stage_name(i).decode(): (ms[i], calls[i]) for i in range(n)}

    def __repr__(self):
        buf = C.create_string_buffer(256)
        lib().hctr_repr(self._h, buf, 256)
        return buf.value.decode()

    def debug(self):
        buf = C.create_string_buffer(512)
        lib().hctr_debug(self._h, buf, 512)
        return buf.value.decode()

    def close(self):
        if getattr(self, "_h", None):
            lib().hctr_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _ptrs(vals):
    return (C.c_void_p * len(vals))(*[C.c_void_p(int(v) or None) for v in vals])


def group_preprocess(tables, key_ptrs, ns):
    """Lock-step preprocess of every shard of a loopback group from one caller."""
    hs = (C.c_void_p * len(tables))(*[t._h for t in tables])
    sizes = (C.c_size_t * len(tables))(*ns)
    _check(lib().hctr_group_preprocess(hs, len(tables), _ptrs(key_ptrs), sizes))


def group_push_pull(tables, grad_ptrs, dst_ptrs):
    hs = (C.c_void_p * len(tables))(*[t._h for t in tables])
    _check(lib().hctr_group_push_pull(hs, len(tables), _ptrs(grad_ptrs), _ptrs(dst_ptrs)))


class GroupStep:
    """The two lock-step calls of a loopback group with their argument arrays built once: a caller that steps the same
    buffers again and again (a benchmark loop, a training loop with fixed staging buffers) pays two foreign calls per
    step and no array construction."""

    def __init__(self, tables, key_ptrs, ns, grad_ptrs, dst_ptrs):
        self._lib = lib()
        self._n = len(tables)
        self._hs = (C.c_void_p * self._n)(*[t._h for t in tables])
        self._keys = _ptrs(key_ptrs)
        self._sizes = (C.c_size_t * self._n)(*ns)
        self._grads = _ptrs(grad_ptrs)
        self._dsts = _ptrs(dst_ptrs)

    def preprocess(self):
        if self._lib.hctr_group_preprocess(self._hs, self._n, self._keys, self._sizes):
            _check(1)

    def push_pull(self):
        if self._lib.hctr_group_push_pull(self._hs, self._n, self._grads, self._dsts):
            _check(1)


def group_push_pull_pooled(tables, grad_ptrs, dst_ptrs, bag):
    hs = (C.c_void_p * len(tables))(*[t._h for t in tables])
    _check(lib().hctr_group_push_pull_pooled(hs, len(tables), _ptrs(grad_ptrs), _ptrs(dst_ptrs), bag))
