"""The reference's python module `hetuCTR_partition` (csrc/partition/pybind.cc:6-25) on top of the C ABI, and the
driver its experimental/partition.py runs on it.

    import hetuctr_amd.partition as hetuCTR_partition
    p = hetuCTR_partition.partition(data, comm_mat, n_part, batch_size)
    p.refine_data(); p.refine_embed(); p.get_communication(); p.get_priority(); p.get_result() ...

Results are those of the reference run without OpenMP threads.  The sweeps run on the host; `cache_lists` (what the
reference's script does with numpy argsort) runs on the GPU.
"""
import ctypes as C
import time

import numpy as np

from . import capi


class _PartitionStruct:
    def __init__(self, input_data, comm_mat, n_part, batch_size, seed=1):
        data = np.asarray(input_data)
        comm = np.asarray(comm_mat)
        # the reference refuses arrays that are not C-contiguous (partition.cc:200-201) and asserts the shapes (:202-205)
        for name, arr in (("_input_data", data), ("_comm_mat", comm)):
            if not arr.flags.c_contiguous:
                raise RuntimeError("Array not continuous in C: " + name)
        if data.ndim != 2 or comm.ndim != 2 or comm.shape != (n_part, n_part):
            raise RuntimeError("partition: input_data must be 2-d and comm_mat n_part x n_part")
        data = np.ascontiguousarray(data, dtype=np.int32)
        comm = np.ascontiguousarray(comm, dtype=np.float32)
        h = C.c_void_p()
        capi._check(capi.lib().hctr_part_create(data.ctypes.data, data.shape[0], data.shape[1], comm.ctypes.data,
                                                int(n_part), int(batch_size), int(seed), C.byref(h)))
        self._h = h
        nd, ne, npart = C.c_size_t(), C.c_size_t(), C.c_int()
        capi._check(capi.lib().hctr_part_sizes(h, C.byref(nd), C.byref(ne), C.byref(npart)))
        self.n_data, self.n_embed, self.n_part = nd.value, ne.value, npart.value

    def refine_data(self):
        capi._check(capi.lib().hctr_part_refine_data(self._h))

    def refine_embed(self):
        capi._check(capi.lib().hctr_part_refine_embed(self._h))

    def get_communication(self):
        out = np.empty((self.n_part, self.n_part), np.float32)
        capi._check(capi.lib().hctr_part_get_communication(self._h, out.ctypes.data))
        return out

    def get_priority(self):
        out = np.empty((self.n_part, self.n_embed), np.float32)
        capi._check(capi.lib().hctr_part_get_priority(self._h, out.ctypes.data))
        return out

    def get_result(self):
        d, e = np.empty(self.n_data, np.int32), np.empty(self.n_embed, np.int32)
        capi._check(capi.lib().hctr_part_get_result(self._h, d.ctypes.data, e.ctypes.data))
        return d, e

    def get_data_cnt(self):
        d = np.empty(self.n_part, np.int32)
        capi._check(capi.lib().hctr_part_get_counts(self._h, d.ctypes.data, None))
        return d

    def get_embed_cnt(self):
        e = np.empty(self.n_part, np.int32)
        capi._check(capi.lib().hctr_part_get_counts(self._h, None, e.ctypes.data))
        return e

    def cache_lists(self, max_len=None):
        """Per part the embeddings it does not own, best cache candidates first (GPU).  Returns (lists, kernel ms)."""
        max_len = self.n_embed if max_len is None else int(max_len)
        buf = np.empty((self.n_part, max(max_len, 1)), np.int32)
        lens = (C.c_size_t * self.n_part)()
        ms = C.c_float()
        capi._check(capi.lib().hctr_part_cache_lists(self._h, max_len, buf.ctypes.data, lens, C.byref(ms)))
        return [buf[i, :lens[i]].copy() for i in range(self.n_part)], ms.value

    def close(self):
        if getattr(self, "_h", None):
            capi.lib().hctr_part_destroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def partition(input_data, comm_mat, n_part, batch_size, seed=1):
    """hetuCTR_partition.partition (csrc/partition/partition.cc:196-206)."""
    return _PartitionStruct(input_data, comm_mat, n_part, batch_size, seed)


def get_comm_mat(nrank, ngpus):
    """experimental/partition.py:20-30: 0 to oneself, 0.1 inside a node of `ngpus` ranks, 1 across nodes."""
    r = np.arange(nrank)
    mat = np.where(r[:, None] // ngpus == r[None, :] // ngpus, 0.1, 1.0)
    mat[r, r] = 0
    return mat.astype(np.float32)


def direct_partition(data, nparts, ngpus, batch_size, rerun, max_cache=None, log=None):
    """experimental/partition.py:32-61 without the file output: `rerun` rounds of both sweeps, then the dict the
    script saves ("embed_partition", "data_partition" and, per part, "<part>": its cache candidates, best first)."""
    log = log or (lambda *a: None)
    start = time.time()
    mat = get_comm_mat(nparts, ngpus)
    p = partition(data, mat, nparts, batch_size)
    log("Initial cost : {}".format(np.multiply(p.get_communication(), mat).sum()))
    for i in range(rerun):
        p.refine_data()
        p.refine_embed()
        log("Refine round {} : {}".format(i, np.multiply(p.get_communication(), mat).sum()))
    item_partition, idx_partition = p.get_result()
    log("Partition Time : ", time.time() - start)
    start = time.time()
    lists, _ = p.cache_lists(max_cache)
    log("Sort priority Time : ", time.time() - start)
    out = {"embed_partition": idx_partition, "data_partition": item_partition}
    for i in range(nparts):
        out[str(i)] = lists[i]
    p.close()
    return out
