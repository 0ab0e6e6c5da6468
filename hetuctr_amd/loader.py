"""The click log the reference's benchmark draws its batches from (tests/benchmark.py:19-31): an int64 array of
samples x fields sparse ids (its Criteo file `train_sparse_feats.npy`), sampled with replacement one batch at a time
and flattened into the key vector `preprocess` takes.

    log = SparseFeatureLog.synthetic("cfg2", samples=1_000_000)      # or SparseFeatureLog.load("feats.npy")
    keys = log.sample(2048)                                          # numpy int64[2048 * fields], like the reference
    dev = log.cuda(); keys = dev.sample(2048)                        # the same on the GPU, ready for preprocess
"""
import numpy as np


class SparseFeatureLog:
    def __init__(self, data):
        data = np.ascontiguousarray(data)
        if data.ndim != 2:
            raise ValueError("a click log is a samples x fields array")
        self.data = data.astype(np.int64, copy=False)      # tests/benchmark.py:30

    @classmethod
    def load(cls, path):
        """`np.load(path).astype(np.int64)` of the reference's loader (tests/benchmark.py:26-31); nothing is unpickled."""
        return cls(np.load(path, allow_pickle=False))

    def save(self, path):
        np.save(path, self.data)

    @classmethod
    def synthetic(cls, config="cfg2", samples=100_000, seed=0, scale=1.0):
        """A log of the same shape over one of the benchmark workloads: per-field Zipf ids, global id = field offset +
        local id (there is no Criteo file here)."""
        from . import workloads
        cfg = dict(workloads.CONFIGS[config])
        cfg["samples"] = int(np.ceil(samples / scale))      # scale shrinks the table, not the log
        ks = workloads.KeyStream(cfg, seed=seed, scale=scale)
        ks.samples, ks.n = samples, samples * ks.fields * ks.hot
        data = ks.batch().reshape(-1, ks.fields * ks.hot)
        ks.release_tables()
        log = cls(data)
        log.rows = ks.rows
        return log

    @property
    def samples(self):
        return self.data.shape[0]

    @property
    def fields(self):
        return self.data.shape[1]

    def sample(self, batch_size, rng=np.random):
        """get_sample_data of the reference (tests/benchmark.py:19-23): `batch_size` sample rows drawn with
        replacement by `rng.randint`, flattened."""
        idx = rng.randint(self.samples, size=batch_size)
        return self.data[idx].flatten()

    def cuda(self):
        return DeviceLog(self)


class DeviceLog:
    """The same log resident in HBM; batches are gathered by a kernel and never touch the host."""

    def __init__(self, log):
        import torch
        self.samples, self.fields = log.samples, log.fields
        self.data = torch.from_numpy(log.data).cuda()

    def sample(self, batch_size, rng=np.random, rows=None):
        """Device int64[batch_size * fields] for the same row numbers `SparseFeatureLog.sample` would draw (or for
        `rows`, a device int64 tensor of row numbers)."""
        import torch
        from . import capi
        if rows is None:
            rows = torch.from_numpy(rng.randint(self.samples, size=batch_size).astype(np.int64)).cuda()
        out = torch.empty(rows.numel() * self.fields, dtype=torch.int64, device="cuda")
        torch.cuda.synchronize()
        capi.sample_rows(self.data.data_ptr(), self.samples, self.fields, rows.data_ptr(), rows.numel(), out.data_ptr())
        return out
