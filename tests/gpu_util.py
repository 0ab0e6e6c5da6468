"""Drives the HIP library through its C ABI next to the CPU oracle, on the same inputs."""
import numpy as np
import torch

from hetuctr_amd import capi
from oracle import oracle as orc

INT_ITEMS_PRE = [capi.UNIQUE, capi.SORTED_ARG, capi.RUN_START, capi.IDX_MAP, capi.ROOT, capi.OFFSET, capi.SEND_CNT,
                 capi.RECV_CNT, capi.NEED_UPDATE, capi.UPDATE_PREFIX, capi.PUSH_CNT, capi.PUSHRECV_CNT, capi.SIZES,
                 capi.KEYS]
INT_ITEMS_POST = [capi.OUTDATED, capi.GOT, capi.VERSION, capi.UPDATES, capi.STATS]
_port = [40000]


class Pair:
    """R shards on the GPU (one loopback group) and the same R logical ranks in the oracle."""

    def __init__(self, nrank, length, width, root, storage, init=("Zero", 0.0, 0.0), lr=0.1, bounds=(0, 0), seed=0,
                 with_oracle=True):
        self.R, self.W, self.length = nrank, width, length
        _port[0] += 1
        capi.seed(seed)
        self.tables = [capi.Table(r, nrank, 0, "127.0.0.1", _port[0], length, width, bounds[0], bounds[1], root,
                                  storage[r], init, lr, 0) for r in range(nrank)]
        self.oracle = orc.Oracle(nrank, length, width, bounds[0], bounds[1], root, storage, init=init,
                                 learning_rate=lr, seed=seed) if with_oracle else None
        self.keep = []

    def preprocess(self, keys, device_keys=False):
        keys = [np.ascontiguousarray(k, dtype=np.int64) for k in keys]
        self.n = [k.shape[0] for k in keys]
        if device_keys:
            dk = [torch.from_numpy(k).cuda() for k in keys]
            torch.cuda.synchronize()
            ptrs = [d.data_ptr() if d.numel() else 0 for d in dk]
            self.keep = dk
        else:
            ptrs = [k.ctypes.data for k in keys]
            self.keep = keys
        capi.group_preprocess(self.tables, ptrs, self.n)
        if self.oracle:
            self.oracle.preprocess(keys)

    def push_pull(self, grads):
        """grads: list of numpy [Nprev, W] or None.  Returns (gpu dsts, oracle dsts)."""
        dg = [None if g is None else torch.from_numpy(np.ascontiguousarray(g, dtype=np.float32)).cuda() for g in grads]
        dd = [torch.full((max(n, 1), self.W), float("nan"), device="cuda") for n in self.n]
        torch.cuda.synchronize()
        capi.group_push_pull(self.tables, [0 if g is None else (g.data_ptr() if g.numel() else 0) for g in dg],
                             [d.data_ptr() for d in dd])
        out = [d.cpu().numpy()[:n] for d, n in zip(dd, self.n)]
        ref = self.oracle.push_pull(grads) if self.oracle else None
        return out, ref

    def compare_ints(self, items, where=""):
        for r in range(self.R):
            for it in items:
                a, b = self.tables[r].fetch(it), self.oracle.fetch(r, it)
                assert a.shape == b.shape and np.array_equal(a, b), "item %d rank %d %s differs" % (it, r, where)

    def compare_state(self, rtol=1e-5, where=""):
        for r in range(self.R):
            for it in (capi.EMBEDDING, capi.PENDING):
                a, b = self.tables[r].fetch(it), self.oracle.fetch(r, it)
                assert a.shape == b.shape
                assert_close(a, b, rtol, "state item %d rank %d %s" % (it, r, where))

    def close(self):
        for t in self.tables:
            t.close()
        if self.oracle:
            self.oracle.close()


def assert_close(a, b, rtol=1e-5, what="", exact=True):
    """|a-b| <= rtol * max(|b|, scale) with scale = largest magnitude in b: 1e-5 relative, as stated for the
    updated fp32 embeddings, without blowing up on entries that cancel to ~0."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    assert a.shape == b.shape, what
    if a.size == 0:
        return
    assert np.isfinite(a).all(), what + ": non-finite values"
    if exact:
        # Gradient rows are added in the reference's order and nothing is contracted into fused multiply-adds
        # on either side, so the HIP result is expected to equal the CPU restatement bit for bit.  The
        # contractual bound (1e-5 relative) is checked below as well.
        nd = int((a != b).sum())
        assert nd == 0, "%s: %d of %d entries are not bit-identical (max abs diff %.3e)" % (what, nd, a.size, np.abs(a - b).max())
    scale = max(np.abs(b).max(), 1e-30)
    err = np.abs(a - b)
    tol = rtol * np.maximum(np.abs(b), 1e-2 * scale)
    bad = err > tol
    assert not bad.any(), "%s: %d of %d entries off, worst abs err %.3e (scale %.3e)" % (what, bad.sum(), a.size, err.max(), scale)
