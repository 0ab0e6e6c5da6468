"""Seeded synthetic CTR-shaped sparse-id workloads (no dataset is needed or read).

A table is a concatenation of categorical fields; a sample holds one id per field (or `hot` ids per field for
multi-hot bags, flattened: the table API has no pooling, a bag is just more keys).  Ids of a field follow a
truncated Zipf law over the field's own range; by default the Zipf rank IS the local id (rank 0 = local id 0), i.e.
the hot rows of every field are its first rows and lie next to each other in HBM.  With `permute` every field maps
its ranks to local ids through a seeded permutation, so the hot rows are spread over the field's whole range.
Batches are laid out sample-major: key[s * nfields*hot + f*hot + h].
"""
import numpy as np

# name -> (rows, width, samples, fields, ids per field, zipf alpha or None for uniform, lr, init)
CONFIGS = {
    # CPU-runnable reference case
    "cfg1": dict(rows=1_000_000, width=16, samples=8192, fields=26, hot=1, alpha=None, lr=0.1,
                 init=("Uniform", -0.01, 0.01), single_field=True),
    # headline: ~33M rows in 26 log-uniform fields (10 .. 10M), dim 128
    "cfg2": dict(rows=33_762_577, width=128, samples=65536, fields=26, hot=1, alpha=1.05, lr=0.05,
                 init=("Normal", 0.0, 0.1), single_field=False),
    # the headline with the hot rows of every field scattered over the field (rank -> id through a permutation)
    "cfg2_permuted": dict(rows=33_762_577, width=128, samples=65536, fields=26, hot=1, alpha=1.05, lr=0.05,
                          init=("Normal", 0.0, 0.1), single_field=False, permute=True),
    # the same table and batch with uniform ids: nearly every key of a batch is distinct (no duplicates to sum)
    "cfg2_uniform": dict(rows=33_762_577, width=128, samples=65536, fields=26, hot=1, alpha=None, lr=0.05,
                         init=("Normal", 0.0, 0.1), single_field=True),
    # one GPU's shard of an 8-way partition of the cfg2 table: rank 0 owns 1/8 of the rows and caches the hottest
    # 10 % of the others; the peers live on the same GPU behind the loopback and only serve rank 0
    "cfg3": dict(rows=33_762_577, width=128, samples=65536, fields=26, hot=1, alpha=1.05, lr=0.05,
                 init=("Normal", 0.0, 0.1), single_field=False, nrank=8, cache_frac=0.10),
    # large table: 100M rows dim 128 (51.2 GB)
    "cfg4": dict(rows=100_000_000, width=128, samples=131072, fields=26, hot=1, alpha=1.2, lr=0.05,
                 init=("Normal", 0.0, 0.1), single_field=False),
    # multi-hot extremes, dim 64, 50M rows: heavy duplicates / ~all unique
    "cfg5_zipf": dict(rows=50_000_000, width=64, samples=32768, fields=26, hot=10, alpha=1.4, lr=0.05,
                      init=("Normal", 0.0, 0.1), single_field=False),
    "cfg5_uniform": dict(rows=50_000_000, width=64, samples=32768, fields=26, hot=10, alpha=None, lr=0.05,
                         init=("Normal", 0.0, 0.1), single_field=False),
}


def field_cardinalities(total_rows, nfields, seed=0, lo=1.0, hi=7.0):
    """Seeded log-uniform cardinalities 10^U(lo, hi), rescaled so that they sum to total_rows exactly."""
    rng = np.random.default_rng(seed)
    c = np.power(10.0, rng.uniform(lo, hi, nfields))
    c = np.maximum(10, np.floor(c * (total_rows / c.sum()))).astype(np.int64)
    c[np.argmax(c)] += total_rows - c.sum()
    assert c.sum() == total_rows and c.min() >= 10
    return c


class KeyStream:
    """Draws batches of global ids for one config."""

    def __init__(self, cfg, seed=0, scale=1.0):
        """scale < 1 shrinks rows and samples proportionally (tests, CPU samples)."""
        self.cfg = dict(cfg)
        self.rows = max(int(cfg["rows"] * scale), cfg["fields"] * 10)
        self.samples = max(int(cfg["samples"] * scale), 1)
        self.fields, self.hot, self.alpha = cfg["fields"], cfg["hot"], cfg["alpha"]
        if cfg.get("single_field"):
            self.card = np.full(self.fields, self.rows, dtype=np.int64)   # every field draws over the whole table
            self.base = np.zeros(self.fields, dtype=np.int64)
        else:
            self.card = field_cardinalities(self.rows, self.fields, seed)
            self.base = np.concatenate([[0], np.cumsum(self.card)[:-1]]).astype(np.int64)
        self.rng = np.random.default_rng(seed + 1)
        self.permute = bool(cfg.get("permute"))
        self.seed = seed
        self._perm = {}
        self._cdf = {}
        self.n = self.samples * self.fields * self.hot

    def _draw_field(self, f, count):
        c = int(self.card[f])
        if self.alpha is None:
            return self.rng.integers(0, c, size=count, dtype=np.int64)
        if f not in self._cdf:
            w = np.power(np.arange(1, c + 1, dtype=np.float64), -self.alpha)
            cdf = np.cumsum(w)
            cdf /= cdf[-1]
            self._cdf[f] = cdf
        u = self.rng.random(count)
        rank = np.minimum(np.searchsorted(self._cdf[f], u, side="left"), c - 1).astype(np.int64)
        if not self.permute:
            return rank
        if f not in self._perm:
            self._perm[f] = np.random.default_rng(self.seed + 1000 + f).permutation(c)
        return self._perm[f][rank]

    def batch(self):
        out = np.empty((self.samples, self.fields, self.hot), dtype=np.int64)
        for f in range(self.fields):
            out[:, f, :] = (self._draw_field(f, self.samples * self.hot) + self.base[f]).reshape(self.samples, self.hot)
        return out.reshape(-1)

    def release_tables(self):
        self._cdf.clear()
        self._perm.clear()


def shard_layout(ks, nrank, cache_frac, seed=0, cached_ranks=(0,)):
    """Owner of every id (seeded uniform, as the reference's benchmark draws it, tests/benchmark.py:16) and the
    resident ids of every rank: a rank in `cached_ranks` stores what it owns plus the hottest `cache_frac` of the ids
    it does not own (per field the ids of lowest Zipf rank, i.e. the first ids of the field); the others store
    what they own."""
    rng = np.random.default_rng(seed + 100)
    root = rng.integers(0, nrank, size=ks.rows, dtype=np.uint8)
    storage = [np.flatnonzero(root == r).astype(np.int64) for r in range(nrank)]
    for r in cached_ranks:
        hot = []
        for f in range(ks.fields):
            lo, c = int(ks.base[f]), int(ks.card[f])
            ids = np.arange(lo, lo + c, dtype=np.int64)
            remote = ids[root[lo:lo + c] != r]
            hot.append(remote[:int(np.ceil(cache_frac * remote.shape[0]))])
        storage[r] = np.concatenate([storage[r]] + hot)
    return root, storage


def partitioned_layout(ks, nrank, cache_frac, log_samples, batch_samples, rounds=3, cached_ranks=(0,), log=None):
    """Owners, resident ids and per-rank batches as the reference's offline flow produces them
    (experimental/partition.py): a click log of `log_samples` samples is drawn from the stream, the partitioner
    assigns its samples and the ids to `nrank` parts, a rank in `cached_ranks` stores what it owns plus the first
    `cache_frac` of its cache candidates (counted like shard_layout: a fraction of the ids it does not own), and a
    rank's batches are its own samples in log order, `batch_samples` at a time.  Ids beyond the largest id of the log
    are owned round-robin.  Returns (root, storage, batches per rank, info)."""
    from . import partition as hp
    saved = ks.samples
    ks.samples = log_samples
    data = ks.batch().reshape(log_samples, ks.fields * ks.hot).astype(np.int32)
    ks.samples = saved
    mat = hp.get_comm_mat(nrank, nrank)
    p = hp.partition(data, mat, nrank, batch_samples)
    cost = [float((p.get_communication() * mat).sum())]
    for _ in range(rounds):
        p.refine_data()
        p.refine_embed()
        cost.append(float((p.get_communication() * mat).sum()))
    part_of_sample, part_of_id = p.get_result()
    root = (np.arange(ks.rows) % nrank).astype(np.uint8)
    root[:p.n_embed] = part_of_id
    keep = {r: int(np.ceil(cache_frac * (ks.rows - int((root == r).sum())))) for r in cached_ranks}
    lists, kernel_ms = p.cache_lists(max(keep.values()) if keep else 0)
    p.close()
    storage = [np.flatnonzero(root == r).astype(np.int64) for r in range(nrank)]
    for r in cached_ranks:
        storage[r] = np.concatenate([storage[r], lists[r][:keep[r]].astype(np.int64)])
    batches = {}
    for r in range(nrank):
        mine = data[part_of_sample == r].astype(np.int64)
        full = mine.shape[0] // batch_samples
        batches[r] = [mine[b * batch_samples:(b + 1) * batch_samples].reshape(-1) for b in range(full)]
    info = {"log_samples": log_samples, "rounds": rounds, "cost_per_round": cost, "cache_list_kernel_ms": kernel_ms,
            "samples_per_rank": np.bincount(part_of_sample, minlength=nrank).tolist(),
            "ids_per_rank": np.bincount(root, minlength=nrank).tolist()}
    if log:
        log("partitioned layout: cost %s, samples per rank %s" % (["%.0f" % c for c in cost], info["samples_per_rank"]))
    return root, storage, batches, info


def sharded_extra_bytes(width, touched_cached, pushed, received, queried, returned, refreshed):
    """Bytes a step moves on top of algorithmic_bytes when rows are sharded and cached (same accounting): the
    pending-gradient store and update counter of touched cached rows, every pushed row written once (into its owner's
    receive area: id, count, row), applying received gradient rows, the query (id, version, directory slot, flag, both
    ways), every returned row read from the owner's table and written once (into the requester's buffer, with its
    version), refreshing cached rows.  No term for a transport: on one GPU the shards write into each other's buffers."""
    row = 4 * width
    return (touched_cached * (2 * row + 16) + pushed * (row + 16) + received * (2 * row + 32) +
            queried * 2 * (8 + 8 + 16 + 8) + returned * (2 * row + 8) + refreshed * (3 * row + 8))


def algorithmic_bytes(n_keys, n_unique, width, bag=1):
    """Bytes one full step must move at least, all rows local (one shard): gradient read and output write per
    key (per bag of `bag` keys when the lookups are sum-pooled), one gather read and one read-modify-write per unique
    row, plus the index traffic per key (41 B) and per unique key (81 B), counted with the reference's 8-byte
    indices."""
    row = 4 * width
    return row * (2 * (n_keys // bag) + 3 * n_unique) + 41 * n_keys + 81 * n_unique


def stage_bytes(stage, n_keys, n_unique, n_prev, u_prev, width, bag=1):
    """Algorithmic bytes of one launch of a W-wide stage (same accounting as algorithmic_bytes)."""
    row = 4 * width
    if stage == "segment_sum_apply":   # gradient rows + row RMW; sorted_arg read per key; offset, run_start, version RMW per unique
        return row * (n_prev // bag) + 2 * row * u_prev + 8 * n_prev + (8 + 8 + 16) * u_prev
    if stage == "gather":              # output write + unique-row read; idx_map read per key; offset read per unique
        return row * (n_keys // bag) + row * n_unique + 8 * n_keys + 8 * n_unique
    raise KeyError(stage)


def cache_list_bytes(n_embed, n_part, kept):
    """Algorithmic bytes of the partitioner's cache-candidate kernels: per embedding one counter row (4 B per part) and
    the owner read, one 4-byte key per part written; per part a 32-bit radix sort in four 8-bit passes (key read for
    the counts, key + position read and written for the move; the first pass reads no positions) and the kept list
    (position read, id written)."""
    keys = n_embed * (4 * n_part + 4 + 4 * n_part)
    sort = n_part * n_embed * (4 * (4 + 8 + 8) - 4)
    return keys + sort + n_part * min(kept, n_embed) * 8
