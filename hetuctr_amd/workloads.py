"""Seeded synthetic CTR-shaped sparse-id workloads (no dataset is needed or read).

A table is a concatenation of categorical fields; a sample holds one id per field (or `hot` ids per field for
multi-hot bags, flattened: the table API has no pooling, a bag is just more keys).  Ids of a field follow a
truncated Zipf law over the field's own range; the Zipf rank IS the local id (rank 0 = local id 0), i.e. the
hot rows of every field are its first rows.  Batches are laid out sample-major: key[s * nfields*hot + f*hot + h].
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
        return np.minimum(np.searchsorted(self._cdf[f], u, side="left"), c - 1).astype(np.int64)

    def batch(self):
        out = np.empty((self.samples, self.fields, self.hot), dtype=np.int64)
        for f in range(self.fields):
            out[:, f, :] = (self._draw_field(f, self.samples * self.hot) + self.base[f]).reshape(self.samples, self.hot)
        return out.reshape(-1)

    def release_tables(self):
        self._cdf.clear()


def algorithmic_bytes(n_keys, n_unique, width):
    """Bytes one full step must move at least, all rows local (one shard): gradient read and output write per
    key, one gather read and one read-modify-write per unique row, plus the index traffic per key (41 B) and
    per unique key (81 B), counted with the reference's 8-byte indices."""
    row = 4 * width
    return row * (2 * n_keys + 3 * n_unique) + 41 * n_keys + 81 * n_unique


def stage_bytes(stage, n_keys, n_unique, n_prev, u_prev, width):
    """Algorithmic bytes of one launch of a W-wide stage (same accounting as algorithmic_bytes)."""
    row = 4 * width
    if stage == "segment_sum_apply":   # gradient rows + row RMW; sorted_arg read per key; offset, run_start, version RMW per unique
        return row * n_prev + 2 * row * u_prev + 8 * n_prev + (8 + 8 + 16) * u_prev
    if stage == "gather":              # output write + unique-row read; idx_map read per key; offset read per unique
        return row * n_keys + row * n_unique + 8 * n_keys + 8 * n_unique
    raise KeyError(stage)
