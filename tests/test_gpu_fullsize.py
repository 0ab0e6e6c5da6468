"""The benchmark configurations (hetuctr_amd.workloads.CONFIGS) at their full sizes on the GPU.

cfg2 (headline) runs next to the CPU oracle and must agree bit for bit.  The larger ones are checked through
properties that do not need an oracle of that size: the integer outputs against numpy's own unique / lexsort on
the same keys, and the update arithmetic with integer-valued gradients, whose sums are exact in any order, against
a float64 scatter-add (np.add.at)."""
import numpy as np
import pytest
import torch

from hetuctr_amd import capi, workloads
from oracle import oracle as orc
from tests.gpu_util import assert_close

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def single_table(rows, width, init, lr):
    capi.seed(0)
    return capi.Table(0, 1, 0, "127.0.0.1", 0, rows, width, 0, 0, np.zeros(rows, np.uint8),
                      np.arange(rows, dtype=np.int64), init, lr, 0)


def check_integers(t, keys):
    """unique / sorted_arg / run_start / idx_map of the table's current batch against numpy on the same keys."""
    n = keys.shape[0]
    uniq, first, inverse, counts = np.unique(keys, return_index=True, return_inverse=True, return_counts=True)
    assert np.array_equal(t.fetch(capi.UNIQUE), uniq)
    run_start = np.concatenate([[0], np.cumsum(counts)])
    assert np.array_equal(t.fetch(capi.RUN_START), run_start)
    assert np.array_equal(t.fetch(capi.IDX_MAP), inverse.reshape(-1))
    sa = t.fetch(capi.SORTED_ARG)
    assert np.array_equal(sa, np.argsort(keys, kind="stable"))   # stable: equal keys in ascending position
    assert np.array_equal(t.fetch(capi.OFFSET), uniq)            # identity storage: offset == id
    assert t.fetch(capi.SIZES)[:2].tolist() == [n, uniq.shape[0]]
    return uniq, counts


def test_cfg2_headline_bit_exact_against_oracle():
    cfg = workloads.CONFIGS["cfg2"]
    ks = workloads.KeyStream(cfg, seed=0)
    rows, width, n = ks.rows, cfg["width"], ks.n
    say("cfg2 full size: %d rows x %d, %d keys" % (rows, width, n))
    t = single_table(rows, width, ("Zero", 0.0, 0.0), cfg["lr"])
    o = orc.Oracle(1, rows, width, 0, 0, np.zeros(rows, np.uint8), [np.arange(rows, dtype=np.int64)],
                   init=("Zero", 0.0, 0.0), learning_rate=cfg["lr"])
    o.set_parallel(True)
    rng = np.random.default_rng(3)
    dst = torch.empty((n, width), device="cuda")
    ref = np.empty((n, width), np.float32)
    grad = None
    for step in range(3):
        keys = ks.batch()
        dk = torch.from_numpy(keys).cuda()
        dg = None if grad is None else torch.from_numpy(grad).cuda()
        torch.cuda.synchronize()
        t.preprocess(dk.data_ptr(), n)
        t.push_pull(0 if dg is None else dg.data_ptr(), dst.data_ptr())
        o.preprocess_raw([keys])
        o.push_pull_into([grad], [ref])
        for item in (capi.UNIQUE, capi.SORTED_ARG, capi.RUN_START, capi.IDX_MAP, capi.OFFSET):
            assert np.array_equal(t.fetch(item), o.fetch(0, item)), "item %d step %d" % (item, step)
        got = dst.cpu().numpy()
        assert np.array_equal(got, ref), "step %d: %d rows differ" % (step, int((got != ref).any(axis=1).sum()))
        assert_close(got, ref, 1e-5, "cfg2 step %d" % step)
        grad = rng.normal(0, 1e-3, size=(n, width)).astype(np.float32)
    u = o.fetch(0, orc.UNIQUE)
    ver_gpu = t.fetch(capi.VERSION)
    assert np.array_equal(ver_gpu, o.fetch(0, orc.VERSION))
    t.close(); o.close()


@pytest.mark.parametrize("name", ["cfg2_uniform", "cfg4", "cfg5_zipf", "cfg5_uniform"])
def test_large_configs_by_properties(name):
    cfg = workloads.CONFIGS[name]
    ks = workloads.KeyStream(cfg, seed=0)
    rows, width, n = ks.rows, cfg["width"], ks.n
    say("%s full size: %d rows x %d, %d keys" % (name, rows, width, n))
    t = single_table(rows, width, ("Zero", 0.0, 0.0), -1.0)      # lr = -1: rows accumulate the gradients
    dst = torch.empty((n, width), device="cuda")
    rng = np.random.default_rng(5)
    total = {}                                                   # id -> accumulated column-0 value (float64)
    acc = np.zeros(0)
    prev_keys, prev_g = None, None
    table_sum = np.zeros(width)
    for step in range(3):
        keys = ks.batch()
        dk = torch.from_numpy(keys).cuda()
        if prev_keys is None:
            dg = None
        else:
            # integer-valued gradients in [-3, 3]: every partial sum is exact in fp32, in any order
            g_int = rng.integers(-3, 4, size=(prev_keys.shape[0], 1)).astype(np.float32)
            prev_g = g_int
            dg = (torch.from_numpy(g_int).cuda() * torch.arange(1, width + 1, device="cuda", dtype=torch.float32)).contiguous()
        torch.cuda.synchronize()
        t.preprocess(dk.data_ptr(), n)
        t.push_pull(0 if dg is None else dg.data_ptr(), dst.data_ptr())
        uniq, counts = check_integers(t, keys)
        if prev_keys is not None:
            u_prev, inv = np.unique(prev_keys, return_inverse=True)
            s = np.zeros(u_prev.shape[0])
            np.add.at(s, inv.reshape(-1), prev_g[:, 0].astype(np.float64))
            for k, v in zip(u_prev[s != 0].tolist(), s[s != 0].tolist()):
                total[k] = total.get(k, 0.0) + v
        got = dst.cpu().numpy()
        expect0 = np.array([total.get(k, 0.0) for k in uniq.tolist()])[np.searchsorted(uniq, keys)]
        assert np.array_equal(got[:, 0], expect0.astype(np.float32)), "%s step %d column 0" % (name, step)
        # column w holds (w+1) times column 0, exactly
        assert np.array_equal(got[:, width - 1], (expect0 * width).astype(np.float32))
        # equal keys pulled equal rows
        first_pos = np.unique(keys, return_index=True)[1]
        assert np.array_equal(got, got[first_pos][np.searchsorted(uniq, keys)])
        prev_keys = keys
    ver = t.fetch(capi.VERSION)
    assert int(ver.sum()) == 2 * n                               # two batches were pushed, one count per key
    t.close()


@pytest.mark.parametrize("feeders,bounds,steps", [((0,), (0, 0), 3), (tuple(range(8)), (2, 3), 5)])
def test_cfg3_eight_shards_full_size_bit_exact(feeders, bounds, steps):
    """The 8-shard configuration at its full size (33.8M rows x 128 over eight shards of one loopback group) next to the
    CPU oracle with the same eight logical ranks.  First the benchmark's own case: rank 0 feeds full batches and caches
    the hottest tenth of its remote rows, the peers only serve, bounds 0/0.  Then every rank feeds an eighth of a
    batch, every rank caches, and the bounds let rows go stale (pull 2, push 3), so that pending gradients, refreshed
    rows and pushes from several sources to one row all occur at this size."""
    from tests.gpu_util import Pair, INT_ITEMS_PRE, INT_ITEMS_POST
    cfg = workloads.CONFIGS["cfg3"]
    R, width = cfg["nrank"], cfg["width"]
    ks = workloads.KeyStream(cfg, seed=0)
    root, storage = workloads.shard_layout(ks, R, cfg["cache_frac"], cached_ranks=feeders)
    say("cfg3 full size: %d rows x %d over %d shards, feeders %s, bounds %s, %d keys per full batch" %
        (ks.rows, width, R, feeders, bounds, ks.n))
    p = Pair(R, ks.rows, width, root, storage, init=("Zero", 0.0, 0.0), lr=cfg["lr"], bounds=bounds)
    p.oracle.set_parallel(True)
    rng = np.random.default_rng(11)
    share = ks.n // len(feeders)
    empty = np.zeros(0, np.int64)
    grads = [None] * R
    light = [it for it in INT_ITEMS_PRE if it not in (capi.KEYS, capi.IDX_MAP)] # those two are covered at small sizes
    for step in range(steps + 1):
        last = step == steps                       # the last step pulls without gradients (inference)
        full = ks.batch()
        if len(feeders) == 1:
            keys = [full if r == feeders[0] else empty for r in range(R)]
        else:
            keys = [full[r * share:(r + 1) * share] if r in feeders else empty for r in range(R)]
        p.preprocess(keys, device_keys=True)
        p.compare_ints(light, "step %d" % step)
        out, ref = p.push_pull([None] * R if last else grads)
        for r in feeders:
            assert np.array_equal(out[r], ref[r]), "step %d rank %d: %d rows differ" % (
                step, r, int((out[r] != ref[r]).any(axis=1).sum()))
        p.compare_ints([capi.OUTDATED, capi.GOT, capi.STATS, capi.UPDATES], "step %d" % step)
        grads = [rng.normal(0, 1e-3, size=(k.shape[0], width)).astype(np.float32) if k.shape[0] else None for k in keys]
        say("  step %d ok; stats of rank 0 (hit, miss, refreshed, pushed, served, received): %s" %
            (step, p.tables[0].fetch(capi.STATS)[:6].tolist()))
    for r in range(R):                             # versions of all rows, pending gradients of all cached rows
        assert np.array_equal(p.tables[r].fetch(capi.VERSION), p.oracle.fetch(r, capi.VERSION)), "versions rank %d" % r
        assert np.array_equal(p.tables[r].fetch(capi.PENDING), p.oracle.fetch(r, capi.PENDING)), "pending rank %d" % r
    if len(feeders) > 1:
        st = np.sum([p.tables[r].fetch(capi.STATS)[:6] for r in range(R)], axis=0)
        assert st[0] > 0, "no cached row was fresh enough to be used: the bounds were meant to allow it"
    p.close()
