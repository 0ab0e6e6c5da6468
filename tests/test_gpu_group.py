"""Several shards on one GPU behind the in-process loopback: the reference's multi-GPU tests
(tests/test_update.py, tests/check.py) with their closed forms, plus step-by-step parity with the oracle
including cache hit / miss / refresh decisions and bounded staleness."""
import threading

import numpy as np
import pytest
import torch

from hetuctr_amd import capi
from tests.gpu_util import Pair, INT_ITEMS_PRE, INT_ITEMS_POST, assert_close
from tests.helpers import zipf_sampler

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def update_pair(nrank, length, width, bounds=(0, 0), init=("Zero", 0.0, 0.0), lr=-1.0, cache="lower", seed=0):
    rs = np.random.RandomState(seed)
    root = rs.randint(nrank, size=length).astype(np.uint8)
    if cache == "lower":      # tests/test_update.py:21
        storage = [np.where(root <= r)[0].astype(np.int64) for r in range(nrank)]
    elif cache == "none":     # tests/check.py:30
        storage = [np.where(root == r)[0].astype(np.int64) for r in range(nrank)]
    else:                     # a random third of the remote rows, shuffled
        storage = []
        for r in range(nrank):
            own, other = np.where(root == r)[0], np.where(root != r)[0]
            st = np.concatenate([own, rs.choice(other, other.shape[0] // 3, replace=False)])
            rs.shuffle(st)
            storage.append(st.astype(np.int64))
    return Pair(nrank, length, width, root, storage, init=init, lr=lr, bounds=bounds, seed=seed), root


@pytest.mark.parametrize("nrank", [2, 4])
def test_occurrence_count_closed_form(nrank):
    say("test_update::test_one nrank", nrank)
    length, width, bs = 1024, 128, 1024
    p, root = update_pair(nrank, length, width)
    rngs = [np.random.RandomState(r) for r in range(nrank)]
    store = np.zeros(length)
    p.preprocess([np.zeros(0, np.int64)] * nrank)
    prev = [np.zeros(0, np.int64)] * nrank
    for step in range(50):
        for r in range(nrank):
            np.add.at(store, prev[r], 1.0)
        keys = [rngs[r].randint(length, size=bs).astype(np.int64) for r in range(nrank)]
        p.preprocess(keys)
        out, ref = p.push_pull([np.ones((prev[r].shape[0], width), np.float32) for r in range(nrank)])
        for r in range(nrank):
            assert np.array_equal(out[r][:, 0], store[keys[r]].astype(np.float32)), (step, r)
            assert np.array_equal(out[r], ref[r])
        prev = keys
    p.compare_ints(INT_ITEMS_PRE + INT_ITEMS_POST)
    p.close()


def test_gradient_sum_closed_form():
    say("test_update::test_two")
    nrank, length, width, bs = 4, 1024, 16, 1024
    p, root = update_pair(nrank, length, width)
    rngs = [np.random.RandomState(100 + r) for r in range(nrank)]
    store = np.zeros((length, width))
    prev = [np.zeros(0, np.int64)] * nrank
    for step in range(50):
        grads = [rngs[r].rand(prev[r].shape[0], width).astype(np.float32) for r in range(nrank)]
        for r in range(nrank):
            np.add.at(store, prev[r], grads[r].astype(np.float64))
        keys = [rngs[r].randint(length, size=bs).astype(np.int64) for r in range(nrank)]
        p.preprocess(keys)
        out, ref = p.push_pull(grads)
        for r in range(nrank):
            assert np.max(np.abs(out[r] - store[keys[r]])) < 1e-4   # tests/test_update.py:70
            assert_close(out[r], ref[r], 1e-5, "step %d rank %d" % (step, r))
        prev = keys
    p.close()


@pytest.mark.parametrize("nrank,bounds,cache,width", [(4, (0, 0), "lower", 8), (4, (10, 10), "none", 128),
                                                      (3, (2, 3), "third", 20), (8, (1, 0), "third", 64),
                                                      (2, (0, 5), "lower", 3)])
def test_stepwise_parity_with_staleness(nrank, bounds, cache, width):
    say("stepwise", nrank, bounds, cache, width)
    length, bs = 3000, 2500
    p, root = update_pair(nrank, length, width, bounds=bounds, init=("Uniform", -1.0, 1.0), lr=0.5, cache=cache, seed=3)
    rng = np.random.default_rng(nrank * 10 + bounds[0])
    draw = zipf_sampler(length, 1.05, rng)
    prev_n = [0] * nrank
    for step in range(12):
        keys = [draw(bs - 7 * r) if step % 3 else rng.integers(0, length, bs - 7 * r).astype(np.int64) for r in range(nrank)]
        if step == 5:
            keys[0] = np.zeros(0, np.int64)       # one shard sits a step out
        p.preprocess(keys)
        p.compare_ints(INT_ITEMS_PRE, "step %d" % step)
        grads = [rng.normal(0, 0.1, size=(prev_n[r], width)).astype(np.float32) for r in range(nrank)]
        if step == 8:
            grads[1] = None                        # inference on one shard
        out, ref = p.push_pull(grads)
        p.compare_ints(INT_ITEMS_POST, "step %d" % step)
        for r in range(nrank):
            assert_close(out[r], ref[r], 1e-5, "dst step %d rank %d" % (step, r))
        p.compare_state(1e-5, "step %d" % step)
        prev_n = [k.shape[0] for k in keys]
    p.close()


@pytest.mark.parametrize("nrank,cache,width", [(3, "third", 20), (5, "lower", 128)])
def test_steps_without_a_look_at_the_index(nrank, cache, width):
    # Nothing is fetched between preprocess and push_pull, so push_pull finds the index of the current batches still
    # running and never waits for it on the host: the queries are placed and counted on the device, and the grids of
    # the query kernels are cut from what the step before had.  Batch sizes jump by orders of magnitude both ways,
    # shards sit steps out, one step has no keys at all.
    say("no look at the index", nrank, cache, width)
    length = 40_000
    p, root = update_pair(nrank, length, width, bounds=(1, 2), init=("Uniform", -1.0, 1.0), lr=0.5, cache=cache, seed=5)
    rng = np.random.default_rng(nrank)
    draw = zipf_sampler(length, 1.05, rng)
    sizes = [300, 120_000, 7, 60_000, 0, 1, 90_000, 2_000]
    prev_n = [0] * nrank
    for step, bs in enumerate(sizes):
        keys = [draw(max(bs - 5 * r, 0)) if step % 2 else rng.integers(0, length, max(bs - 5 * r, 0)).astype(np.int64)
                for r in range(nrank)]
        if step in (1, 6):
            keys[step % nrank] = np.zeros(0, np.int64)     # a shard sits out a large step
        p.preprocess(keys, device_keys=bool(step % 3))
        grads = [rng.normal(0, 0.1, size=(prev_n[r], width)).astype(np.float32) for r in range(nrank)]
        out, ref = p.push_pull(grads)
        p.compare_ints(INT_ITEMS_PRE + INT_ITEMS_POST, "step %d" % step)
        for r in range(nrank):
            assert_close(out[r], ref[r], 1e-5, "dst step %d rank %d" % (step, r))
        p.compare_state(1e-5, "step %d" % step)
        prev_n = [k.shape[0] for k in keys]
    p.close()


@pytest.mark.parametrize("bounds,cached", [((0, 0), (0,)), ((2, 3), tuple(range(8)))])
def test_partitioned_table_with_hot_row_cache(bounds, cached):
    # the 8-way partition of the Criteo-like table at 1/100 scale: uniform owners, the hottest 10 % of the remote
    # rows cached; either rank 0 alone feeds batches while the peers only serve, or every rank does
    from hetuctr_amd import workloads
    say("partitioned", bounds, cached)
    cfg = workloads.CONFIGS["cfg3"]
    ks = workloads.KeyStream(cfg, seed=0, scale=0.01)
    R, width = cfg["nrank"], cfg["width"]
    root, storage = workloads.shard_layout(ks, R, cfg["cache_frac"], cached_ranks=cached)
    p = Pair(R, ks.rows, width, root, storage, init=("Uniform", -0.1, 0.1), lr=cfg["lr"], bounds=bounds, seed=0)
    rng = np.random.default_rng(4)
    prev_n = [0] * R
    totals = np.zeros(6)
    for step in range(5):
        keys = [ks.batch() if r in cached else np.zeros(0, np.int64) for r in range(R)]
        p.preprocess(keys, device_keys=True)
        p.compare_ints(INT_ITEMS_PRE, "step %d" % step)
        out, ref = p.push_pull([rng.normal(0, 1e-2, size=(prev_n[r], width)).astype(np.float32) for r in range(R)])
        p.compare_ints(INT_ITEMS_POST, "step %d" % step)
        for r in cached:
            assert_close(out[r], ref[r], 1e-5, "dst step %d rank %d" % (step, r))
        for r in range(R):
            totals += p.tables[r].fetch(capi.STATS)[:6]
        prev_n = [k.shape[0] for k in keys]
    p.compare_state(1e-5, "end")
    hit, miss, refreshed, pushed, returned, received = totals
    assert hit > 0 and miss > 0 and pushed == received and returned == miss + refreshed
    assert refreshed > 0                            # at least the first fetch of every touched cached row
    p.close()


def test_layout_from_the_offline_partitioner():
    # the whole offline flow at 1/100 scale: click log -> partitioner (owners, cache candidates, samples per rank)
    # -> eight tables that train on their own samples; parity with the oracle, and fewer rows cross ranks than
    # with uniform owners and the hottest rows cached
    from hetuctr_amd import workloads
    say("layout from the partitioner")
    cfg = workloads.CONFIGS["cfg3"]
    R, width = cfg["nrank"], cfg["width"]
    ranks = tuple(range(R))
    ks = workloads.KeyStream(cfg, seed=0, scale=0.01)
    steps = 4
    root, storage, batches, info = workloads.partitioned_layout(ks, R, cfg["cache_frac"], R * ks.samples * (steps + 1),
                                                                ks.samples, rounds=3, cached_ranks=ranks)
    assert info["cost_per_round"][-1] < 0.8 * info["cost_per_round"][0]
    assert min(len(b) for b in batches.values()) >= steps
    for r in ranks:                                   # a rank stores what it owns and nothing twice
        assert np.array_equal(np.sort(storage[r][:int((root == r).sum())]), np.flatnonzero(root == r))
        assert np.unique(storage[r]).shape[0] == storage[r].shape[0]

    def run(root, storage, batches, check):
        p = Pair(R, ks.rows, width, root, storage, init=("Uniform", -0.1, 0.1), lr=cfg["lr"], bounds=(2, 3), seed=0)
        rng = np.random.default_rng(4)
        prev_n = [0] * R
        totals = np.zeros(6)
        for step in range(steps):
            keys = [batches[r][step] for r in range(R)]
            p.preprocess(keys, device_keys=True)
            if check:
                p.compare_ints(INT_ITEMS_PRE, "step %d" % step)
            out, ref = p.push_pull([rng.normal(0, 1e-2, size=(prev_n[r], width)).astype(np.float32) for r in range(R)])
            if check:
                p.compare_ints(INT_ITEMS_POST, "step %d" % step)
                for r in range(R):
                    assert_close(out[r], ref[r], 1e-5, "dst step %d rank %d" % (step, r))
            for r in range(R):
                totals += p.tables[r].fetch(capi.STATS)[:6]
            prev_n = [k.shape[0] for k in keys]
        if check:
            p.compare_state(1e-5, "end")
        p.close()
        return totals

    hit, miss, refreshed, pushed, returned, received = run(root, storage, batches, True)
    assert pushed == received and returned == miss + refreshed
    ks2 = workloads.KeyStream(cfg, seed=0, scale=0.01)
    root2, storage2 = workloads.shard_layout(ks2, R, cfg["cache_frac"], cached_ranks=ranks)
    plain = {r: [ks2.batch() for _ in range(steps)] for r in range(R)}
    _, miss2, refreshed2, pushed2, returned2, _ = run(root2, storage2, plain, False)
    say("  rows returned by owners: %d partitioned, %d uniform owners; pushed %d vs %d" %
        (returned, returned2, pushed, pushed2))
    assert returned < returned2 and pushed < pushed2


def test_hand_computed_staleness_scenario():
    # same scenario as tests/test_oracle_update.py::test_staleness_scenario_both_update, on the GPU
    root = np.array([0, 1], np.uint8)
    p = Pair(2, 2, 4, root, [np.array([0, 1]), np.array([1])], lr=-1.0, bounds=(1, 2))
    one = np.array([1], np.int64)
    r0, r1 = [], []
    n_prev = 0
    for step in range(4):
        p.preprocess([one, one])
        g = np.ones((n_prev, 4), np.float32)
        out, ref = p.push_pull([g, g]); n_prev = 1
        r0.append(float(out[0][0, 0])); r1.append(float(out[1][0, 0]))
    assert r0 == [0.0, 1.0, 4.0, 5.0] and r1 == [0.0, 1.0, 2.0, 6.0]
    assert p.tables[0].fetch(capi.STATS).tolist()[:3] == [1, 0, 0]
    p.close()


def test_per_shard_calls_from_threads():
    # the reference's per-process call pattern (tests/check.py:40-44), one thread per shard
    say("threads")
    nrank, length, width, bs = 4, 1024, 32, 512
    p, root = update_pair(nrank, length, width, bounds=(0, 0))
    rng = np.random.RandomState(5)
    steps = 6
    keys = [[rng.randint(length, size=bs).astype(np.int64) for _ in range(steps)] for _ in range(nrank)]
    outs = [[None] * steps for _ in range(nrank)]
    errors = []

    def worker(r):
        try:
            dst = torch.zeros((bs, width), device="cuda")
            grad = torch.ones((bs, width), device="cuda")
            torch.cuda.synchronize()
            for s in range(steps):
                p.tables[r].preprocess(keys[r][s].ctypes.data, bs)
                p.tables[r].push_pull(grad.data_ptr() if s else 0, dst.data_ptr())
                outs[r][s] = dst.cpu().numpy().copy()
        except Exception as e:  # pragma: no cover
            errors.append(e)

    ts = [threading.Thread(target=worker, args=(r,)) for r in range(nrank)]
    [t.start() for t in ts]
    [t.join(60) for t in ts]
    assert not errors, errors
    store = np.zeros(length)
    for s in range(steps):
        if s > 0:
            for r in range(nrank):
                np.add.at(store, keys[r][s - 1], 1.0)
        for r in range(nrank):
            assert np.array_equal(outs[r][s][:, 0], store[keys[r][s]].astype(np.float32)), (s, r)
    p.close()


def test_group_errors():
    root = np.array([0, 1], np.uint8)
    t0 = capi.Table(0, 2, 0, "10.0.0.1", 999, 2, 4, 0, 0, root, np.array([0]), ("Zero", 0, 0), 0.1)
    k = np.array([0], np.int64)
    with pytest.raises(RuntimeError, match="every rank|missing ranks"):
        capi.group_preprocess([t0], [k.ctypes.data], [1])
    with pytest.raises(RuntimeError, match="already exists"):
        capi.Table(0, 2, 0, "10.0.0.1", 999, 2, 4, 0, 0, root, np.array([0]), ("Zero", 0, 0), 0.1)
    t0.close()


@pytest.mark.parametrize("nrank", [33, 200])
def test_many_shards(nrank):
    """More shards than any benchmark uses (the owner-side kernels walk up to 256 sources per target row, the exchanges
    describe nrank * nrank segment pairs): three steps with caches and staleness against the oracle."""
    rng = np.random.default_rng(nrank)
    length, width = 5000, 12
    root = rng.integers(0, nrank, size=length).astype(np.uint8)
    storage = []
    for r in range(nrank):
        own, other = np.flatnonzero(root == r), np.flatnonzero(root != r)
        storage.append(np.concatenate([own, rng.choice(other, other.shape[0] // 4, replace=False)]).astype(np.int64))
    p = Pair(nrank, length, width, root, storage, init=("Uniform", -0.1, 0.1), lr=0.1, bounds=(1, 2))
    draw = zipf_sampler(length, 1.2, rng)
    prev = [0] * nrank
    for step in range(3):
        sizes = [int(rng.choice([0, 40, 400])) for _ in range(nrank)]
        keys = [draw(k) if k else np.zeros(0, np.int64) for k in sizes]
        p.preprocess(keys)
        p.compare_ints(INT_ITEMS_PRE, "step %d" % step)
        out, ref = p.push_pull([rng.normal(0, 0.1, size=(prev[r], width)).astype(np.float32) for r in range(nrank)])
        p.compare_ints(INT_ITEMS_POST, "step %d" % step)
        for r in range(nrank):
            assert_close(out[r], ref[r], 1e-5, "dst step %d rank %d" % (step, r))
        p.compare_state(1e-5, "step %d" % step)
        prev = sizes
    p.close()
