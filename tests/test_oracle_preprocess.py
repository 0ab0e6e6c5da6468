"""Pins the integer side of the oracle (reference: csrc/core/preprocess.cu:11-141,
csrc/core/table_initialize.cu:66-114) against numpy's own sort/unique/searchsorted and brute force."""
import numpy as np
import pytest

from oracle import oracle as orc
from tests.helpers import np_preprocess, brute_preprocess, np_offsets


def make(nrank, length, rng, cache_frac=0.3, width=4):
    root = rng.integers(0, nrank, size=length).astype(np.uint8)
    storage = []
    for r in range(nrank):
        own = np.where(root == r)[0]
        other = np.where(root != r)[0]
        extra = rng.choice(other, size=int(cache_frac * other.shape[0]), replace=False) if nrank > 1 else other[:0]
        st = np.concatenate([own, extra])
        rng.shuffle(st)
        storage.append(st.astype(np.int64))
    o = orc.Oracle(nrank, length, width, 0, 0, root, storage, init=("Uniform", -1.0, 1.0), learning_rate=0.5)
    return o, root, storage


@pytest.mark.parametrize("nrank,length,n", [(1, 1000, 5000), (4, 1024, 1024), (8, 50, 3000), (3, 7, 1), (2, 100000, 20000)])
def test_preprocess_matches_numpy(nrank, length, n):
    rng = np.random.default_rng(nrank * 1000 + n)
    o, root, storage = make(nrank, length, rng)
    for step in range(2):
        keys = [rng.integers(0, length, size=n + r).astype(np.int64) for r in range(nrank)]
        o.preprocess(keys)
        for r in range(nrank):
            exp = np_preprocess(keys[r], root, nrank)
            assert np.array_equal(o.fetch(r, orc.SORTED_ARG), exp["sorted_arg"])
            assert np.array_equal(o.fetch(r, orc.UNIQUE), exp["unique"])
            assert np.array_equal(o.fetch(r, orc.RUN_START), exp["run_start"])
            assert np.array_equal(o.fetch(r, orc.IDX_MAP), exp["idx_map"])
            assert np.array_equal(o.fetch(r, orc.ROOT), exp["root"])
            assert np.array_equal(o.fetch(r, orc.SEND_CNT), exp["send_cnt"])
            _, slot, _ = np_offsets(root, storage[r], r)
            assert np.array_equal(o.fetch(r, orc.OFFSET), slot[exp["unique"]])
            # invariants
            u = o.fetch(r, orc.UNIQUE)
            assert np.array_equal(u[o.fetch(r, orc.IDX_MAP)], keys[r])
            assert sorted(o.fetch(r, orc.SORTED_ARG).tolist()) == list(range(n + r))
            comp = root[u].astype(np.int64) * length + u
            assert np.all(np.diff(comp) > 0)
        for r in range(nrank):
            recv = o.fetch(r, orc.RECV_CNT)
            assert recv.tolist() == [int(o.fetch(s, orc.SEND_CNT)[r]) for s in range(nrank)]


def test_preprocess_brute_force_tiny():
    rng = np.random.default_rng(5)
    for trial in range(30):
        nrank = int(rng.integers(1, 5))
        length = int(rng.integers(1, 12))
        n = int(rng.integers(0, 25))
        o, root, _ = make(nrank, length, rng, cache_frac=0.5)
        keys = [rng.integers(0, length, size=n).astype(np.int64) for _ in range(nrank)]
        o.preprocess(keys)
        for r in range(nrank):
            order, uniq, run_start, idx_map = brute_preprocess(keys[r].tolist(), root)
            assert o.fetch(r, orc.SORTED_ARG).tolist() == order
            assert o.fetch(r, orc.UNIQUE).tolist() == uniq
            assert o.fetch(r, orc.RUN_START).tolist() == run_start
            assert o.fetch(r, orc.IDX_MAP).tolist() == idx_map


def test_offsets_layout_and_versions():
    rng = np.random.default_rng(2)
    o, root, storage = make(4, 300, rng)
    for r in range(4):
        ids, slot, ncached = np_offsets(root, storage[r], r)
        assert np.array_equal(o.fetch(r, orc.STORE_IDS), ids)
        ver = o.fetch(r, orc.VERSION)
        assert np.all(ver[:ncached] == np.iinfo(np.int64).min) and np.all(ver[ncached:] == 0)
        assert o.fetch(r, orc.UPDATES).shape[0] == ncached and not o.fetch(r, orc.UPDATES).any()
        assert not o.fetch(r, orc.PENDING).any()
        # initial values depend on the storage offset only (initializer.cu:72-88)
        assert np.array_equal(o.fetch(r, orc.EMBEDDING), orc.init_values(ids.shape[0] * 4, "Uniform", -1.0, 1.0, 0))


def test_parallel_sort_path_is_identical():
    rng = np.random.default_rng(8)
    o, root, _ = make(4, 200000, rng, cache_frac=0.1)
    keys = [rng.integers(0, 200000, size=150000).astype(np.int64) for _ in range(4)]
    o.preprocess(keys)
    a = [o.fetch(r, orc.SORTED_ARG) for r in range(4)]
    o.set_parallel(True)
    o.preprocess(keys)
    for r in range(4):
        assert np.array_equal(a[r], o.fetch(r, orc.SORTED_ARG))
        assert np.array_equal(o.fetch(r, orc.IDX_MAP), np_preprocess(keys[r], root, 4)["idx_map"])


def test_empty_batch_and_errors():
    rng = np.random.default_rng(3)
    o, root, _ = make(2, 10, rng)
    o.preprocess([np.zeros(0, np.int64), np.zeros(0, np.int64)])
    assert o.fetch(0, orc.UNIQUE).shape[0] == 0 and o.fetch(0, orc.RUN_START).tolist() == [0]
    assert o.fetch(0, orc.SEND_CNT).tolist() == [0, 0]
    with pytest.raises(RuntimeError):
        o.preprocess([np.array([10], np.int64), np.zeros(0, np.int64)])
    with pytest.raises(RuntimeError):  # id 0's owner does not store it
        orc.Oracle(1, 4, 2, 0, 0, np.zeros(4, np.uint8), [np.array([1, 2, 3])])
