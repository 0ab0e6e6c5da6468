"""Seeded random configurations of the table (shards, width, bounds, cache layout, initialiser, batch sizes, key
skew, inference steps, empty batches), every step compared with the oracle: integer intermediates exactly, rows and
outputs bit for bit (and within 1e-5 relative, the stated bound)."""
import numpy as np
import pytest

from hetuctr_amd import capi
from tests.gpu_util import Pair, INT_ITEMS_PRE, INT_ITEMS_POST, assert_close
from tests.helpers import zipf_sampler

pytestmark = pytest.mark.gpu


def make_case(seed):
    rs = np.random.default_rng(1000 + seed)
    nrank = int(rs.choice([1, 1, 2, 3, 5, 8]))
    width = int(rs.choice([1, 2, 7, 8, 32, 64, 100, 128, 192]))
    length = int(rs.choice([300, 4000, 60000]))
    bounds = (int(rs.integers(0, 4)), int(rs.integers(0, 4)))
    root = rs.integers(0, nrank, size=length).astype(np.uint8)
    storage = []
    for r in range(nrank):
        own, other = np.flatnonzero(root == r), np.flatnonzero(root != r)
        frac = float(rs.choice([0.0, 0.1, 0.5, 1.0]))
        extra = rs.choice(other, int(frac * other.shape[0]), replace=False) if other.shape[0] else other
        st = np.concatenate([own, extra])
        rs.shuffle(st)
        storage.append(st.astype(np.int64))
    init = [("Zero", 0.0, 0.0), ("Uniform", -0.01, 0.01), ("Uniform", -0.5, 0.5)][int(rs.integers(0, 3))]
    lr = float(rs.choice([0.05, 0.5, -1.0]))
    return rs, nrank, width, length, bounds, root, storage, init, lr


@pytest.mark.parametrize("seed", list(range(40)))
def test_random_configuration(seed):
    rs, nrank, width, length, bounds, root, storage, init, lr = make_case(seed)
    print("case", seed, "nrank", nrank, "width", width, "length", length, "bounds", bounds, "init", init[0], flush=True)
    p = Pair(nrank, length, width, root, storage, init=init, lr=lr, bounds=bounds, seed=seed)
    alpha = float(rs.choice([0.0, 1.05, 1.6]))
    draw = zipf_sampler(length, alpha, rs) if alpha else (lambda k: rs.integers(0, length, k).astype(np.int64))
    prev_n = [0] * nrank
    for step in range(5):
        sizes = [int(rs.choice([0, 1, 63, 700, 9000])) for _ in range(nrank)]
        keys = [draw(k) if k else np.zeros(0, np.int64) for k in sizes]
        p.preprocess(keys, device_keys=bool(rs.integers(0, 2)))
        p.compare_ints(INT_ITEMS_PRE, "case %d step %d" % (seed, step))
        grads = [rs.normal(0, 0.05, size=(prev_n[r], width)).astype(np.float32) for r in range(nrank)]
        if rs.integers(0, 5) == 0:
            grads[int(rs.integers(0, nrank))] = None   # an inference step on one shard
        out, ref = p.push_pull(grads)
        p.compare_ints(INT_ITEMS_POST, "case %d step %d" % (seed, step))
        for r in range(nrank):
            assert_close(out[r], ref[r], 1e-5, "dst case %d step %d rank %d" % (seed, step, r))
        p.compare_state(1e-5, "case %d step %d" % (seed, step))
        prev_n = sizes
    p.close()


@pytest.mark.parametrize("seed", list(range(16)))
def test_random_call_sequences(seed):
    """The two calls in any order a caller may use them: preprocess twice in a row (the skipped batch is pushed later or
    never), push_pull again without a preprocess in between (the same previous batch is pushed once more by the same
    plan), inference steps in between -- every call mirrored in the oracle, everything compared after every call."""
    rs, nrank, width, length, bounds, root, storage, init, lr = make_case(100 + seed)
    print("sequence case", seed, "nrank", nrank, "width", width, "length", length, "bounds", bounds, flush=True)
    p = Pair(nrank, length, width, root, storage, init=init, lr=lr, bounds=bounds, seed=seed)
    draw = zipf_sampler(length, 1.3, rs)
    cur_n, prev_n = [0] * nrank, [0] * nrank
    p.preprocess([np.zeros(0, np.int64)] * nrank)           # Pair.push_pull sizes its outputs from the last preprocess
    for step in range(10):
        op = int(rs.choice([0, 0, 1, 1, 1, 2]))            # 0: preprocess, 1: push_pull with gradients, 2: inference pull
        where = "case %d call %d op %d" % (seed, step, op)
        if op == 0:
            sizes = [int(rs.choice([0, 5, 300, 2500, 20000])) for _ in range(nrank)]
            keys = [draw(k) if k else np.zeros(0, np.int64) for k in sizes]
            p.preprocess(keys, device_keys=bool(rs.integers(0, 2)))
            p.compare_ints(INT_ITEMS_PRE, where)
            prev_n, cur_n = cur_n, sizes
        else:
            grads = [None if op == 2 else rs.normal(0, 0.05, size=(prev_n[r], width)).astype(np.float32)
                     for r in range(nrank)]
            out, ref = p.push_pull(grads)
            p.compare_ints(INT_ITEMS_POST, where)
            for r in range(nrank):
                assert_close(out[r], ref[r], 1e-5, "dst %s rank %d" % (where, r))
            p.compare_state(1e-5, where)
            if op == 2:
                prev_n = [0] * nrank                         # an inference step drops the previous batch (hetu_gpu_table.cu:14-21)
    p.close()
