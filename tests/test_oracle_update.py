"""Pins the floating-point / protocol side of the oracle with the closed forms the reference's own
tests use (tests/test_update.py:17-70, tests/check.py:14-46, tests/driver.py:31-33) and with
hand-computed bounded-staleness scenarios (rules: csrc/core/preprocess.cu:151-161,
csrc/core/generate_query.cu:18-48,51-83, csrc/core/handle_query.cu:17-20, csrc/core/writeback.cu:16-20)."""
import numpy as np
import pytest

from oracle import oracle as orc

INVALID = np.iinfo(np.int64).min


def update_setup(nrank, length, width, seed=0, lr=-1.0, bounds=(0, 0), init=("Zero", 0.0, 0.0)):
    # tests/test_update.py:15,21: random owner per id; rank r stores every id owned by a rank <= r
    rs = np.random.RandomState(seed)
    root = rs.randint(nrank, size=length).astype(np.uint8)
    storage = [np.where(root <= r)[0].astype(np.int64) for r in range(nrank)]
    o = orc.Oracle(nrank, length, width, bounds[0], bounds[1], root, storage, init=init, learning_rate=lr)
    return o, root, storage


@pytest.mark.parametrize("nrank", [1, 4])
def test_occurrence_count_closed_form(nrank):
    # tests/test_update.py::test_one: zero init, lr=-1, grad==1 => dst[:,0] == number of earlier occurrences
    length, width, bs = 1024, 8, 1024
    o, root, _ = update_setup(nrank, length, width)
    rngs = [np.random.RandomState(r) for r in range(nrank)]
    store = np.zeros(length)
    o.preprocess([np.zeros(0, np.int64)] * nrank)           # test_update.py:28-29
    prev = [np.zeros(0, np.int64)] * nrank
    for step in range(50):
        for r in range(nrank):
            np.add.at(store, prev[r], 1.0)
        keys = [rngs[r].randint(length, size=bs).astype(np.int64) for r in range(nrank)]
        o.preprocess(keys)
        grads = [np.ones((prev[r].shape[0], width), np.float32) for r in range(nrank)]
        dst = o.push_pull(grads)
        for r in range(nrank):
            assert np.array_equal(dst[r][:, 0], store[keys[r]].astype(np.float32)), (step, r)
            assert np.all(dst[r] == dst[r][:, :1])
        prev = keys


@pytest.mark.parametrize("nrank", [1, 4])
def test_gradient_sum_closed_form(nrank):
    # tests/test_update.py::test_two: random grads, |dst - sum of grads| < 1e-4
    length, width, bs = 1024, 4, 1024
    o, root, _ = update_setup(nrank, length, width)
    rngs = [np.random.RandomState(100 + r) for r in range(nrank)]
    store = np.zeros((length, width))
    prev = [np.zeros(0, np.int64)] * nrank
    for step in range(50):
        grads = [rngs[r].rand(prev[r].shape[0], width).astype(np.float32) for r in range(nrank)]
        for r in range(nrank):
            np.add.at(store, prev[r], grads[r].astype(np.float64))
        keys = [rngs[r].randint(length, size=bs).astype(np.int64) for r in range(nrank)]
        o.preprocess(keys)
        dst = o.push_pull(grads)
        for r in range(nrank):
            assert np.max(np.abs(dst[r] - store[keys[r]])) < 1e-4
        prev = keys


def test_sgd_sign_scale_and_sum_order():
    # generate_query.cu:35-41: row += (-lr) * (((0+g0)+g1)+...) in ascending position
    o = orc.Oracle(1, 3, 2, 0, 0, np.zeros(3, np.uint8), [np.arange(3)], init=("Uniform", 1.0, 2.0), learning_rate=0.25)
    e0 = o.fetch(0, orc.EMBEDDING).reshape(3, 2).copy()
    keys = np.array([2, 0, 2, 2], np.int64)
    o.preprocess([keys]); o.push_pull([None])
    g = np.array([[1e8, 1.0], [3.0, 4.0], [1.0, 2.0], [-1e8, 0.5]], np.float32)
    o.preprocess([np.array([0, 1, 2], np.int64)])
    dst = o.push_pull([g])[0]
    s2 = (np.float32(0) + g[0]) + g[2]
    s2 = (s2 + g[3]) * np.float32(-0.25)
    s0 = (np.float32(0) + g[1]) * np.float32(-0.25)
    assert np.array_equal(dst[0], e0[0] + s0)
    assert np.array_equal(dst[1], e0[1])
    assert np.array_equal(dst[2], e0[2] + s2)
    assert s2[0] == 0.0  # 1e8 + 1 - 1e8 == 0 in fp32 only in this order
    assert o.fetch(0, orc.VERSION).tolist() == [1, 0, 3]


def test_checkvalue_invariant_with_bounds():
    # tests/check.py: normal init, bounds 10/10, no caches; equal keys => equal rows, every step.
    # The script's second clause (distinct keys => distinct rows) can only hold among keys of ONE owner:
    # every rank draws the same value for the same storage offset (table_initialize.cu:156 passes the
    # same seed and initializer.cu:72-88 indexes by element number), so rows of different owners collide.
    nrank, length, width, bs = 4, 1024, 8, 1024
    rs = np.random.RandomState(0)
    root = rs.randint(nrank, size=length).astype(np.uint8)
    storage = [np.where(root == r)[0].astype(np.int64) for r in range(nrank)]
    o = orc.Oracle(nrank, length, width, 10, 10, root, storage, init=("Normal", 0.0, 1.0), learning_rate=1.0)
    o.preprocess([np.zeros(0, np.int64)] * nrank)      # check.py:40
    grad = [rs.rand(bs, width).astype(np.float32) for _ in range(nrank)]
    prevn = [0] * nrank
    for step in range(5):
        keys = [rs.randint(length, size=bs).astype(np.int64) for _ in range(nrank)]
        o.preprocess(keys)
        dst = o.push_pull([grad[r][:prevn[r]] for r in range(nrank)])
        for r in range(nrank):
            v = dst[r][:, 0]
            first = {}
            for k, x in zip(keys[r].tolist(), v.tolist()):
                assert first.setdefault(k, x) == x
            for own in range(nrank):
                vals = [x for k, x in first.items() if root[k] == own]
                assert len(set(vals)) == len(vals)
        prevn = [bs] * nrank


def test_double_preprocess_and_inference():
    # tests/driver.py:31-33: two preprocess calls, then push_pull applies grads to the FIRST batch
    o = orc.Oracle(1, 4, 1, 0, 0, np.zeros(4, np.uint8), [np.arange(4)], learning_rate=-1.0)
    o.preprocess([np.array([1, 1, 3], np.int64)])
    o.preprocess([np.array([0, 1, 2, 3], np.int64)])
    dst = o.push_pull([np.array([[1.0], [2.0], [4.0]], np.float32)])[0]
    assert dst[:, 0].tolist() == [0.0, 3.0, 0.0, 4.0]
    # inference (grad pointer 0): nothing is applied, rows are still pulled (hetu_gpu_table.cu:14-21)
    o.preprocess([np.array([1], np.int64)])
    assert o.push_pull([None])[0][:, 0].tolist() == [3.0]
    o.preprocess([np.array([1], np.int64)])
    assert o.push_pull([np.array([[5.0]], np.float32)])[0][:, 0].tolist() == [8.0]


def _two_rank(bounds, r0_caches):
    root = np.array([0, 1], np.uint8)
    storage = [np.array([0, 1] if r0_caches else [0], np.int64), np.array([1], np.int64)]
    return orc.Oracle(2, 2, 1, bounds[0], bounds[1], root, storage, learning_rate=-1.0)


def test_staleness_scenario_owner_idle():
    # rank 0 hits cached id 1 every step with grad 1; owner (rank 1) idle; push_bound 2, pull_bound 0
    o = _two_rank((0, 2), True)
    one = np.array([1], np.int64); none = np.zeros(0, np.int64)
    out, owner_emb, owner_ver, upd = [], [], [], []
    n_prev = 0
    for step in range(5):
        o.preprocess([one, none])
        d = o.push_pull([np.ones((n_prev, 1), np.float32), np.zeros((0, 1), np.float32)])
        out.append(float(d[0][0, 0])); n_prev = 1
        owner_emb.append(float(o.fetch(1, orc.EMBEDDING)[0])); owner_ver.append(int(o.fetch(1, orc.VERSION)[0]))
        upd.append(int(o.fetch(0, orc.UPDATES)[0]))
    assert out == [0.0, 1.0, 2.0, 3.0, 4.0]
    assert owner_emb == [0.0, 0.0, 0.0, 3.0, 3.0]       # pushed only when 3 updates are pending (> bound 2)
    assert owner_ver == [0, 0, 0, 3, 3]
    assert upd == [0, 1, 2, 0, 1]
    assert o.fetch(0, orc.VERSION).tolist()[0] == 3    # cached row's version = refreshed 0 + pushed 3
    assert o.fetch(0, orc.STATS).tolist()[:3] == [1, 0, 0]  # last step: a hit


def test_staleness_scenario_both_update():
    # both ranks add 1 to id 1 per step; push_bound 2, pull_bound 1 (hand-computed in the module docstring's rules)
    o = _two_rank((1, 2), True)
    one = np.array([1], np.int64)
    r0, r1, stats = [], [], []
    n_prev = 0
    for step in range(4):
        o.preprocess([one, one])
        g = np.ones((n_prev, 1), np.float32)
        d = o.push_pull([g, g]); n_prev = 1
        r0.append(float(d[0][0, 0])); r1.append(float(d[1][0, 0]))
        stats.append(o.fetch(0, orc.STATS).tolist()[:3])
    assert r0 == [0.0, 1.0, 4.0, 5.0]
    assert r1 == [0.0, 1.0, 2.0, 6.0]
    assert stats == [[0, 0, 1], [1, 0, 0], [0, 0, 1], [1, 0, 0]]   # refresh, hit, refresh, hit
    assert int(o.fetch(1, orc.VERSION)[0]) == 6 and int(o.fetch(0, orc.VERSION)[0]) == 5


def test_not_stored_rows_always_push_and_pull():
    # rank 0 does not cache id 1: every step pushes (type 0) and the row comes from the return buffer
    o = _two_rank((5, 5), False)
    keys0 = np.array([1, 0, 1], np.int64)
    out = []
    n_prev = 0
    for step in range(3):
        o.preprocess([keys0, np.zeros(0, np.int64)])
        g = np.array([[1.0], [10.0], [2.0]], np.float32)[:n_prev]
        d = o.push_pull([g, np.zeros((0, 1), np.float32)]); n_prev = 3
        out.append(d[0][:, 0].tolist())
        assert o.fetch(0, orc.STATS).tolist()[:3] == [0, 1, 0]
    assert out == [[0.0, 0.0, 0.0], [3.0, 10.0, 3.0], [6.0, 20.0, 6.0]]
    assert o.fetch(0, orc.NEED_UPDATE).tolist() == [0, 1] and o.fetch(0, orc.PUSH_CNT).tolist() == [0, 1]
    assert int(o.fetch(1, orc.VERSION)[0]) == 4


# ---- sum-pooled bags (oracle.Oracle.push_pull_pooled): pinned by what the definition fixes -----------------------
@pytest.mark.parametrize("nrank", [1, 4])
def test_pooled_occurrence_count_closed_form(nrank):
    # zero init, lr = -1, every bag's gradient == 1: a key's row counts its earlier occurrences (a key that sits
    # twice in a bag is pushed twice), and a bag pulls the sum of its keys' counts; all integers, exact in fp32
    length, width, bag, bags = 512, 6, 5, 200
    o, root, _ = update_setup(nrank, length, width)
    rngs = [np.random.RandomState(7 + r) for r in range(nrank)]
    store = np.zeros(length)
    prev = [np.zeros(0, np.int64)] * nrank
    for step in range(20):
        for r in range(nrank):
            np.add.at(store, prev[r], 1.0)
        keys = [rngs[r].randint(length, size=bags * bag).astype(np.int64) for r in range(nrank)]
        o.preprocess(keys)
        gp = [np.ones((prev[r].shape[0] // bag, width), np.float32) for r in range(nrank)]
        dst = o.push_pull_pooled(gp, bag)
        for r in range(nrank):
            want = store[keys[r]].reshape(bags, bag).sum(axis=1)
            assert dst[r].shape == (bags, width)
            assert np.array_equal(dst[r][:, 0], want.astype(np.float32)), (step, r)
            assert np.all(dst[r] == dst[r][:, :1])
        prev = keys


def test_pooled_bag_of_one_is_the_plain_step_and_the_sum_runs_in_key_order():
    length, width = 64, 3
    root = np.zeros(length, np.uint8)
    st = [np.arange(length, dtype=np.int64)]
    a = orc.Oracle(1, length, width, 0, 0, root, st, init=("Uniform", -1.0, 1.0), learning_rate=0.5)
    b = orc.Oracle(1, length, width, 0, 0, root, st, init=("Uniform", -1.0, 1.0), learning_rate=0.5)
    rs = np.random.RandomState(1)
    prev_n = 0
    for step in range(4):
        keys = rs.randint(length, size=40).astype(np.int64)
        g = rs.rand(prev_n, width).astype(np.float32)
        a.preprocess([keys]); b.preprocess([keys])
        assert np.array_equal(a.push_pull([g])[0], b.push_pull_pooled([g], 1)[0])
        prev_n = 40
    # order of the additions, with rows 0, 1, 2 holding 1e8, 1, -1e8 (1e8 + 1 == 1e8 in fp32):
    # keys (1, 0, 2): (1 + 1e8) - 1e8 = 0 from left to right, 1 from right to left or pairwise;
    # keys (2, 0, 1): (-1e8 + 1e8) + 1 = 1 from left to right, 0 from right to left
    c = orc.Oracle(1, 3, 1, 0, 0, np.zeros(3, np.uint8), [np.arange(3, dtype=np.int64)], init=("Zero", 0, 0),
                   learning_rate=-1.0)
    c.preprocess([np.array([0, 1, 2], np.int64)])
    c.push_pull([None])
    c.preprocess([np.array([1, 0, 2, 2, 0, 1], np.int64)])
    c.push_pull_pooled([np.array([[1e8], [1.0], [-1e8]], np.float32)], 1)   # lr = -1: the rows become 1e8, 1, -1e8
    c.preprocess([np.array([1, 0, 2, 2, 0, 1], np.int64)])
    pooled = c.push_pull_pooled([None], 3)[0]
    assert pooled[:, 0].tolist() == [0.0, 1.0]
    for x in (a, b, c):
        x.close()
