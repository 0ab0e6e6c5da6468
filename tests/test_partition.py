"""Offline partitioner on the host: the numpy oracle against the reference's own sources compiled without OpenMP
(when that build is present), against the golden cases that build produced, and against what can be known without
it; then the library (C ABI, python mirror hetuctr_amd.partition) against the oracle and the golden cases.  Integer
results are compared exactly, float results bit for bit: both sides perform the same IEEE operations in the same
order."""
import ctypes
import importlib.util
import os

import numpy as np
import pytest

import hetuctr_amd.partition as hp
from oracle import partition_oracle as po

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden", "partition_cases.npz")
REF_DIR = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "partition_serial")


def reference_module():
    """The reference's module built from its sources without OpenMP, or None."""
    if not os.path.isdir(REF_DIR):
        return None
    so = [f for f in os.listdir(REF_DIR) if f.startswith("hetuCTR_partition")]
    if not so:
        return None
    spec = importlib.util.spec_from_file_location("hetuCTR_partition", os.path.join(REF_DIR, so[0]))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def slot_data(rng, nd, ns, card, a):
    """One id per slot from the slot's own range: no embedding occurs n_data times."""
    cols = [np.minimum(rng.zipf(a, size=nd) - 1, card - 1) + f * card for f in range(ns)]
    return np.stack(cols, 1).astype(np.int32)


def same_state(a, b, what):
    da, ea = a.get_result()
    db, eb = b.get_result()
    assert np.array_equal(da, db), what + ": sample assignment"
    assert np.array_equal(ea, eb), what + ": embedding assignment"
    assert np.array_equal(a.get_data_cnt(), b.get_data_cnt()) and np.array_equal(a.get_embed_cnt(), b.get_embed_cnt())
    ca, cb = a.get_communication(), b.get_communication()
    assert ca.dtype == np.float32 and np.array_equal(ca.view(np.uint32), cb.view(np.uint32)), what + ": communication"
    pa, pb = a.get_priority(), b.get_priority()
    assert np.array_equal(pa.view(np.uint32), pb.view(np.uint32)), what + ": priority"


# ---- the generator behind the initial assignment ------------------------------------------------------------

def test_rand_known_answers():
    # the first results of rand() in a fresh glibc process, as printed by any C program that calls it unseeded
    first = [1804289383, 846930886, 1681692777, 1714636915, 1957747793, 424238335, 719885386, 1649760492, 596516649,
             1189641421]
    assert po.glibc_rand(1, 10).tolist() == first
    assert po.glibc_rand(0, 10).tolist() == first                     # srand(0) is srand(1)


def test_rand_against_c_library():
    libc = ctypes.CDLL(None)
    if not hasattr(libc, "gnu_get_libc_version"):
        pytest.skip("not glibc")
    for seed in (1, 2, 12345, 2**31 - 1, 2**31 + 5, 2**32 - 1):
        libc.srand(ctypes.c_uint(seed))
        got = [libc.rand() for _ in range(2000)]
        assert po.glibc_rand(seed, 2000).tolist() == got, seed


def test_library_draws_the_same_initial_assignment():
    rng = np.random.default_rng(1)
    data = slot_data(rng, 700, 4, 50, 1.3)
    mat = np.ones((5, 5), np.float32)
    for seed in (1, 7, 2**31 + 5):
        p = hp.partition(data, mat, 5, 32, seed=seed)
        draws = po.glibc_rand(seed, 700 + p.n_embed)
        d, e = p.get_result()
        assert np.array_equal(d, draws[:700] % 5) and np.array_equal(e, draws[700:] % 5)
        assert np.array_equal(p.get_data_cnt(), np.bincount(d, minlength=5))
        assert np.array_equal(p.get_embed_cnt(), np.bincount(e, minlength=5))


# ---- the soft-count table -----------------------------------------------------------------------------------

def test_soft_table_closed_form():
    for n_data, P, B in ((8000, 8, 128), (3000, 3, 16), (1000, 4, 1)):
        soft = po.soft_table(n_data, P, B)
        m = n_data // P
        i = np.arange(m, dtype=np.float64)
        exact = (1 - (1 - i / m) ** B) * m / B
        assert soft[0] == 0 and np.all(soft[m:] == 1)
        assert np.allclose(soft[:m], exact, rtol=2e-4, atol=1e-6)      # float repeated squaring against double pow
        assert np.all(np.diff(soft[:m].astype(np.float64)) >= -1e-3)   # non-decreasing up to float noise
    # batch 1: (1 - (1 - i/m)) * m = i up to rounding
    assert np.allclose(po.soft_table(1000, 4, 1)[:250], np.arange(250), atol=1e-3)


# ---- oracle against the reference's sources and its golden outputs --------------------------------------------

def test_oracle_against_golden_cases():
    g = np.load(GOLDEN)
    for c in range(int(g["n_cases"])):
        k = "c%d" % c
        P, B, rounds = g[k + "_cfg"].tolist()
        o = po.Partition(g[k + "_data"], g[k + "_mat"], P, B)
        for r in range(rounds + 1):
            if r:
                o.refine_data()
                o.refine_embed()
            s = "%s_r%d_" % (k, r)
            assert np.array_equal(o.get_result()[0], g[s + "res_data"]), s
            assert np.array_equal(o.get_result()[1], g[s + "res_embed"]), s
            assert np.array_equal(o.get_data_cnt(), g[s + "cnt_data"]) and np.array_equal(o.get_embed_cnt(), g[s + "cnt_embed"])
            assert np.array_equal(o.get_communication().view(np.uint32), g[s + "comm"].view(np.uint32)), s
            assert np.array_equal(o.get_priority().view(np.uint32), g[s + "priority"].view(np.uint32)), s


def test_oracle_against_reference_build():
    ref = reference_module()
    if ref is None:
        pytest.skip("oracle/_ref/partition_serial is not built (reference tree absent)")
    libc = ctypes.CDLL(None)
    rng = np.random.default_rng(11)
    for nd, ns, card, a, P, B in ((1200, 7, 60, 1.4, 5, 48), (2500, 3, 2000, 1.1, 8, 100), (64, 2, 9, 1.3, 2, 8)):
        data = slot_data(rng, nd, ns, card, a)
        mat = rng.random((P, P)).astype(np.float32)
        libc.srand(1)
        r = ref.partition(data, mat, P, B)
        o = po.Partition(data, mat, P, B)
        same_state(r, o, "initial")
        for it in range(2):
            r.refine_data(); o.refine_data()
            r.refine_embed(); o.refine_embed()
            same_state(r, o, "round %d" % it)


# ---- the library ----------------------------------------------------------------------------------------------

def test_library_against_golden_cases():
    g = np.load(GOLDEN)
    for c in range(int(g["n_cases"])):
        k = "c%d" % c
        P, B, rounds = g[k + "_cfg"].tolist()
        p = hp.partition(g[k + "_data"], g[k + "_mat"], P, B)
        for r in range(rounds + 1):
            if r:
                p.refine_data()
                p.refine_embed()
            s = "%s_r%d_" % (k, r)
            assert np.array_equal(p.get_result()[0], g[s + "res_data"]), s
            assert np.array_equal(p.get_result()[1], g[s + "res_embed"]), s
            assert np.array_equal(p.get_data_cnt(), g[s + "cnt_data"]) and np.array_equal(p.get_embed_cnt(), g[s + "cnt_embed"])
            assert np.array_equal(p.get_communication().view(np.uint32), g[s + "comm"].view(np.uint32)), s
            assert np.array_equal(p.get_priority().view(np.uint32), g[s + "priority"].view(np.uint32)), s
        p.close()


@pytest.mark.parametrize("nd,ns,card,a,P,B,seed", [
    (1500, 6, 70, 1.3, 4, 64, 1),
    (2000, 26, 30, 1.5, 8, 256, 1),
    (800, 1, 500, 1.2, 3, 16, 9),       # one slot
    (999, 5, 123, 1.05, 7, 50, 3),      # sizes that do not divide by the number of parts
    (600, 4, 40, 1.3, 1, 32, 1),        # one part: nothing can move
    (300, 3, 2000, 1.01, 2, 300, 5),    # nearly every id used once; batch = samples
])
def test_library_against_oracle(nd, ns, card, a, P, B, seed):
    rng = np.random.default_rng(seed)
    data = slot_data(rng, nd, ns, card, a)
    mat = rng.random((P, P)).astype(np.float32)
    np.fill_diagonal(mat, 0)
    p = hp.partition(data, mat, P, B, seed=seed)
    o = po.Partition(data, mat, P, B, seed=seed)
    same_state(p, o, "initial")
    for it in range(3):
        p.refine_data(); o.refine_data()
        same_state(p, o, "round %d after the sample sweep" % it)
        p.refine_embed(); o.refine_embed()
        same_state(p, o, "round %d after the embedding sweep" % it)
    p.close()


def test_library_with_counts_beyond_the_table():
    """An id in every slot of every sample occurs n_slot * n_data times: beyond the end of the soft-count table, where
    the reference reads outside its array.  Library and oracle read 1 there and must agree."""
    rng = np.random.default_rng(4)
    data = slot_data(rng, 400, 3, 30, 1.3)
    data[:, 1] = 7
    data[:, 2] = 7
    mat = np.ones((4, 4), np.float32) - np.eye(4, dtype=np.float32)
    p, o = hp.partition(data, mat, 4, 16), po.Partition(data, mat, 4, 16)
    for it in range(2):
        p.refine_data(); o.refine_data()
        p.refine_embed(); o.refine_embed()
        same_state(p, o, "round %d" % it)


def test_library_against_reference_build_larger():
    ref = reference_module()
    if ref is None:
        pytest.skip("oracle/_ref/partition_serial is not built (reference tree absent)")
    libc = ctypes.CDLL(None)
    rng = np.random.default_rng(21)
    data = slot_data(rng, 120_000, 26, 9000, 1.2)
    mat = hp.get_comm_mat(8, 4)
    libc.srand(1)
    r = ref.partition(data, mat, 8, 4096)
    p = hp.partition(data, mat, 8, 4096)
    same_state(r, p, "initial")
    for it in range(3):
        r.refine_data(); p.refine_data()
        r.refine_embed(); p.refine_embed()
        same_state(r, p, "round %d" % it)
    cost = (p.get_communication() * mat).sum()
    p.close()
    assert np.isfinite(cost)


def test_refinement_lowers_the_cost_and_keeps_the_books():
    rng = np.random.default_rng(8)
    data = slot_data(rng, 20_000, 10, 3000, 1.2)
    mat = hp.get_comm_mat(4, 2)
    p = hp.partition(data, mat, 4, 512)
    before = float((p.get_communication() * mat).sum())
    for _ in range(3):
        p.refine_data()
        p.refine_embed()
    after = float((p.get_communication() * mat).sum())
    assert after < 0.8 * before
    d, e = p.get_result()
    assert np.array_equal(p.get_data_cnt(), np.bincount(d, minlength=4)) and p.get_data_cnt().sum() == 20_000
    assert np.array_equal(p.get_embed_cnt(), np.bincount(e, minlength=4)) and p.get_embed_cnt().sum() == p.n_embed
    pr = p.get_priority()
    used = np.zeros((4, p.n_embed), bool)
    used[np.repeat(d, 10), data.reshape(-1)] = True
    assert np.array_equal(pr != 0, used & (mat[:, e] != 0))           # nonzero exactly where the part uses a costly row
    p.close()


def test_argument_errors():
    data = np.zeros((10, 3), np.int32)
    mat = np.ones((2, 2), np.float32)
    with pytest.raises(RuntimeError, match="not continuous"):
        hp.partition(np.zeros((10, 6), np.int32)[:, ::2], mat, 2, 4)     # the reference's own check, partition.cc:200
    with pytest.raises(RuntimeError):
        hp.partition(data, np.ones((3, 3), np.float32), 2, 4)            # comm_mat is not n_part x n_part
    with pytest.raises(RuntimeError, match="fewer embeddings"):
        hp.partition(data, mat, 2, 4)                                    # one embedding, two parts
    with pytest.raises(RuntimeError, match="negative"):
        hp.partition(np.full((10, 3), -1, np.int32), mat, 2, 4)
    with pytest.raises(RuntimeError, match="finite"):
        hp.partition(np.arange(30, dtype=np.int32).reshape(10, 3), np.full((2, 2), np.nan, np.float32), 2, 4)


def test_comm_mat_of_the_driver_script():
    m = hp.get_comm_mat(4, 2)
    assert np.array_equal(m, np.array([[0, .1, 1, 1], [.1, 0, 1, 1], [1, 1, 0, .1], [1, 1, .1, 0]], np.float32))


def test_cache_list_rule_of_the_oracle():
    """Without equal priorities the order is the script's (experimental/partition.py:53-57) under any sort."""
    rng = np.random.default_rng(0)
    pr = rng.permutation(4 * 50).reshape(4, 50).astype(np.float32) + 1
    owner = rng.integers(0, 4, 50)
    lists = po.cache_lists(pr, owner)
    for i in range(4):
        q = pr[i].copy()
        idx = np.where(owner == i)[0]
        q[idx] = -1
        assert np.array_equal(lists[i], np.argsort(q)[len(idx):][::-1])


def test_importable_under_the_reference_module_name():
    import hetuctr_amd
    mod = hetuctr_amd.install_as_hetuCTR_partition()
    import hetuCTR_partition
    assert hetuCTR_partition is mod
    rng = np.random.default_rng(2)
    p = hetuCTR_partition.partition(slot_data(rng, 200, 3, 20, 1.3), np.ones((2, 2), np.float32), 2, 8)
    for name in ("refine_data", "refine_embed", "get_communication", "get_priority", "get_result", "get_data_cnt",
                 "get_embed_cnt"):                      # csrc/partition/pybind.cc:9-21
        assert callable(getattr(p, name))
    assert type(p).__name__ == "_PartitionStruct"
