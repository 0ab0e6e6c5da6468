"""Cache candidates of the offline partitioner on the GPU (priorities + one radix sort per part) against the oracle's
rule applied to the priorities the host path returns: descending priority, equal priorities by descending id, owned
embeddings left out.  Ids are integers: exact."""
import numpy as np
import pytest

import hetuctr_amd.partition as hp
from oracle import partition_oracle as po

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def slot_data(rng, nd, ns, card, a):
    cols = [np.minimum(rng.zipf(a, size=nd) - 1, card - 1) + f * card for f in range(ns)]
    return np.stack(cols, 1).astype(np.int32)


def check(p, max_len=None):
    pr = p.get_priority()
    owner = p.get_result()[1]
    want = po.cache_lists(pr, owner)
    got, ms = p.cache_lists(max_len)
    for i in range(p.n_part):
        w = want[i] if max_len is None else want[i][:max_len]
        assert got[i].shape == w.shape, "part %d: %d candidates, expected %d" % (i, got[i].shape[0], w.shape[0])
        assert np.array_equal(got[i], w), "part %d" % i
    return ms


@pytest.mark.parametrize("nd,ns,card,a,P,B", [
    (3000, 5, 800, 1.2, 8, 128),
    (500, 3, 17, 1.3, 3, 16),
    (20_000, 26, 3000, 1.3, 8, 1024),
    (5000, 4, 6000, 1.05, 2, 64),       # most embeddings never used by a part: long runs of equal (zero) priority
    (4100, 2, 2049, 1.3, 5, 32),        # a size just past one sort tile
])
def test_cache_lists(nd, ns, card, a, P, B):
    say("cache lists: %d samples x %d slots, %d ids per slot, %d parts" % (nd, ns, card, P))
    rng = np.random.default_rng(nd + P)
    data = slot_data(rng, nd, ns, card, a)
    mat = hp.get_comm_mat(P, max(P // 2, 1))
    p = hp.partition(data, mat, P, B)
    check(p)                                      # on the random initial assignment
    p.refine_data()
    p.refine_embed()
    check(p)
    check(p, max_len=100)                         # truncated lists are prefixes
    check(p, max_len=0)
    p.close()


def test_cache_lists_with_negative_costs():
    """A negative entry of comm_mat gives negative priorities: they rank below the unused embeddings (priority 0).
    Kept above -1, the value the reference's script marks owned embeddings with before it sorts."""
    say("cache lists: negative costs")
    rng = np.random.default_rng(5)
    data = slot_data(rng, 4000, 6, 300, 1.3)
    mat = rng.normal(0, 1e-4, size=(4, 4)).astype(np.float32)
    p = hp.partition(data, mat, 4, 64)
    pr = p.get_priority()
    assert pr.min() < 0 and pr.min() > -1
    check(p)
    p.close()


def test_cache_lists_one_part_owns_everything():
    say("cache lists: single part")
    rng = np.random.default_rng(6)
    data = slot_data(rng, 1000, 3, 50, 1.3)
    p = hp.partition(data, np.zeros((1, 1), np.float32), 1, 16)
    got, _ = p.cache_lists()
    assert len(got) == 1 and got[0].shape[0] == 0
    p.close()


def test_cache_lists_large():
    """2.6 M embeddings x 8 parts."""
    say("cache lists: 300k samples x 26 slots, 100k ids per slot")
    rng = np.random.default_rng(7)
    data = slot_data(rng, 300_000, 26, 100_000, 1.1)
    p = hp.partition(data, hp.get_comm_mat(8, 8), 8, 8192)
    p.refine_data()
    p.refine_embed()
    ms = check(p)
    say("  %d embeddings, kernels %.2f ms" % (p.n_embed, ms))
    p.close()
