"""hctr_push_pull_pooled (sum-pooled multi-hot bags) through the C ABI against the CPU oracle: pooled rows and table
state bit for bit, single shard and loopback groups; the 10-hot benchmark configuration at full size through exact
integer arithmetic."""
import numpy as np
import pytest
import torch

from hetuctr_amd import capi, workloads
from tests.gpu_util import Pair, assert_close
from tests.helpers import zipf_sampler

pytestmark = pytest.mark.gpu


def pooled_step(p, keys, grads_pooled, bag):
    """One step on both sides; returns (gpu pooled rows, oracle pooled rows) per rank."""
    p.preprocess(keys, device_keys=True)
    dg = [None if g is None else torch.from_numpy(np.ascontiguousarray(g, dtype=np.float32)).cuda() for g in grads_pooled]
    dd = [torch.full((max(k.shape[0] // bag, 1), p.W), float("nan"), device="cuda") for k in keys]
    torch.cuda.synchronize()
    capi.group_push_pull_pooled(p.tables, [0 if g is None else (g.data_ptr() if g.numel() else 0) for g in dg],
                                [d.data_ptr() for d in dd], bag)
    out = [d.cpu().numpy()[: k.shape[0] // bag] for d, k in zip(dd, keys)]
    return out, p.oracle.push_pull_pooled(grads_pooled, bag)


@pytest.mark.parametrize("gather", ["from the keys", "through the inverse index"])
@pytest.mark.parametrize("bag,width", [(1, 32), (2, 128), (3, 20), (10, 64), (17, 8)])
def test_single_shard_pooled(bag, width, gather, monkeypatch):
    if gather != "from the keys":          # one shard pools straight from the batch's keys unless told otherwise
        monkeypatch.setenv("HETUCTR_POOLED_FROM_KEYS", "0")
        monkeypatch.setenv("HETUCTR_DIRECT_GATHER_MAX", "0")
    print("pooled single shard, bag", bag, "width", width, flush=True)
    rng = np.random.default_rng(60 + bag)
    length, bags = 20_000, 3000
    root = np.zeros(length, np.uint8)
    p = Pair(1, length, width, root, [np.arange(length, dtype=np.int64)], init=("Uniform", -0.01, 0.01), lr=0.05)
    draw = zipf_sampler(length, 1.2, rng)
    prev_bags = 0
    for step in range(4):
        nb = bags - 7 * step
        keys = draw(nb * bag)
        keys[: 4 * bag] = 5                                  # whole bags of one key: it is pushed `bag` times per bag
        gp = rng.normal(0, 1e-3, size=(prev_bags, width)).astype(np.float32)
        out, ref = pooled_step(p, [keys], [gp], bag)
        assert_close(out[0], ref[0], 1e-5, "pooled rows step %d" % step)
        p.compare_state(1e-5, "step %d" % step)
        p.compare_ints([capi.VERSION, capi.IDX_MAP], "step %d" % step)
        prev_bags = nb
    p.close()


def test_pooled_matches_the_plain_call_with_replicated_gradients():
    # the definition itself, on the GPU alone: same table state as hctr_push_pull with every bag's gradient repeated,
    # pooled rows = the plain rows added up in key order
    rng = np.random.default_rng(70)
    length, width, bag, bags = 5000, 48, 4, 2000
    root = np.zeros(length, np.uint8)
    st = np.arange(length, dtype=np.int64)
    capi.seed(2)
    a = capi.Table(0, 1, 0, "", 0, length, width, 0, 0, root, st, ("Normal", 0.0, 0.1), 0.1)
    b = capi.Table(0, 1, 0, "", 0, length, width, 0, 0, root, st, ("Normal", 0.0, 0.1), 0.1)
    plain = torch.empty((bags * bag, width), device="cuda")
    pooled = torch.empty((bags, width), device="cuda")
    gp = None
    for step in range(3):
        keys = torch.from_numpy(rng.integers(0, length, size=bags * bag).astype(np.int64)).cuda()
        torch.cuda.synchronize()
        a.preprocess(keys.data_ptr(), bags * bag)
        b.preprocess(keys.data_ptr(), bags * bag)
        if gp is None:
            a.push_pull(0, plain.data_ptr())
            b.push_pull_pooled(0, pooled.data_ptr(), bag)
        else:
            rep = gp.repeat_interleave(bag, dim=0).contiguous()
            torch.cuda.synchronize()
            a.push_pull(rep.data_ptr(), plain.data_ptr())
            b.push_pull_pooled(gp.data_ptr(), pooled.data_ptr(), bag)
        v = plain.cpu().numpy().reshape(bags, bag, width)
        acc = v[:, 0, :].copy()
        for h in range(1, bag):
            acc = acc + v[:, h, :]
        assert np.array_equal(pooled.cpu().numpy(), acc), "step %d" % step
        assert np.array_equal(a.fetch(capi.EMBEDDING), b.fetch(capi.EMBEDDING))
        gp = torch.from_numpy(rng.normal(0, 1e-2, size=(bags, width)).astype(np.float32)).cuda()
    with pytest.raises(RuntimeError, match="whole number of bags"):
        b.push_pull_pooled(0, pooled.data_ptr(), 7)
    a.close()
    b.close()


@pytest.mark.parametrize("nrank", [1, 2])
def test_refused_bag_size_leaves_the_table_as_it_was(nrank):
    # A pooled call whose bag does not divide the batch is refused before anything is launched, with the index of the
    # current batch still pending from a preprocess that returned early: the same step repeated with a good bag must
    # then give what a table that never saw the bad call gives, gradient of the previous batch included.
    print("refused bag, shards", nrank, flush=True)
    rng = np.random.default_rng(90 + nrank)
    length, width, bag, bags = 9000, 16, 4, 1200
    root = rng.integers(0, nrank, size=length).astype(np.uint8)
    storage = []
    for r in range(nrank):
        own, other = np.where(root == r)[0], np.where(root != r)[0]
        storage.append(np.concatenate([other[::3], own]).astype(np.int64))
    mk = lambda: Pair(nrank, length, width, root, storage, init=("Uniform", -0.01, 0.01), lr=0.05, with_oracle=False)
    a, b = mk(), mk()
    draw = zipf_sampler(length, 1.15, rng)
    prev = 0
    for step in range(4):
        keys = [draw(bags * bag) for _ in range(nrank)]
        gp = [torch.from_numpy(rng.normal(0, 1e-3, size=(max(prev, 1), width)).astype(np.float32)).cuda() for _ in range(nrank)]
        outs = []
        for p in (a, b):
            p.preprocess(keys, device_keys=True)
            dd = [torch.full((bags, width), float("nan"), device="cuda") for _ in range(nrank)]
            gptr = [g.data_ptr() if prev else 0 for g in gp]
            torch.cuda.synchronize()
            if p is b and step in (1, 2):
                with pytest.raises(RuntimeError, match="whole number of bags"):   # 7 divides neither batch
                    capi.group_push_pull_pooled(p.tables, gptr, [d.data_ptr() for d in dd], 7)
                if step == 1:                                                     # the batches are still there (the
                    for r in range(nrank):                                        # fetch waits for the pending index;
                        assert p.tables[r].fetch(capi.SIZES)[1] > 0               # at step 2 the good call finds it pending)
            capi.group_push_pull_pooled(p.tables, gptr, [d.data_ptr() for d in dd], bag)
            outs.append([d.cpu().numpy() for d in dd])
        for r in range(nrank):
            assert np.array_equal(outs[0][r], outs[1][r]), "rank %d step %d" % (r, step)
            for it in (capi.EMBEDDING, capi.VERSION, capi.PENDING, capi.UPDATES, capi.SIZES):
                assert np.array_equal(a.tables[r].fetch(it), b.tables[r].fetch(it)), (r, step, it)
        prev = bags
    a.close()
    b.close()


@pytest.mark.parametrize("nrank,bounds", [(2, (0, 0)), (3, (3, 3))])
def test_group_pooled(nrank, bounds):
    print("pooled group, shards", nrank, "bounds", bounds, flush=True)
    rng = np.random.default_rng(80 + nrank)
    length, width, bag, bags = 12_000, 32, 5, 1500
    root = rng.integers(0, nrank, size=length).astype(np.uint8)
    storage = []
    for r in range(nrank):
        own, other = np.where(root == r)[0], np.where(root != r)[0]
        storage.append(np.concatenate([other[::3], own]).astype(np.int64))
    p = Pair(nrank, length, width, root, storage, init=("Uniform", -0.01, 0.01), lr=0.05, bounds=bounds)
    draw = zipf_sampler(length, 1.1, rng)
    prev = 0
    for step in range(5):
        keys = [draw(bags * bag) for _ in range(nrank)]
        gp = [rng.normal(0, 1e-3, size=(prev, width)).astype(np.float32) for _ in range(nrank)]
        out, ref = pooled_step(p, keys, gp, bag)
        for r in range(nrank):
            assert_close(out[r], ref[r], 1e-5, "rank %d step %d" % (r, step))
        p.compare_state(1e-5, "step %d" % step)
        p.compare_ints([capi.VERSION, capi.UPDATES], "step %d" % step)
        prev = bags
    p.close()


def test_cfg5_ten_hot_full_size_pooled():
    # 50 M x 64 table, 32,768 samples x 26 fields x 10 ids: every bag of 10 ids pooled.  Zero table, lr = -1 and
    # integer gradients: rows count integer sums exactly, so a float64 scatter-add on the host is the checker.
    cfg = workloads.CONFIGS["cfg5_zipf"]
    ks = workloads.KeyStream(cfg, seed=0)
    rows, width, n, bag = ks.rows, cfg["width"], ks.n, cfg["hot"]
    nb = n // bag
    print("cfg5_zipf pooled: %d rows x %d, %d keys in %d bags of %d" % (rows, width, n, nb, bag), flush=True)
    capi.seed(0)
    t = capi.Table(0, 1, 0, "", 0, rows, width, 0, 0, np.zeros(rows, np.uint8), np.arange(rows, dtype=np.int64),
                   ("Zero", 0.0, 0.0), -1.0, 0)
    pooled = torch.empty((nb, width), device="cuda")
    rng = np.random.default_rng(9)
    store = np.zeros(rows)                                 # column 0 of every row
    prev_keys, g_int = None, None
    for step in range(3):
        keys = ks.batch()
        dk = torch.from_numpy(keys).cuda()
        dg = None
        if prev_keys is not None:
            g_int = rng.integers(-2, 3, size=nb).astype(np.float32)
            dg = (torch.from_numpy(g_int).cuda()[:, None] * torch.arange(1, width + 1, device="cuda", dtype=torch.float32)).contiguous()
            np.add.at(store, prev_keys, np.repeat(g_int.astype(np.float64), bag))
        torch.cuda.synchronize()
        t.preprocess(dk.data_ptr(), n)
        t.push_pull_pooled(0 if dg is None else dg.data_ptr(), pooled.data_ptr(), bag)
        got = pooled.cpu().numpy()
        want = store[keys].reshape(nb, bag).sum(axis=1)
        assert np.abs(store).max() < 2 ** 23                 # integers this small are exact in fp32, in any order
        assert np.array_equal(got[:, 0], want.astype(np.float32)), "step %d" % step
        assert np.array_equal(got[:, width - 1], (want * width).astype(np.float32))
        prev_keys = keys
    t.close()
