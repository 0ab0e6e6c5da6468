"""hctr_save / hctr_load through the C ABI: a shard's rows, versions, pending gradients and update counters survive
the round trip bit for bit, and a table restored from a file goes on exactly like the one that wrote it."""
import os

import numpy as np
import pytest
import torch

from hetuctr_amd import capi
from tests.gpu_util import Pair
from tests.helpers import zipf_sampler

pytestmark = pytest.mark.gpu

STATE = (capi.EMBEDDING, capi.VERSION, capi.PENDING, capi.UPDATES, capi.STORE_IDS)


def layout(nrank, length, rng):
    root = rng.integers(0, nrank, size=length).astype(np.uint8)
    storage = []
    for r in range(nrank):
        own = np.where(root == r)[0]
        other = np.where(root != r)[0]
        storage.append(np.concatenate([other[: len(other) // 3], own]).astype(np.int64))  # a third of the others cached
    return root, storage


def steps(p, rng, draw, n, width, count, prev_n):
    outs = []
    for _ in range(count):
        p.preprocess([draw(n) for _ in range(p.R)], device_keys=True)
        g = [rng.normal(0, 1e-2, size=(prev_n, width)).astype(np.float32) for _ in range(p.R)]
        outs.append(p.push_pull(g)[0])
        prev_n = n
    return outs


@pytest.mark.parametrize("nrank", [1, 3])
def test_round_trip_and_continue(nrank, tmp_path):
    print("checkpoint round trip, shards", nrank, flush=True)
    rng = np.random.default_rng(50 + nrank)
    length, width, n = 30_000, 24, 20_000
    root, storage = layout(nrank, length, rng)
    draw = zipf_sampler(length, 1.1, rng)
    a = Pair(nrank, length, width, root, storage, init=("Normal", 0.0, 0.1), lr=0.05, bounds=(4, 4), seed=1,
             with_oracle=False)
    steps(a, rng, draw, n, width, 4, 0)
    paths = [str(tmp_path / ("shard%d.ckpt" % r)) for r in range(nrank)]
    for r in range(nrank):
        a.tables[r].save(paths[r])
    want = [[a.tables[r].fetch(it) for it in STATE] for r in range(nrank)]
    if nrank > 1:                                        # the state worth saving is there: pending gradients, counters
        assert any(np.abs(w[2]).max() > 0 for w in want) and any(w[3].max() > 0 for w in want)
    b = Pair(nrank, length, width, root, storage, init=("Uniform", -1.0, 1.0), lr=0.05, bounds=(4, 4), seed=9,
             with_oracle=False)
    assert not np.array_equal(b.tables[0].fetch(capi.EMBEDDING), want[0][0])
    for r in range(nrank):
        b.tables[r].load(paths[r])
    for r in range(nrank):
        for it, w in zip(STATE, want[r]):
            assert np.array_equal(b.tables[r].fetch(it), w), "item %d of rank %d after load" % (it, r)
        assert os.path.getsize(paths[r]) == 64 + sum(w.nbytes for w in want[r])
    # both go on from here: the writer drops the gradients of its last batch (an inference step), the restored
    # table has no last batch; after that the same steps give the same rows
    state = rng.bit_generator.state
    for p in (a, b):
        rng.bit_generator.state = state
        p.preprocess([draw(n) for _ in range(nrank)], device_keys=True)
        first = p.push_pull([None] * nrank)[0]
        rest = steps(p, rng, draw, n, width, 3, n)
        if p is a:
            ref = [first] + rest
        else:
            for x, y in zip([first] + rest, ref):
                for r in range(nrank):
                    assert np.array_equal(x[r], y[r])
    for r in range(nrank):
        for it in STATE:
            assert np.array_equal(a.tables[r].fetch(it), b.tables[r].fetch(it))
    a.close()
    b.close()


def test_refusals(tmp_path):
    length, width = 500, 8
    root = np.zeros(length, np.uint8)
    st = np.arange(length, dtype=np.int64)
    t = capi.Table(0, 1, 0, "", 0, length, width, 0, 0, root, st, ("Uniform", -1, 1), 0.1)
    good = str(tmp_path / "t.ckpt")
    t.save(good)
    other = capi.Table(0, 1, 0, "", 0, length, width + 4, 0, 0, root, st, ("Zero", 0, 0), 0.1)
    with pytest.raises(RuntimeError, match="width"):
        other.load(good)
    perm = capi.Table(0, 1, 0, "", 0, length, width, 0, 0, root, st[::-1].copy(), ("Zero", 0, 0), 0.1)
    with pytest.raises(RuntimeError, match="resident ids"):
        perm.load(good)
    assert not os.path.exists(good + ".tmp")              # written beside the target, renamed when complete
    # a step moves the table away from what the file holds: a refused load must leave it exactly there
    keys = torch.arange(0, 300, 3, dtype=torch.int64, device="cuda")
    dst = torch.empty((100, width), device="cuda")
    g = torch.full((100, width), 0.25, device="cuda")
    torch.cuda.synchronize()
    t.preprocess(keys.data_ptr(), 100)
    t.push_pull(0, dst.data_ptr())
    t.preprocess(keys.data_ptr(), 100)
    t.push_pull(g.data_ptr(), dst.data_ptr())
    emb, ver = t.fetch(capi.EMBEDDING), t.fetch(capi.VERSION)
    saved = np.fromfile(good, dtype=np.float32, offset=64 + 8 * length, count=length * width)
    assert not np.array_equal(emb, saved)
    cut = str(tmp_path / "cut.ckpt")
    open(cut, "wb").write(open(good, "rb").read()[:-100])
    with pytest.raises(RuntimeError, match="shorter than the table"):
        t.load(cut)
    longer = str(tmp_path / "long.ckpt")
    open(longer, "wb").write(open(good, "rb").read() + b"\0" * 8)
    with pytest.raises(RuntimeError, match="longer than the table"):
        t.load(longer)
    assert np.array_equal(t.fetch(capi.EMBEDDING), emb) and np.array_equal(t.fetch(capi.VERSION), ver)
    with pytest.raises(RuntimeError, match="cannot open"):  # a target that cannot be written leaves nothing behind
        t.save(str(tmp_path / "no_such_dir" / "t.ckpt"))
    junk = str(tmp_path / "junk.ckpt")
    open(junk, "wb").write(b"x" * 4096)
    with pytest.raises(RuntimeError, match="not a hetuCTR checkpoint"):
        t.load(junk)
    with pytest.raises(RuntimeError, match="cannot open"):
        t.load(str(tmp_path / "missing.ckpt"))
    t.load(good)                                          # and the table is still usable
    keys = torch.arange(100, dtype=torch.int64, device="cuda")
    dst = torch.empty((100, width), device="cuda")
    torch.cuda.synchronize()
    t.preprocess(keys.data_ptr(), 100)
    t.push_pull(0, dst.data_ptr())
    assert np.array_equal(dst.cpu().numpy().reshape(-1), t.fetch(capi.EMBEDDING)[: 100 * width])
    for x in (t, other, perm):
        x.close()
