"""Parity of the HIP path (through the C ABI) against the CPU oracle on the same seeded inputs.
Integers bit-exact; fp32 table values and pulled rows within 1e-5 relative (see gpu_util.assert_close)."""
import numpy as np
import pytest

from hetuctr_amd import capi
from oracle import oracle as orc
from tests.gpu_util import Pair, INT_ITEMS_PRE, INT_ITEMS_POST, assert_close
from tests.helpers import zipf_sampler

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


def single(length, width, init=("Uniform", -0.01, 0.01), lr=0.1, seed=0):
    root = np.zeros(length, np.uint8)
    return Pair(1, length, width, root, [np.arange(length, dtype=np.int64)], init=init, lr=lr, seed=seed)


@pytest.mark.parametrize("kind,a,b,tol", [("Zero", 0, 0, 0), ("Uniform", -0.01, 0.01, 0), ("Uniform", 2.0, 5.0, 0),
                                          ("Normal", 0.0, 0.1, 3e-6), ("TruncatedNormal", 1.0, 2.0, 3e-6)])
def test_init_values(kind, a, b, tol):
    say("init", kind)
    length, width = 3000, 24
    for seed in (0, 17):
        p = single(length, width, init=(kind, a, b), seed=seed)
        got = p.tables[0].fetch(capi.EMBEDDING)
        ref = orc.init_values(length * width, kind, a, b, seed)
        if tol == 0:
            assert np.array_equal(got, ref)
        else:  # device erfcinvf vs a double-precision erfcinv: a few ulp of sigma * |z| (|z| < 6.3) plus the rounding
            # of the result next to the mean
            assert np.max(np.abs(got - ref)) <= tol * abs(b) + 2.4e-7 * abs(a)
        p.close()


def test_uniform_init_golden_vectors():
    # the HIP initialiser against the committed known answers (tests/golden/minstd_uniform.json)
    import json
    import os
    say("init golden")
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "minstd_uniform.json")
    length, width = 4400, 16                      # 70,400 values: every offset below 70,000 is covered
    for c in json.load(open(path))["cases"]:
        p = single(length, width, init=("Uniform", c["a"], c["b"]), seed=c["seed"])
        got = p.tables[0].fetch(capi.EMBEDDING).reshape(-1).view(np.uint32)
        for n, bits in zip(c["offsets"], c["f32_bits"]):
            if n < got.shape[0]:
                assert int(got[n]) == bits, (c["seed"], c["a"], c["b"], n)
        p.close()


@pytest.mark.parametrize("gather", ["from the keys", "sorted"])
@pytest.mark.parametrize("width", [1, 3, 4, 16, 20, 64, 128, 200, 256, 300, 512])
def test_single_shard_steps_all_widths(width, gather, monkeypatch):
    # a small batch of one shard is gathered in batch order straight from its keys, a large one in sorted order behind
    # the index: both at every width
    if gather == "sorted":
        monkeypatch.setenv("HETUCTR_DIRECT_GATHER_MAX", "0")
    say("single shard width", width, gather)
    rng = np.random.default_rng(width)
    length, n = 5000, 3000
    p = single(length, width, lr=0.05)
    prev_n = 0
    for step in range(4):
        keys = rng.integers(0, length, size=n - step).astype(np.int64)
        p.preprocess([keys], device_keys=(step % 2 == 1))
        p.compare_ints(INT_ITEMS_PRE, "step %d" % step)
        g = rng.normal(0, 1e-3, size=(prev_n, width)).astype(np.float32)
        out, ref = p.push_pull([g])
        assert_close(out[0], ref[0], 1e-5, "dst step %d" % step)
        p.compare_ints(INT_ITEMS_POST, "step %d" % step)
        p.compare_state(1e-5, "step %d" % step)
        prev_n = keys.shape[0]
    p.close()


@pytest.mark.parametrize("gather", ["from the keys", "sorted"])
def test_one_shard_steps_without_a_look_at_the_index(gather, monkeypatch):
    # nothing is fetched between preprocess and push_pull: with the gather from the keys push_pull returns while the
    # index of its batch may still be running, and the next preprocess (or the fetch below) takes it over
    if gather == "sorted":
        monkeypatch.setenv("HETUCTR_DIRECT_GATHER_MAX", "0")
    say("one shard, no look at the index", gather)
    rng = np.random.default_rng(91)
    length, width = 150_000, 20
    draw = zipf_sampler(length, 1.1, rng)
    p = single(length, width, lr=0.05)
    prev_n = 0
    for step, n in enumerate([5000, 180_000, 3, 70_000, 0, 1, 40_000, 40_000]):
        keys = draw(n) if step % 2 else rng.integers(0, length, size=n).astype(np.int64)
        p.preprocess([keys], device_keys=bool(step % 3))
        g = rng.normal(0, 1e-3, size=(prev_n, width)).astype(np.float32)
        out, ref = p.push_pull([g])
        if step == 6:                                           # the same batches once more, no preprocess in between
            out, ref = p.push_pull([g])
        assert_close(out[0], ref[0], 1e-5, "dst step %d" % step)
        if step % 2:
            p.compare_ints(INT_ITEMS_PRE + INT_ITEMS_POST, "step %d" % step)
            p.compare_state(1e-5, "step %d" % step)
        prev_n = n
    p.compare_ints(INT_ITEMS_PRE + INT_ITEMS_POST, "end")
    p.compare_state(1e-5, "end")
    p.close()


def test_cfg1_cpu_runnable_reference_case():
    # 1,000,000 x 16 table U(-0.01, 0.01); 8,192 x 26 uniform ids; grads N(0, 1e-3); lr 0.1; 10 steps
    say("cfg1")
    rng = np.random.default_rng(0)
    length, width, n = 1_000_000, 16, 8192 * 26
    p = single(length, width, lr=0.1)
    prev_n = 0
    for step in range(10):
        keys = rng.integers(0, length, size=n).astype(np.int64)
        p.preprocess([keys])
        p.compare_ints(INT_ITEMS_PRE, "step %d" % step)
        g = rng.normal(0, 1e-3, size=(prev_n, width)).astype(np.float32)
        out, ref = p.push_pull([g])
        assert_close(out[0], ref[0], 1e-5, "dst step %d" % step)
        prev_n = n
    p.compare_ints([capi.VERSION])
    p.compare_state(1e-5)
    p.close()


@pytest.mark.parametrize("alpha,width", [(1.05, 128), (1.4, 64), (3.0, 16)])
def test_skewed_keys_long_runs(alpha, width):
    # heavy duplicates: runs far longer than a tile, cut by many tile boundaries
    say("skew", alpha, width)
    rng = np.random.default_rng(11)
    length, n = 200_000, 60_000
    draw = zipf_sampler(length, alpha, rng)
    p = single(length, width, lr=0.05)
    prev_n = 0
    for step in range(3):
        keys = draw(n)
        p.preprocess([keys])
        p.compare_ints(INT_ITEMS_PRE, "step %d" % step)
        g = rng.normal(0, 1e-3, size=(prev_n, width)).astype(np.float32)
        out, ref = p.push_pull([g])
        assert_close(out[0], ref[0], 1e-5, "dst step %d" % step)
        p.compare_state(1e-5, "step %d" % step)
        prev_n = n
    p.close()


@pytest.mark.parametrize("nrank", [1, 2])
@pytest.mark.parametrize("width", [128, 20])
def test_gradient_and_output_pointers_off_by_four_bytes(width, nrank):
    # width % 4 == 0 but neither pointer 16-byte aligned: both kernels must fall back to 4-byte lanes (a 64-lane group
    # per row at width 128) and still match the oracle bit for bit; skewed keys, so every role of the push runs
    import torch
    say("unaligned grad / dst, width", width, "shards", nrank)
    rng = np.random.default_rng(700 + width + nrank)
    length, n = 60_000, 50_000
    root = rng.integers(0, nrank, size=length).astype(np.uint8)
    storage = []
    for r in range(nrank):
        own, other = np.where(root == r)[0], np.where(root != r)[0]
        storage.append(np.concatenate([other[::4], own]).astype(np.int64))
    p = Pair(nrank, length, width, root, storage, init=("Uniform", -0.01, 0.01), lr=0.05, bounds=(2, 2) if nrank > 1 else (0, 0))
    draw = zipf_sampler(length, 1.25, rng)
    prev_n = 0
    for step in range(4):
        keys = [draw(n - 3 * step) for _ in range(nrank)]
        p.preprocess(keys, device_keys=True)
        grads = [rng.normal(0, 1e-3, size=(prev_n, width)).astype(np.float32) for _ in range(nrank)]
        gbuf = [torch.empty(prev_n * width + 1, device="cuda") for _ in range(nrank)]   # one float of slack in front
        dbuf = [torch.full((keys[r].shape[0] * width + 1,), float("nan"), device="cuda") for r in range(nrank)]
        for r in range(nrank):
            gbuf[r][1:].copy_(torch.from_numpy(grads[r].reshape(-1)))
        torch.cuda.synchronize()
        gptr = [gbuf[r].data_ptr() + 4 if prev_n else 0 for r in range(nrank)]
        dptr = [dbuf[r].data_ptr() + 4 for r in range(nrank)]
        assert all(q % 16 == 4 for q in dptr)
        capi.group_push_pull(p.tables, gptr, dptr)
        ref = p.oracle.push_pull([g if prev_n else None for g in grads])
        for r in range(nrank):
            out = dbuf[r][1:].cpu().numpy().reshape(-1, width)
            assert_close(out, ref[r], 1e-5, "dst rank %d step %d" % (r, step))
            assert np.isnan(dbuf[r][0].item())                 # nothing was written in front of the first row
        p.compare_state(1e-5, "step %d" % step)
        p.compare_ints([capi.VERSION, capi.UPDATES], "step %d" % step)
        prev_n = n - 3 * step
    p.close()


@pytest.mark.parametrize("width", [48, 192, 256, 512, 1024])
def test_long_runs_slice_layouts(width):
    # long runs with row widths that are cut into 1..32 column slices, or (48) take the path without slices
    say("long runs, width", width)
    rng = np.random.default_rng(width)
    length, n = 50_000, 40_000
    draw = zipf_sampler(length, 1.2, rng)
    p = single(length, width, lr=0.05)
    prev_n = 0
    for step in range(3):
        keys = draw(n)
        p.preprocess([keys], device_keys=True)
        g = rng.normal(0, 1e-3, size=(prev_n, width)).astype(np.float32)
        out, ref = p.push_pull([g])
        assert_close(out[0], ref[0], 1e-5, "dst step %d" % step)
        p.compare_ints(INT_ITEMS_POST, "step %d" % step)
        p.compare_state(1e-5, "step %d" % step)
        prev_n = n
    p.close()


@pytest.mark.parametrize("width", [64, 128])
def test_one_chain_longer_than_every_length_class(width):
    # 140,000 occurrences of one key (more than 2^17) among skewed others, random gradients: the sum must come out in
    # the reference's serial order
    say("giant chain, width", width)
    rng = np.random.default_rng(5)
    length = 30_000
    draw = zipf_sampler(length, 1.1, rng)
    p = single(length, width, lr=0.05)
    prev_n = 0
    for step in range(2):
        keys = np.concatenate([np.full(140_000, 7, np.int64), draw(30_000)])
        rng.shuffle(keys)
        p.preprocess([keys], device_keys=True)
        g = rng.normal(0, 1e-3, size=(prev_n, width)).astype(np.float32)
        out, ref = p.push_pull([g])
        assert_close(out[0], ref[0], 1e-5, "dst step %d" % step)
        p.compare_state(1e-5, "step %d" % step)
        prev_n = keys.shape[0]
    p.close()


def test_one_key_repeated_and_all_distinct():
    say("extremes")
    length, width = 70_000, 32
    p = single(length, width, init=("Zero", 0, 0), lr=-1.0)
    n = 40_000
    for keys in (np.full(n, 123, np.int64), np.arange(n, dtype=np.int64), np.arange(n, dtype=np.int64)[::-1].copy()):
        p.preprocess([keys])
        p.compare_ints(INT_ITEMS_PRE)
        out, ref = p.push_pull([np.ones((p.tables[0].fetch(capi.SIZES)[2], width), np.float32)])
        assert np.array_equal(out[0], ref[0])  # integer-valued sums: exact in any order
    p.close()


def test_empty_batches_double_preprocess_inference():
    say("protocol edge cases")
    length, width = 100, 8
    p = single(length, width, init=("Zero", 0, 0), lr=-1.0)
    p.preprocess([np.zeros(0, np.int64)])                    # tests/check.py:40
    p.compare_ints(INT_ITEMS_PRE)
    out, ref = p.push_pull([np.zeros((0, width), np.float32)])
    a = np.array([1, 1, 3], np.int64)
    b = np.array([0, 1, 2, 3], np.int64)
    p.preprocess([a]); p.preprocess([b])                     # tests/driver.py:31-32
    p.compare_ints(INT_ITEMS_PRE)
    out, ref = p.push_pull([np.array([[1.0] * width, [2.0] * width, [4.0] * width], np.float32)])
    assert out[0][:, 0].tolist() == [0.0, 3.0, 0.0, 4.0] and np.array_equal(out[0], ref[0])
    p.preprocess([np.array([1], np.int64)])
    out, ref = p.push_pull([None])                           # inference, hetu_gpu_table.cu:14-21
    assert out[0][0, 0] == 3.0 and np.array_equal(out[0], ref[0])
    p.preprocess([np.array([1], np.int64)])
    out, ref = p.push_pull([np.full((1, width), 5.0, np.float32)])
    assert out[0][0, 0] == 8.0 and np.array_equal(out[0], ref[0])
    p.compare_ints([capi.VERSION])
    p.close()


def test_out_of_range_key_is_reported():
    p = single(10, 4)
    with pytest.raises(RuntimeError, match="outside"):
        p.tables[0].preprocess(np.array([3, 10], np.int64).ctypes.data, 2)
    with pytest.raises(RuntimeError, match="outside"):
        p.tables[0].preprocess(np.array([-1], np.int64).ctypes.data, 1)
    k = np.array([3, 9], np.int64)
    p.tables[0].preprocess(k.ctypes.data, 2)                 # still usable afterwards
    assert p.tables[0].fetch(capi.UNIQUE).tolist() == [3, 9]
    p.close()


def test_constructor_errors_and_strings():
    root = np.zeros(8, np.uint8)
    with pytest.raises(RuntimeError, match="every id"):
        capi.Table(0, 1, 0, "", 0, 8, 4, 0, 0, root, np.arange(7), ("Zero", 0, 0), 0.1)
    with pytest.raises(RuntimeError, match="twice"):
        capi.Table(0, 1, 0, "", 0, 8, 4, 0, 0, root, np.array([0, 1, 2, 3, 4, 5, 6, 7, 7]), ("Zero", 0, 0), 0.1)
    with pytest.raises(RuntimeError, match="device"):
        capi.Table(0, 1, 99, "", 0, 8, 4, 0, 0, root, np.arange(8), ("Zero", 0, 0), 0.1)
    t = capi.Table(0, 1, 0, "", 0, 8, 4, 3, 5, root, np.arange(8), ("Zero", 0, 0), 0.1)
    assert repr(t) == "<HetuTable root/store/all=8/8/8>"       # csrc/core/debug.cu:5-12
    assert t.debug() == "<HetuTable root/store/all=8/8/8 rank=0 nrank=1 device_id=0 width=4 push/pull=5/3>"
    t.close()


def test_key_buffer_is_free_when_preprocess_returns():
    # preprocess returns before the batch is sorted; the caller may overwrite its id buffer at once, whether it
    # lives on the device or on the host, and every step still matches the oracle
    import torch
    say("ids overwritten right after preprocess")
    rng = np.random.default_rng(31)
    length, width, n = 40_000, 32, 30_000
    p = single(length, width, lr=0.05)
    t, o = p.tables[0], p.oracle
    with pytest.raises(RuntimeError, match="call timing is off"):
        t.last_times()                                    # no silent switch: the getter refuses while timing is off
    t.call_timing(True)
    dev = torch.empty(n, dtype=torch.int64, device="cuda")
    host = np.empty(n, np.int64)
    dst = torch.empty((n, width), device="cuda")
    prev = 0
    for step in range(8):
        keys = rng.integers(0, length, size=n).astype(np.int64)
        if step % 2:
            dev.copy_(torch.from_numpy(keys))
            torch.cuda.synchronize()
            t.preprocess(dev.data_ptr(), n)
            dev.fill_(-1)                                 # next work on the default stream: ordered after ours
        else:
            host[:] = keys
            t.preprocess(host.ctypes.data, n)
            host[:] = -1
        g = rng.normal(0, 1e-3, size=(prev, width)).astype(np.float32)
        dg = torch.from_numpy(g).cuda()
        torch.cuda.synchronize()
        t.push_pull(dg.data_ptr() if prev else 0, dst.data_ptr())
        o.preprocess([keys])
        ref = o.push_pull([g if prev else None])[0]
        assert np.array_equal(dst.cpu().numpy(), ref), "step %d" % step
        pre_ms, pp_ms = t.last_times()
        assert pre_ms > 0 and pp_ms > 0 and 0 <= t.last_push_ms() <= pp_ms   # device times of the two calls
        for item in (capi.UNIQUE, capi.SORTED_ARG, capi.RUN_START, capi.IDX_MAP, capi.KEYS):
            assert np.array_equal(t.fetch(item), o.fetch(0, item)), (step, item)
        prev = n
    p.close()


def test_repeated_and_changing_batch_sizes():
    # many steps of one batch size, then size changes, an empty batch, a doubled preprocess and state fetches between
    # preprocess and push_pull (each of which has to wait for the index still running on the second stream)
    say("repeated and changing batch sizes")
    rng = np.random.default_rng(32)
    length, width = 60_000, 16
    p = single(length, width, lr=0.1)
    sizes = [20_000] * 7 + [5_000, 20_000, 20_000, 0, 20_000, 20_000, 45_000, 45_000, 45_000, 45_000, 20_000, 20_000]
    prev_n = 0
    for step, n in enumerate(sizes):
        keys = rng.integers(0, length, size=n).astype(np.int64)
        if step == 12:                                     # preprocess twice in a row: the first batch becomes "previous"
            extra = rng.integers(0, length, size=20_000).astype(np.int64)
            p.preprocess([extra], device_keys=True)
            prev_n = 20_000
        p.preprocess([keys], device_keys=(step % 3 != 0))
        if step % 4 == 1:
            p.compare_ints(INT_ITEMS_PRE, "step %d before push_pull" % step)
        g = rng.normal(0, 1e-3, size=(prev_n, width)).astype(np.float32)
        out, ref = p.push_pull([g])
        assert_close(out[0], ref[0], 1e-5, "dst step %d" % step)
        p.compare_ints([capi.UNIQUE, capi.SORTED_ARG, capi.RUN_START, capi.IDX_MAP, capi.SIZES, capi.VERSION], "step %d" % step)
        prev_n = n
    p.compare_state(1e-5, "end")
    p.close()


@pytest.mark.parametrize("tile_sorted", [True, False])
@pytest.mark.parametrize("nrank", [1, 2])
def test_batch_sizes_where_the_sort_changes_shape(nrank, tile_sorted, monkeypatch):
    # Both sorts of the index.  The tile-sorted passes: 2, 4, 8, 13 keys per thread (tiles of 1024 ... 6656 keys, at most
    # 256 tiles) up to 1.5 M keys, the first launch from ids or -- from 2^20 keys on, when preprocess returns early --
    # from keys made by a kernel of its own.  The three-launch passes (all sizes when HETUCTR_TILE_SORT=0, else above
    # 1.5 M keys): 1024-key tiles up to 2^17 keys (up to 64 of them without scan launches), 4096- and 8192-key tiles
    # above.  The sizes on both sides of every switch, one after the other on one table (the scratch of one size is
    # reused by the next).
    if not tile_sorted:
        monkeypatch.setenv("HETUCTR_TILE_SORT", "0")
    say("sort shapes, shards", nrank, "tile-sorted passes" if tile_sorted else "three-launch passes")
    rng = np.random.default_rng(35 + nrank)
    length, width = 3_000_000, 4                           # 22-bit ids (+ 1 bit of rank): three digit widths in a sort
    root = rng.integers(0, nrank, size=length).astype(np.uint8)
    storage = [np.flatnonzero(root == r).astype(np.int64) for r in range(nrank)]
    p = Pair(nrank, length, width, root, storage, init=("Zero", 0.0, 0.0), lr=0.5)
    sizes = [1024, 1025, 65536, 65537, 65536 + 1024, 131072, 131073, 1023, 140_000, 64 * 1024 - 1,
             262144, 262145, 524288, 524289, 5000, 1048575, 1048576, 1048577, 3 << 19, (3 << 19) + 1, 2047]
    prev_n = [0] * nrank
    for step, n in enumerate(sizes):
        ns = [n if r == 0 else max(n // 3, 1) for r in range(nrank)]
        keys = [rng.integers(0, length, size=k).astype(np.int64) for k in ns]
        p.preprocess(keys, device_keys=True)
        p.compare_ints([capi.UNIQUE, capi.SORTED_ARG, capi.RUN_START, capi.IDX_MAP, capi.SIZES, capi.KEYS], "n %d" % n)
        out, ref = p.push_pull([rng.normal(0, 1e-2, size=(k, width)).astype(np.float32) for k in prev_n])
        for r in range(nrank):
            assert_close(out[r], ref[r], 1e-5, "dst n %d rank %d" % (n, r))
        prev_n = ns
    p.compare_state(1e-5, "end")
    p.close()


@pytest.mark.parametrize("bits,nrank,digit", [(3, 1, 0), (10, 1, 0), (11, 1, 0), (20, 1, 0), (21, 1, 0), (24, 2, 0),
                                              (22, 1, 3), (23, 2, 5)])
def test_sort_passes_for_every_key_width(bits, nrank, digit, monkeypatch):
    # one, two and three digit passes with digits of 3 to 10 bits, and (digit: a narrower widest digit) eight and five
    # passes; skewed keys, so that some blocks of a pass see a single digit value and others hundreds; preprocess
    # returns early (first launch beside the call) and, every other step, only when all is done
    if digit:
        monkeypatch.setenv("HETUCTR_TILE_DIGIT_BITS", str(digit))
    say("id bits", bits, "shards", nrank, "digits of at most", digit or 10, "bits")
    rng = np.random.default_rng(900 + bits)
    length, width = (1 << bits) - (3 if bits > 2 else 0), 1
    root = rng.integers(0, nrank, size=length).astype(np.uint8)
    storage = [np.flatnonzero(root == r).astype(np.int64) for r in range(nrank)]
    p = Pair(nrank, length, width, root, storage, init=("Zero", 0.0, 0.0), lr=1.0)
    prev_n = [0] * nrank
    for step, n in enumerate([100_000, 300_000, 7, 40_000]):
        p.tables[0].defer_index(step % 2 == 0)
        # Zipf ranks spread over the id range by a fixed odd multiplier: hot ids everywhere, every digit in use
        keys = [(np.minimum(rng.zipf(1.1, size=n), length) - 1) * 2654435761 % length for _ in range(nrank)]
        p.preprocess(keys, device_keys=True)
        p.compare_ints([capi.UNIQUE, capi.SORTED_ARG, capi.RUN_START, capi.IDX_MAP, capi.ROOT, capi.SIZES, capi.KEYS], "n %d" % n)
        out, ref = p.push_pull([rng.integers(-2, 3, size=(k, width)).astype(np.float32) for k in prev_n])
        for r in range(nrank):
            assert_close(out[r], ref[r], 1e-5, "dst n %d rank %d" % (n, r))
        prev_n = [n] * nrank
    p.close()


def test_large_batches_of_ids_in_pageable_host_memory():
    # ids handed over as numpy arrays (the reference's drivers do), megabytes at a time: sizes around powers of two and
    # odd ones, the same array object reused and overwritten right after the call
    say("large host batches")
    rng = np.random.default_rng(36)
    length, width = 500_000, 4
    p = single(length, width, init=("Zero", 0.0, 0.0), lr=0.5)
    buf = np.zeros(400_003, np.int64)
    # (a copy of 1 MiB or more is staged by several threads in 128 KiB pieces and transferred 1 MiB at a time)
    for step, n in enumerate([262_143, 262_144, 262_145, 400_003, 131_072 * 3 + 1, 300_000, 5, 100_000, 131_071, 131_072,
                              16_384 * 9 + 1, 16_384 * 17 - 1]):
        want = rng.integers(0, length, size=n).astype(np.int64)
        buf[:n] = want
        p.tables[0].preprocess(buf.ctypes.data, n)
        buf[:n] = -1                                        # overwritten as soon as the call is back
        p.oracle.preprocess([want])
        p.n = [n]
        p.compare_ints([capi.UNIQUE, capi.SORTED_ARG, capi.RUN_START, capi.IDX_MAP, capi.KEYS], "n %d" % n)
        out, ref = p.push_pull([None])
        assert_close(out[0], ref[0], 1e-5, "dst n %d" % n)
    # an id out of range in the middle of a large host batch is reported by the call
    # (ids from host memory travel as 32-bit words when the table's ids fit: one that does not fit must not alias a valid id)
    for bad in (length, -1, 1 << 40, (1 << 32) + 5, -(1 << 33)):
        keys = rng.integers(0, length, size=300_000).astype(np.int64)
        keys[123_456] = bad
        with pytest.raises(RuntimeError, match="outside"):
            p.tables[0].preprocess(keys.ctypes.data, keys.shape[0])
        want = keys.copy()
        want[123_456] = 0                                   # "it was treated as id 0"
        p.oracle.preprocess([want])
        p.n = [keys.shape[0]]
        p.compare_ints([capi.UNIQUE, capi.SORTED_ARG, capi.RUN_START, capi.KEYS], "bad id %d" % bad)
    p.close()


def test_host_ids_from_two_threads_at_once():
    # two tables, each fed large host batches by a thread of its own: the threads that stage host ids are shared by
    # the process, a copy posted while another is under way must leave both batches intact
    import threading
    say("host ids from two threads")
    length, width, steps = 300_000, 4, 6
    tables = [single(length, width, init=("Zero", 0.0, 0.0), lr=0.5) for _ in range(2)]
    errors = []

    def feed(i):
        try:
            rng = np.random.default_rng(50 + i)
            t = tables[i].tables[0]
            for step in range(steps):
                n = 200_000 + 37 * i + 1000 * step               # 1.6 MB of ids: staged by the crew
                want = rng.integers(0, length, size=n).astype(np.int64)
                buf = want.copy()
                t.preprocess(buf.ctypes.data, n)
                buf[:] = -1
                got = t.fetch(capi.KEYS)
                if not np.array_equal(got, want):
                    errors.append("table %d step %d: %d ids differ" % (i, step, int((got != want).sum())))
        except Exception as e:                                   # noqa: BLE001 - reported by the main thread
            errors.append("table %d: %r" % (i, e))

    threads = [threading.Thread(target=feed, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    for p in tables:
        p.close()
    assert not errors, errors


@pytest.mark.parametrize("nrank", [1, 3])
def test_64_bit_sort_keys_at_every_sort_shape(nrank, monkeypatch):
    # sort keys wider than 32 bits (owner and id of a huge id space) are forced on a small table; batch sizes from
    # the three tile shapes of the sort, the largest one with its count columns scanned in pieces
    monkeypatch.setenv("HETUCTR_FORCE_WIDE_KEYS", "1")
    say("64-bit sort keys, shards", nrank)
    rng = np.random.default_rng(37 + nrank)
    length, width = 2_000_000, 2
    root = rng.integers(0, nrank, size=length).astype(np.uint8)
    storage = [np.flatnonzero(root == r).astype(np.int64) for r in range(nrank)]
    p = Pair(nrank, length, width, root, storage, init=("Zero", 0.0, 0.0), lr=0.5)
    prev_n = [0] * nrank
    for n in [3000, 70_000, 200_000, 4_300_000, 1_100_000, 300_000, 600_000, 1_572_864]:
        ns = [n if r == 0 else max(n // 5, 1) for r in range(nrank)]
        keys = [rng.integers(0, length, size=k).astype(np.int64) for k in ns]
        p.preprocess(keys, device_keys=True)
        p.compare_ints([capi.UNIQUE, capi.SORTED_ARG, capi.RUN_START, capi.IDX_MAP, capi.SIZES], "n %d" % n)
        out, ref = p.push_pull([rng.integers(-2, 3, size=(k, width)).astype(np.float32) for k in prev_n])
        for r in range(nrank):
            assert_close(out[r], ref[r], 1e-5, "dst n %d rank %d" % (n, r))
        prev_n = ns
    p.compare_state(1e-5, "end")
    p.close()


def test_key_error_is_raised_by_preprocess_and_the_table_goes_on():
    say("bad key, early return")
    length, width, n = 1000, 8, 500
    p = single(length, width)
    t = p.tables[0]
    rng = np.random.default_rng(33)
    good = rng.integers(0, length, size=n).astype(np.int64)
    bad = good.copy()
    bad[17] = length + 5
    p.preprocess([good])
    p.push_pull([np.zeros((0, width), np.float32)])
    with pytest.raises(RuntimeError, match="outside"):
        t.preprocess(bad.ctypes.data, n)
    import torch
    dst = torch.empty((n, width), device="cuda")
    t.push_pull(0, dst.data_ptr())                         # the batch is usable (the key counted as id 0)
    for _ in range(3):                                     # and the flag does not come back
        t.preprocess(good.ctypes.data, n)
        t.push_pull(0, dst.data_ptr())
    ref = p.oracle.fetch(0, capi.EMBEDDING).reshape(length, width)[good]
    assert np.array_equal(dst.cpu().numpy(), ref)
    p.close()


def test_preprocess_that_waits_for_all_its_work(monkeypatch):
    # HETUCTR_DEFER_INDEX=0: the reference's call protocol literally (preprocess returns when the batch is indexed)
    say("synchronous preprocess")
    monkeypatch.setenv("HETUCTR_DEFER_INDEX", "0")
    rng = np.random.default_rng(34)
    length, width, n = 30_000, 64, 25_000
    p = single(length, width, lr=0.05)
    prev_n = 0
    for step in range(5):
        keys = rng.integers(0, length, size=n).astype(np.int64)
        p.preprocess([keys], device_keys=True)
        g = rng.normal(0, 1e-3, size=(prev_n, width)).astype(np.float32)
        out, ref = p.push_pull([g])
        assert_close(out[0], ref[0], 1e-5, "dst step %d" % step)
        prev_n = n
    p.compare_ints([capi.VERSION])
    p.close()


def test_table_closed_while_the_index_is_still_running():
    # preprocess returns early; destroying the table right away must wait for what it left on the GPU
    say("close right after preprocess")
    import torch
    rng = np.random.default_rng(35)
    length, width, n = 200_000, 32, 150_000
    for _ in range(3):
        p = single(length, width)
        keys = torch.from_numpy(rng.integers(0, length, size=n).astype(np.int64)).cuda()
        torch.cuda.synchronize()
        p.tables[0].preprocess(keys.data_ptr(), n)
        p.close()
    p = single(length, width)                      # and a fresh table works afterwards
    k = rng.integers(0, length, size=n).astype(np.int64)
    p.preprocess([k])
    out, ref = p.push_pull([np.zeros((0, width), np.float32)])
    assert np.array_equal(out[0], ref[0])
    p.close()


@pytest.mark.parametrize("nrank", [1, 2])
def test_push_pull_twice_without_preprocess(nrank):
    # The same previous batch pushed twice: the reference applies the whole gradient again
    # (csrc/core/hetu_gpu_table.cu:9-41 keeps no "already pushed" state), including the keys with more than 128
    # duplicates, whose blocks draw their work from counters that have to be back at zero for the second launch.
    say("push_pull twice, shards", nrank)
    rng = np.random.default_rng(36 + nrank)
    length, width, n = 20_000, 128, 30_000
    root = (np.arange(length) % nrank).astype(np.uint8)
    storage = [np.concatenate([np.where(root == r)[0], np.where(root != r)[0][:500]]).astype(np.int64)
               for r in range(nrank)]
    p = Pair(nrank, length, width, root, storage, init=("Uniform", -0.01, 0.01), lr=0.05, bounds=(2, 2))
    draw = zipf_sampler(length, 1.2, rng)

    def batch():
        k = np.concatenate([np.full(3000, 5, np.int64), np.full(700, 6, np.int64), np.full(200, 9, np.int64),
                            draw(n - 3900)])
        rng.shuffle(k)
        return k

    p.preprocess([batch() for _ in range(nrank)], device_keys=True)
    p.preprocess([batch() for _ in range(nrank)], device_keys=True)
    for rep in range(3):
        g = [rng.normal(0, 1e-3, size=(n, width)).astype(np.float32) for _ in range(nrank)]
        out, ref = p.push_pull(g)
        for r in range(nrank):
            assert_close(out[r], ref[r], 1e-5, "dst rank %d, push %d" % (r, rep))
        p.compare_ints([capi.VERSION, capi.UPDATES], "push %d" % rep)
        p.compare_state(1e-5, "push %d" % rep)
    p.preprocess([batch() for _ in range(nrank)])          # and the table goes on as usual
    out, ref = p.push_pull([rng.normal(0, 1e-3, size=(n, width)).astype(np.float32) for _ in range(nrank)])
    for r in range(nrank):
        assert_close(out[r], ref[r], 1e-5, "dst rank %d after" % r)
    p.compare_state(1e-5, "after")
    p.close()
