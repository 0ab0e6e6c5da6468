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
        else:  # device erfcinvf vs a double-precision erfcinv: last-bit differences, scaled by sigma
            assert np.max(np.abs(got - ref)) <= tol * max(abs(b), 1.0) * 10
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


@pytest.mark.parametrize("width", [1, 3, 4, 16, 20, 64, 128, 200, 256, 300, 512])
def test_single_shard_steps_all_widths(width):
    say("single shard width", width)
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
