"""The reference's own test scripts (tests/check.py, tests/test_update.py, tests/driver.py) against the
`hetuCTR` python module, with one thread per rank instead of one process per GPU: all shards live on the one GPU
and the loopback group replaces NCCL."""
import threading

import numpy as np
import pytest
import torch

import hetuctr_amd

pytestmark = pytest.mark.gpu
_port = [23456]


def run_ranks(nrank, worker):
    """Starts worker(rank, port) on nrank threads (tests/check.py:48-51 forks processes) and re-raises failures."""
    _port[0] += 1
    errors = []

    def wrap(r):
        try:
            worker(r, _port[0])
        except BaseException as e:  # noqa: BLE001
            errors.append((r, e))

    ts = [threading.Thread(target=wrap, args=(r,)) for r in range(nrank)]
    [t.start() for t in ts]
    [t.join(120) for t in ts]
    assert not any(t.is_alive() for t in ts), "a rank did not finish"
    if errors:
        raise errors[0][1]


def test_check_py():
    # tests/check.py with its parameters: 4 ranks, width 128, 1024 ids, bounds 10/10, lr 1, Normal(0, 1)
    hetuCTR = hetuctr_amd.load_hetuCTR()
    nrank, width, length, batch_size = 4, 128, 1024, 1024
    np.random.seed(0)
    root_arr = np.random.randint(nrank, size=length)
    lock = threading.Lock()

    def checkvalue(k, v):
        # equal keys -> equal rows (check.py:14-23).  The script's "distinct keys -> distinct values" clause only
        # holds among keys of one owner: every rank draws the same values for equal storage offsets.
        v = v[:len(k), 0]
        kv = {}
        for i in range(len(k)):
            if k[i] in kv:
                assert kv[k[i]] == v[i]
            else:
                kv[k[i]] = v[i]
        for own in range(nrank):
            vals = [x for key, x in kv.items() if root_arr[key] == own]
            assert len(set(vals)) == len(vals)

    def worker(rank, port):
        dest = torch.zeros([batch_size, width]).cuda()
        grad = torch.rand([batch_size, width]).cuda()
        init = hetuCTR.Initializer(hetuCTR.InitType.Normal, 0, 1)
        storage_arr = np.where(root_arr == rank)[0]
        table = hetuCTR.HetuTable(
            rank=rank, nrank=nrank, device_id=0, ip="127.0.0.1", port=port,
            pull_bound=10, push_bound=10, init=init, learning_rate=1,
            length=length, width=width,
            root_arr=root_arr, storage_arr=storage_arr, verbose=0)
        with lock:
            embed_id = np.random.randint(length, size=batch_size, dtype=np.int64)
        table.preprocess(embed_id.ctypes.data, 0)
        for i in range(5):
            with lock:
                embed_id = np.random.randint(length, size=batch_size, dtype=np.int64)
            table.preprocess(embed_id.ctypes.data, embed_id.shape[0])
            table.push_pull(grad.data_ptr(), dest.data_ptr())
            checkvalue(embed_id, dest.cpu())
        assert repr(table).startswith("<HetuTable root/store/all=") and "push/pull=10/10" in table.debug()

    run_ranks(nrank, worker)


@pytest.mark.parametrize("random_grads", [False, True])
def test_update_py(random_grads):
    # tests/test_update.py::test_one (grad == 1, exact) and ::test_two (random grads, 1e-4)
    hetuCTR = hetuctr_amd.load_hetuCTR()
    nrank, width, length, batch_size = 4, 128, 1024, 1024
    np.random.seed(0)
    root_arr = np.random.randint(nrank, size=length)
    # the per-rank key / gradient streams are drawn up front: the script's np.random.seed(rank) is per process
    rngs = [np.random.RandomState(rank) for rank in range(nrank)]
    steps = 50
    keys = [[rngs[r].randint(length, size=batch_size).astype(np.int64) for _ in range(steps)] for r in range(nrank)]
    grads = [[rngs[r].rand(batch_size, width).astype(np.float32) if random_grads else
              np.ones((batch_size, width), np.float32) for _ in range(steps)] for r in range(nrank)]
    final = [None] * nrank

    def worker(rank, port):
        dest = torch.zeros([batch_size, width]).cuda()
        init = hetuCTR.Initializer(hetuCTR.InitType.Zero, 0, 0)
        storage_arr = np.where(root_arr <= rank)[0]
        table = hetuCTR.HetuTable(
            rank=rank, nrank=nrank, device_id=0, ip="127.0.0.1", port=port,
            pull_bound=0, push_bound=0, init=init, learning_rate=-1,
            length=length, width=width,
            root_arr=root_arr, storage_arr=storage_arr, verbose=0)
        empty = np.zeros(0, np.int64)
        table.preprocess(empty.ctypes.data, 0)
        for i in range(steps):
            g = torch.from_numpy(grads[rank][i - 1] if i else grads[rank][0]).cuda()
            torch.cuda.synchronize()
            table.preprocess(keys[rank][i].ctypes.data, batch_size)
            table.push_pull(g.data_ptr(), dest.data_ptr())
        final[rank] = dest.cpu().numpy()[:, 0].copy()

    run_ranks(nrank, worker)
    store = np.zeros(length)
    for r in range(nrank):
        for i in range(steps - 1):   # the last batch's gradients are never pushed
            np.add.at(store, keys[r][i], grads[r][i][:, 0].astype(np.float64))
    for r in range(nrank):
        expect = store[keys[r][steps - 1]]
        if random_grads:
            assert np.max(np.abs(final[r] - expect)) < 1e-4          # test_update.py:70
        else:
            assert np.array_equal(final[r], expect.astype(np.float32))  # test_update.py:43


def test_driver_py_sequence_and_async():
    # tests/driver.py:31-38: two preprocess calls, one push_pull, then the async forms with wait()
    hetuCTR = hetuctr_amd.load_hetuCTR()
    length, width = 1000, 16
    root_arr = np.zeros(length, np.int64)
    hetuCTR.seed(5)
    table = hetuCTR.HetuTable(rank=0, nrank=1, device_id=0, ip="127.0.0.1", port=1, length=length, width=width,
                              pull_bound=0, push_bound=0, root_arr=root_arr, storage_arr=np.arange(length),
                              init=hetuCTR.Initializer(hetuCTR.InitType.Uniform, -1, 1), learning_rate=0.5, verbose=0)
    hetuCTR.seed(0)
    dest = torch.zeros([10, width]).cuda()
    grad = torch.ones([10, width]).cuda()
    torch.cuda.synchronize()
    embed_id = np.arange(10, dtype=np.int64)
    table.preprocess(embed_id.ctypes.data, 10)
    table.preprocess(embed_id.ctypes.data, 10)
    table.push_pull(grad.data_ptr(), dest.data_ptr())
    first = dest.cpu().numpy().copy()
    emb0 = table.debug_fetch(16).reshape(length, width)[:10] + 0.5      # state after the push: init - 0.5
    assert np.allclose(first, emb0 - 0.5, rtol=1e-6)
    w1 = table.async_preprocess(embed_id.ctypes.data, 10)
    w2 = table.async_push_pull(grad.data_ptr(), dest.data_ptr())
    w1.wait(); w2.wait()
    assert np.allclose(dest.cpu().numpy(), first - 0.5, rtol=1e-6)
    w3 = table.async_preprocess(np.array([length], np.int64).ctypes.data, 1)   # error travels through wait()
    with pytest.raises(RuntimeError, match="outside"):
        w3.wait()
    # a seed changes the table, the same seed reproduces it (csrc/pybind/pybind.cu:77)
    def first_rows(seed):
        hetuCTR.seed(seed)
        t = hetuCTR.HetuTable(rank=0, nrank=1, device_id=0, ip="", port=0, length=8, width=4, pull_bound=0,
                              push_bound=0, root_arr=np.zeros(8, np.int64), storage_arr=np.arange(8),
                              init=hetuCTR.Initializer(hetuCTR.InitType.Normal, 0, 1), learning_rate=0.1, verbose=0)
        hetuCTR.seed(0)
        return t.debug_fetch(16)
    assert np.array_equal(first_rows(9), first_rows(9)) and not np.array_equal(first_rows(9), first_rows(10))
