"""The click-log loader: the host path against the reference driver's own numpy expression on a fixed log, the file
round trip, and (on the GPU) the device gather against the host path."""
import numpy as np
import pytest

from hetuctr_amd.loader import SparseFeatureLog


def small_log():
    rng = np.random.RandomState(3)
    return SparseFeatureLog(rng.randint(0, 1000, size=(500, 26)).astype(np.int32))


def test_host_sampling_shape_and_draws(tmp_path):
    log = small_log()
    assert log.data.dtype == np.int64 and (log.samples, log.fields) == (500, 26)
    keys = log.sample(64, np.random.RandomState(0))
    assert keys.dtype == np.int64 and keys.shape == (64 * 26,)
    # the rows are the ones numpy's randint names, in order, each sample's fields together
    idx = np.random.RandomState(0).randint(500, size=64)
    for b in (0, 17, 63):
        assert np.array_equal(keys[b * 26:(b + 1) * 26], log.data[idx[b]])
    path = str(tmp_path / "feats.npy")
    log.save(path)
    again = SparseFeatureLog.load(path)
    assert np.array_equal(again.data, log.data)
    with pytest.raises(ValueError):
        SparseFeatureLog(np.zeros(5))


def test_synthetic_log_covers_the_workload():
    log = SparseFeatureLog.synthetic("cfg2", samples=2000, seed=1, scale=0.01)
    assert log.fields == 26 and log.samples == 2000
    assert log.data.min() >= 0 and log.data.max() < log.rows
    # a field's ids stay inside that field's own range of the table: column f lies below column f + 1
    lo, hi = log.data.min(axis=0), log.data.max(axis=0)
    assert np.all(hi[:-1] < lo[1:])


@pytest.mark.gpu
def test_device_sampling_matches_host():
    import torch
    from hetuctr_amd import capi
    log = small_log()
    dev = log.cuda()
    for bs in (1, 64, 1000):
        want = log.sample(bs, np.random.RandomState(bs))
        got = dev.sample(bs, np.random.RandomState(bs))
        assert np.array_equal(got.cpu().numpy(), want)
    rows = torch.tensor([0, 499, 7], dtype=torch.int64, device="cuda")
    assert np.array_equal(dev.sample(0, rows=rows).cpu().numpy(), log.data[[0, 499, 7]].flatten())
    bad = torch.tensor([3, 500], dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="outside"):
        dev.sample(0, rows=bad)
    # and the keys go straight into a table
    t = capi.Table(0, 1, 0, "", 0, 1000, 8, 0, 0, np.zeros(1000, np.uint8), np.arange(1000), ("Uniform", -1, 1), 0.1)
    keys = dev.sample(32, np.random.RandomState(5))
    dst = torch.empty((32 * 26, 8), device="cuda")
    torch.cuda.synchronize()
    t.preprocess(keys.data_ptr(), keys.numel())
    t.push_pull(0, dst.data_ptr())
    emb = t.fetch(capi.EMBEDDING).reshape(1000, 8)
    assert np.array_equal(dst.cpu().numpy(), emb[keys.cpu().numpy()])
    t.close()
