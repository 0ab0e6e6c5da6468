"""The entry point that allocates nothing (hctr_preprocess_noalloc) against hctr_preprocess, through the C ABI:
two tables with the same configuration, one driven by each call, must agree bit for bit in every integer
intermediate, in the pulled rows and in the table state.  Two calls in a row, the second with a smaller batch."""
import numpy as np
import pytest
import torch

from hetuctr_amd import capi
from tests.helpers import zipf_sampler

pytestmark = pytest.mark.gpu

ITEMS = [capi.UNIQUE, capi.SORTED_ARG, capi.RUN_START, capi.IDX_MAP, capi.ROOT, capi.OFFSET, capi.SIZES, capi.KEYS]


def make(length, width):
    root = np.zeros(length, np.uint8)
    capi.seed(3)
    return capi.Table(0, 1, 0, "", 0, length, width, 0, 0, root, np.arange(length, dtype=np.int64),
                      ("Uniform", -0.01, 0.01), 0.05, 0)


@pytest.mark.parametrize("wide", [False, True])
def test_preprocess_noalloc_matches_preprocess(wide, monkeypatch):
    if wide:
        monkeypatch.setenv("HETUCTR_FORCE_WIDE_KEYS", "1")     # 64-bit sort keys: the larger scratch layout
    print("no-alloc preprocess, wide keys:", wide, flush=True)
    rng = np.random.default_rng(41)
    length, width = 300_000, 32
    a, b = make(length, width), make(length, width)
    draw = zipf_sampler(length, 1.1, rng)
    n_max = 200_000
    warm = [torch.from_numpy(draw(n_max)).cuda() for _ in range(2)]
    dst_a = torch.empty((n_max, width), device="cuda")
    dst_b = torch.empty((n_max, width), device="cuda")
    torch.cuda.synchronize()
    for t, dst in ((a, dst_a), (b, dst_b)):                    # two ordinary calls size both batch buffers
        for k in warm:
            t.preprocess(k.data_ptr(), n_max)
        t.push_pull(0, dst.data_ptr())
    prev_n = 0
    for step, n in enumerate((n_max, 70_001, 150_000, 0, 4096)):   # the second call is smaller than the first
        keys = torch.from_numpy(draw(n)).cuda() if n else torch.zeros(1, dtype=torch.int64, device="cuda")
        grad = torch.from_numpy(rng.normal(0, 1e-3, size=(max(prev_n, 1), width)).astype(np.float32)).cuda()
        torch.cuda.synchronize()
        a.preprocess(keys.data_ptr(), n)
        free_before = torch.cuda.mem_get_info()[0]             # hipMemGetInfo: bytes free on the device
        b.preprocess_noalloc(keys.data_ptr(), n)
        assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed at step %d" % step
        for it in ITEMS:
            x, y = a.fetch(it), b.fetch(it)
            assert x.shape == y.shape and np.array_equal(x, y), "item %d differs at step %d" % (it, step)
        gp = grad.data_ptr() if prev_n else 0
        a.push_pull(gp, dst_a.data_ptr())
        b.push_pull(gp, dst_b.data_ptr())
        assert torch.equal(dst_a[:n], dst_b[:n]), "pulled rows differ at step %d" % step
        prev_n = n
    assert np.array_equal(a.fetch(capi.EMBEDDING), b.fetch(capi.EMBEDDING))
    assert np.array_equal(a.fetch(capi.VERSION), b.fetch(capi.VERSION))
    # refusals: too many keys, host ids, buffers that would have to grow
    big = torch.zeros(capi.NOALLOC_MAX_KEYS + 1, dtype=torch.int64, device="cuda")
    with pytest.raises(RuntimeError, match="at most"):
        b.preprocess_noalloc(big.data_ptr(), capi.NOALLOC_MAX_KEYS + 1)
    host = np.zeros(16, np.int64)
    with pytest.raises(RuntimeError, match="device memory"):
        b.preprocess_noalloc(host.ctypes.data, 16)
    with pytest.raises(RuntimeError, match="batch buffers"):
        b.preprocess_noalloc(big.data_ptr(), n_max + 50_000)
    k = torch.from_numpy(draw(1000)).cuda()                    # and the table goes on after a refusal
    torch.cuda.synchronize()
    a.preprocess(k.data_ptr(), 1000)
    b.preprocess_noalloc(k.data_ptr(), 1000)
    assert np.array_equal(a.fetch(capi.SORTED_ARG), b.fetch(capi.SORTED_ARG))
    a.close()
    b.close()
