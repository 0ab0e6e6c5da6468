"""Shared helpers of the test-suite: definitional (numpy) restatements used to pin the oracle, and
seeded workload generators."""
import numpy as np


def np_preprocess(keys, root_arr, nrank):
    """What csrc/core/preprocess.cu:92-141 must produce, from the definitions of its primitives:
    stable radix sort by (owner, id) == lexsort with position as last tie-break; run-length encode ==
    np.unique on the composite key; exclusive scan == first index; inverse == searchsorted."""
    keys = np.asarray(keys, dtype=np.int64)
    n = keys.shape[0]
    owner = root_arr[keys].astype(np.int64) if n else np.zeros(0, np.int64)
    sorted_arg = np.lexsort((np.arange(n), keys, owner)).astype(np.int64)
    comp = owner * np.int64(root_arr.shape[0]) + keys
    ucomp, first, inverse, counts = np.unique(comp, return_index=True, return_inverse=True, return_counts=True)
    unique = keys[first] if n else np.zeros(0, np.int64)
    run_start = np.concatenate([np.zeros(1, np.int64), np.cumsum(counts)]).astype(np.int64)
    uroot = root_arr[unique].astype(np.int64) if n else np.zeros(0, np.int64)
    send_cnt = np.bincount(uroot, minlength=nrank).astype(np.int64)
    return dict(sorted_arg=sorted_arg, unique=unique, run_start=run_start, idx_map=inverse.astype(np.int64).reshape(-1),
                root=uroot, send_cnt=send_cnt)


def brute_preprocess(keys, root_arr):
    """O(N^2) pure-python version for tiny inputs."""
    n = len(keys)
    comp = [(int(root_arr[k]), int(k)) for k in keys]
    order = sorted(range(n), key=lambda i: (comp[i], i))
    uniq = []
    run_start = []
    for j, i in enumerate(order):
        if j == 0 or comp[i] != comp[order[j - 1]]:
            uniq.append(comp[i])
            run_start.append(j)
    run_start.append(n)
    idx_map = [uniq.index(c) for c in comp]
    return order, [u[1] for u in uniq], run_start, idx_map


def np_offsets(root_arr, storage_arr, rank):
    """csrc/core/table_initialize.cu:76-91: ids owned by other ranks first (order kept), then own ids."""
    st = np.asarray(storage_arr, dtype=np.int64)
    cached = st[root_arr[st] != rank]
    owned = st[root_arr[st] == rank]
    ids = np.concatenate([cached, owned])
    slot = np.full(root_arr.shape[0], -1, dtype=np.int64)
    slot[ids] = np.arange(ids.shape[0])
    return ids, slot, cached.shape[0]


def zipf_sampler(card, alpha, rng):
    """Returns f(n) drawing n local ids in [0, card) with P(rank k) ~ 1/(k+1)^alpha; rank == id."""
    w = 1.0 / np.power(np.arange(1, card + 1, dtype=np.float64), alpha)
    cdf = np.cumsum(w)
    cdf /= cdf[-1]

    def draw(n):
        return np.minimum(np.searchsorted(cdf, rng.random(n), side="left"), card - 1).astype(np.int64)

    return draw


def ctr_fields(total_rows, nfields, seed, lo=1.0, hi=7.0):
    """Seeded log-uniform field cardinalities 10^U(lo,hi), rescaled so that they sum to ~total_rows."""
    rng = np.random.default_rng(seed)
    c = np.power(10.0, rng.uniform(lo, hi, nfields))
    c = np.maximum(10, np.round(c * (total_rows / c.sum()))).astype(np.int64)
    # clip the big ones again after rescaling small ones up to 10
    c[np.argmax(c)] += total_rows - c.sum()
    return c
