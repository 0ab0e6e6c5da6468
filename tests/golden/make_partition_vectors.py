"""Writes tests/golden/partition_cases.npz: inputs and outputs of the reference's offline partitioner on small cases.

The outputs come from the reference's own C++ sources (csrc/partition/partition.cc, pybind.cc) compiled in place
WITHOUT OpenMP by `make -C oracle ref_partition` into oracle/_ref/partition_serial (a build output that is never
committed).  Run where that build exists:

    python tests/golden/make_partition_vectors.py

Every sample holds one id per slot from the slot's own id range, so no embedding occurs n_data times (where the
reference would read past its soft-count table).  Per case the file keeps the input (data, comm_mat, n_part, batch),
and after the construction and after each of `rounds` rounds of refine_data + refine_embed: both assignments, both
size vectors, the communication matrix and the priorities.
"""
import ctypes
import importlib.util
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
# (samples, slots, ids per slot, zipf exponent, parts, batch, rounds)
CASES = [(500, 3, 17, 1.3, 3, 16, 3), (2000, 6, 80, 1.3, 4, 64, 3), (3000, 5, 800, 1.2, 8, 128, 2),
         (1500, 26, 40, 1.5, 8, 256, 2), (900, 4, 300, 1.1, 2, 32, 2)]


def slot_data(rng, nd, ns, card, a):
    cols = [np.minimum(rng.zipf(a, size=nd) - 1, card - 1) + f * card for f in range(ns)]
    return np.stack(cols, 1).astype(np.int32)


def load_reference():
    d = os.path.join(ROOT, "oracle", "_ref", "partition_serial")
    so = [f for f in os.listdir(d) if f.startswith("hetuCTR_partition")][0]
    spec = importlib.util.spec_from_file_location("hetuCTR_partition", os.path.join(d, so))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def snapshot(out, key, p):
    d, e = p.get_result()
    out[key + "_res_data"], out[key + "_res_embed"] = d.copy(), e.copy()
    out[key + "_cnt_data"], out[key + "_cnt_embed"] = p.get_data_cnt().copy(), p.get_embed_cnt().copy()
    out[key + "_comm"], out[key + "_priority"] = p.get_communication().copy(), p.get_priority().copy()


def main():
    ref = load_reference()
    libc = ctypes.CDLL(None)
    rng = np.random.default_rng(2024)
    out = {"n_cases": np.int64(len(CASES))}
    for c, (nd, ns, card, a, P, B, rounds) in enumerate(CASES):
        data = slot_data(rng, nd, ns, card, a)
        assert np.bincount(data.ravel()).max() < nd
        mat = rng.random((P, P)).astype(np.float32)
        np.fill_diagonal(mat, 0)
        libc.srand(1)                                   # a fresh process' rand() state
        p = ref.partition(data, mat, P, B)
        k = "c%d" % c
        out[k + "_data"], out[k + "_mat"] = data, mat
        out[k + "_cfg"] = np.array([P, B, rounds], np.int64)
        snapshot(out, k + "_r0", p)
        for r in range(rounds):
            p.refine_data()
            p.refine_embed()
            snapshot(out, k + "_r%d" % (r + 1), p)
    np.savez_compressed(os.path.join(HERE, "partition_cases.npz"), **out)
    print("wrote partition_cases.npz:", len(CASES), "cases")


if __name__ == "__main__":
    main()
