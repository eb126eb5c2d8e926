"""Writes the small fixtures of tests/golden/ (run once; the outputs are committed).

Nothing here touches the oracle or the HIP library: expected outputs come from plain numpy
slicing / sorting / searching, or are written out by hand from the inputs that the reference's own
tests use (tests/test_sub.py, tests/test_table.py, tests/test_copy.py of bigrl-team/gear).
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from helpers import Schema, fill_random, numpy_window_gather  # noqa: E402


def reference_test_vectors():
    """Hand-derived from the inputs of the reference's tests.

    tests/test_sub.py:10-28: one column fp32[1,2,3,4] (96 B/step), T=100, capacity 32,
    SubscribePattern(-1, 100, head), indices = timesteps = 0..9, lengths = 10.
    handler.cc:107-121 then gives start=max(i-1,0), end=10, copy_len=(10-start)*96,
    src_off=i*9600+start*96, dst_off=i*9600+9600-copy_len, return value 9600.
    tests/test_table.py:15-24: T=100, capacity 1000, fp32[3,32] + int32[1]:
    step bytes 384 and 4, trajectory stride 38 800, table 38 800 000 bytes.
    """
    return {
        "test_sub": {
            "step_bytes": 96, "trajectory_length": 100, "capacity": 32, "traj_stride": 9600,
            "offset": -1, "length": 100, "pad": "head",
            "indices": list(range(10)), "timesteps": list(range(10)), "lengths": [10] * 10,
            "expected_return": 9600,
            "copy_lens": [960, 960, 864, 768, 672, 576, 480, 384, 288, 192],
            "src_offsets": [0, 9600, 19296, 28992, 38688, 48384, 58080, 67776, 77472, 87168],
            "dst_offsets": [8640, 18240, 27936, 37632, 47328, 57024, 66720, 76416, 86112, 95808],
        },
        "test_table": {
            "trajectory_length": 100, "capacity": 1000,
            "columns": [{"shape": [3, 32], "dtype": "float32"}, {"shape": [1], "dtype": "int32"}],
            "step_bytes": [384, 4], "accu": [0, 384, 388], "traj_stride": 38800,
            "table_bytes": 38800000,
        },
        "dtype_sizes": {"bool": 1, "uint8": 1, "int8": 1, "int16": 2, "int32": 4, "int64": 8,
                        "float32": 4, "float64": 8},
    }


def gather_fixture():
    """A 4-column table (odd byte sizes included) and three window batches."""
    cols = [("obs", "float32", (17,)), ("act", "int16", (3,)), ("rew", "float32", ()),
            ("done", "uint8", ())]
    schema = Schema(cols, T=12, capacity=9)
    table = fill_random(schema, 20240)
    rng = np.random.default_rng(20241)
    B = 40
    idxs = rng.integers(0, 9, size=B).astype(np.int64)
    lens = rng.integers(0, 13, size=B).astype(np.int64)
    tss = rng.integers(0, 14, size=B).astype(np.int64)
    out = {"table": table, "idxs": idxs, "tss": tss, "lens": lens,
           "step_bytes": np.array(schema.step_bytes, np.int64),
           "T": np.int64(12), "capacity": np.int64(9)}
    cases = [(-3, 5, True), (0, 4, False), (-20, 6, True), (2, 7, False)]
    out["cases"] = np.array([[o, s, int(p)] for o, s, p in cases], np.int64)
    for ci, (ofst, span, pad_head) in enumerate(cases):
        for c in range(4):
            dst, mask = numpy_window_gather(schema, table, c, idxs, tss, lens, ofst, span, pad_head)
            out["dst_%d_%d" % (ci, c)] = dst
            out["mask_%d_%d" % (ci, c)] = mask
    return out


def sampler_fixture():
    rng = np.random.default_rng(20242)
    n = 5000
    p = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    p[rng.integers(0, n, size=50)] = 0.0
    prefix = np.cumsum(p.astype(np.float64))          # sequential fp64 accumulation
    u = (rng.random(300) * prefix[-1]).astype(np.float32)
    idx = np.minimum(np.searchsorted(prefix, u.astype(np.float64), side="right"), n - 1)
    total = float(prefix[-1])
    w = np.array([(n * float(p[i]) / total) ** -0.4 for i in idx])
    w = (w / w.max()).astype(np.float32)
    pint = rng.integers(0, 50, size=3000).astype(np.float32)
    k = 137
    order = np.argsort(-p.astype(np.float64), kind="stable")[:k]
    ties = rng.integers(0, 7, size=4000).astype(np.float32)
    tie_order = np.argsort(-ties.astype(np.float64), kind="stable")[:1500]
    keys = rng.integers(0, 1 << 20, size=777).astype(np.int64)
    keys[100:200] = keys[5]
    vals = rng.integers(-1000, 1000, size=777).astype(np.int64)
    so = np.argsort(keys, kind="stable")
    w0 = rng.random(1000).astype(np.float32)
    sidx = rng.integers(-2, 1003, size=400).astype(np.int64)
    sval = rng.random(400).astype(np.float32)
    w1 = w0.copy()
    for j in range(len(sidx)):
        if 0 <= sidx[j] < len(w1):
            w1[sidx[j]] = sval[j]
    return {"p": p, "prefix": prefix, "u": u, "idx": idx.astype(np.int64), "is_weights": w,
            "pint": pint, "pint_prefix": np.cumsum(pint.astype(np.float64)),
            "topk_k": np.int64(k), "topk_idx": order.astype(np.int64), "topk_val": p[order],
            "ties": ties, "ties_idx": tie_order.astype(np.int64),
            "sort_keys": keys, "sort_vals": vals, "sorted_keys": keys[so], "sorted_vals": vals[so],
            "scatter_w0": w0, "scatter_idx": sidx, "scatter_val": sval, "scatter_w1": w1}


if __name__ == "__main__":
    with open(os.path.join(HERE, "reference_tests.json"), "w") as f:
        json.dump(reference_test_vectors(), f, indent=1)
    np.savez_compressed(os.path.join(HERE, "gather_small.npz"), **gather_fixture())
    np.savez_compressed(os.path.join(HERE, "sampler_small.npz"), **sampler_fixture())
    print("fixtures written to", HERE)
