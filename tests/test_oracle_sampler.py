"""CPU tests: the oracle's scan / search / importance weights / top-k / sort / scatter against
numpy, Python floats, brute force and the committed fixtures."""
import math
import os

import numpy as np
import pytest
from hypothesis import given, settings
from hypothesis import strategies as st

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def fx():
    return np.load(os.path.join(GOLD, "sampler_small.npz"))


def test_scan_fixture_and_closed_forms(oracle, fx):
    assert np.array_equal(oracle.scan_f32_f64(fx["p"]), fx["prefix"])
    assert np.array_equal(oracle.scan_f32_f64(fx["pint"]), fx["pint_prefix"])
    n = 100_000
    assert np.array_equal(oracle.scan_f32_f64(np.ones(n, np.float32)), np.arange(1, n + 1, dtype=np.float64))
    k = np.arange(1, 2001, dtype=np.float32)          # 1 + 2 + ... + k = k(k+1)/2
    assert np.array_equal(oracle.scan_f32_f64(k), (np.arange(1, 2001.0) * np.arange(2, 2002.0)) / 2)
    assert oracle.scan_f32_f64(np.zeros(0, np.float32)).size == 0
    w = np.random.default_rng(1).integers(0, 1000, size=5000)
    assert np.array_equal(oracle.scan_i64(w), np.cumsum(w))


def test_sum(oracle, fx):
    assert abs(oracle.sum_f32(fx["p"]) - math.fsum(float(x) for x in fx["p"])) <= 1e-9
    assert oracle.sum_f32(np.zeros(0, np.float32)) == 0.0


def test_search_fixture_and_brute_force(oracle, fx):
    assert np.array_equal(oracle.upper_bound_f64(fx["prefix"], fx["u"]), fx["idx"])
    # zero-priority entries are never drawn (draws are < total)
    assert np.all(fx["p"][fx["idx"]] > 0)
    rng = np.random.default_rng(2)
    for n in (1, 2, 5, 64):
        p = rng.integers(0, 3, size=n).astype(np.float64)
        p[0] = 1
        P = np.cumsum(p)
        u = np.concatenate([P, P - 0.5, [0.0, 1e9], rng.random(40) * P[-1]]).clip(0).astype(np.float32)
        got = oracle.upper_bound_f64(P, u)
        brute = [min(sum(1 for i in range(n) if P[i] <= float(t)), n - 1) for t in u]
        assert list(got) == brute
    u01 = rng.random(100, dtype=np.float32)
    t = u01.astype(np.float64) * fx["prefix"][-1]
    want = np.minimum(np.searchsorted(fx["prefix"], t, "right"), len(fx["prefix"]) - 1)
    assert np.array_equal(oracle.upper_bound_f64(fx["prefix"], u01, unit_uniforms=True), want)


def test_search_i64(oracle):
    rng = np.random.default_rng(4)
    lens = rng.integers(200, 1001, size=1000)
    P = np.cumsum(lens)
    t = rng.integers(0, P[-1], size=500)
    assert np.array_equal(oracle.upper_bound_i64(P, t), np.searchsorted(P, t, "right"))
    # every step of every trajectory maps to its trajectory
    P2 = np.cumsum([3, 1, 4])
    assert list(oracle.upper_bound_i64(P2, np.arange(8))) == [0, 0, 0, 1, 2, 2, 2, 2]
    u = rng.random(200)
    want = np.minimum(np.searchsorted(P, np.floor(u * float(P[-1])).astype(np.int64), "right"), 999)
    assert np.array_equal(oracle.upper_bound_i64(P, u, unit_uniforms=True), want)


def test_importance_weights(oracle, fx):
    got = oracle.is_weights(fx["p"], float(fx["prefix"][-1]), fx["idx"], 0.4)
    assert np.array_equal(got, fx["is_weights"])
    assert got.max() == 1.0 and got.min() > 0
    # uniform priorities: every weight is 1
    p = np.full(100, 0.25, np.float32)
    assert np.all(oracle.is_weights(p, 25.0, np.arange(10), 0.4) == 1.0)


def test_topk_fixture_and_special_cases(oracle, fx):
    vals, idx = oracle.topk_f32(fx["p"], int(fx["topk_k"]), True)
    assert np.array_equal(idx, fx["topk_idx"]) and np.array_equal(vals, fx["topk_val"])
    _, idx = oracle.topk_f32(fx["ties"], 1500, True)
    assert np.array_equal(idx, fx["ties_idx"])
    _, uidx = oracle.topk_f32(fx["ties"], 1500, False)
    assert np.array_equal(uidx, np.sort(fx["ties_idx"]))
    same = np.full(50, 3.0, np.float32)                 # all equal: the first k indices
    assert list(oracle.topk_f32(same, 7, True)[1]) == list(range(7))
    distinct = np.arange(100, dtype=np.float32)         # all distinct: the last k, descending
    assert list(oracle.topk_f32(distinct, 5, True)[1]) == [99, 98, 97, 96, 95]
    sp = np.array([0.0, np.inf, 1e-45, -0.0, 2.0, 1e-45], np.float32)
    assert list(oracle.topk_f32(sp, 6, True)[1]) == [1, 4, 2, 5, 0, 3]


@settings(max_examples=60, deadline=None)
@given(st.lists(st.integers(0, 6), min_size=1, max_size=200), st.data())
def test_topk_property(w, data):
    from oracle import oracle as orc
    w = np.array(w, np.float32)
    k = data.draw(st.integers(1, len(w)))
    _, idx = orc.topk_f32(w, k, True)
    assert np.array_equal(idx, np.argsort(-w.astype(np.float64), kind="stable")[:k])


def test_sort_fixture(oracle, fx):
    ko, vo = oracle.sort_i64(fx["sort_keys"], fx["sort_vals"])
    assert np.array_equal(ko, fx["sorted_keys"]) and np.array_equal(vo, fx["sorted_vals"])


def test_scatter_last_wins(oracle, fx):
    got = oracle.scatter_f32(fx["scatter_w0"].copy(), fx["scatter_idx"], fx["scatter_val"])
    assert np.array_equal(got, fx["scatter_w1"])
    w = np.zeros(4, np.float32)
    oracle.scatter_f32(w, [1, 1, 3, 1, 9, -1], np.array([1, 2, 3, 4, 5, 6], np.float32))
    assert list(w) == [0, 4, 0, 3]


@pytest.mark.parametrize("threads", [2, 3, 8])
def test_multithreaded_baselines_equal_the_sequential_oracle(oracle, threads):
    """The all-cores legs of the CPU baseline (chunked scan, per-chunk top-k + merge, draws split
    over threads) against the single-threaded functions they stand beside."""
    rng = np.random.default_rng(threads)
    ints = rng.integers(0, 1000, size=100_003).astype(np.float32)
    assert np.array_equal(oracle.scan_f32_f64(ints, threads=threads), np.cumsum(ints.astype(np.float64)))
    p = (rng.lognormal(0, 1, size=100_003) ** 0.6).astype(np.float32)
    seq = oracle.scan_f32_f64(p)
    par = oracle.scan_f32_f64(p, threads=threads)
    assert np.max(np.abs(par - seq) / seq) <= 1e-13
    u = rng.random(1000, dtype=np.float32)
    assert np.array_equal(oracle.upper_bound_f64(seq, u, True, threads=threads),
                          oracle.upper_bound_f64(seq, u, True))
    w = rng.integers(0, 50, size=50_001).astype(np.float32)        # many ties
    for k in (1, 777, 50_001):
        for by_value in (True, False):
            a = oracle.topk_f32(w, k, by_value)
            b = oracle.topk_f32(w, k, by_value, threads=threads)
            assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    assert np.array_equal(oracle.topk_f32(w, 777, True, threads=threads)[1],
                          np.argsort(-w.astype(np.float64), kind="stable")[:777])
