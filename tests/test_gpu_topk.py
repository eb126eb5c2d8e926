"""GPU parity of the sort / top-k / priority-update path through the C ABI vs the CPU oracle."""
import numpy as np
import pytest

from conftest import announce

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _check_topk(oracle, ops, w, k, label):
    announce("topk %s n=%d k=%d" % (label, len(w), k))
    dw = _dev(w)
    vals, idx = ops.topk(dw, k, sorted_by_value=True)
    uvals, uidx = ops.topk(dw, k, sorted_by_value=False)
    torch.cuda.synchronize()
    evals, eidx = oracle.topk_f32(w, k, True)
    assert np.array_equal(idx.cpu().numpy(), eidx)
    assert np.array_equal(vals.cpu().numpy().view(np.uint32), evals.view(np.uint32))
    _, euidx = oracle.topk_f32(w, k, False)
    assert np.array_equal(uidx.cpu().numpy(), euidx)
    assert np.array_equal(uvals.cpu().numpy().view(np.uint32), w[euidx].view(np.uint32))
    # independent statement: stable descending argsort
    ref = np.argsort(-w.astype(np.float64), kind="stable")[:k]
    assert np.array_equal(eidx, ref)


def test_topk_cases(oracle):
    from gear_amd import ops
    rng = np.random.default_rng(31)
    ln = lambda n: (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    _check_topk(oracle, ops, ln(1000), 1, "lognormal")
    _check_topk(oracle, ops, ln(1000), 1000, "k == n")
    _check_topk(oracle, ops, ln(5000), 4999, "k == n-1")
    _check_topk(oracle, ops, ln(4097), 33, "tile + 1")
    _check_topk(oracle, ops, np.full(10000, 2.5, np.float32), 777, "all equal")
    _check_topk(oracle, ops, rng.integers(0, 4, size=100_000).astype(np.float32), 30_000,
                "four distinct values")
    _check_topk(oracle, ops, rng.integers(0, 1000, size=1_000_000).astype(np.float32), 65_536,
                "many ties at the threshold")
    special = ln(20_000)
    special[:6] = [0.0, np.inf, np.float32(1e-45), np.float32(1e-40), 3.4e38, 0.0]
    _check_topk(oracle, ops, special, 19_998, "zeros / inf / denormals")
    mixed = rng.normal(size=50_000).astype(np.float32)  # negative values order correctly too
    _check_topk(oracle, ops, mixed, 12_345, "signed")
    # clustered maxima: every selected entry sits in a few waves, whose candidate lists overflow,
    # so the write launch takes its re-reading path; ascending, descending, and one hot block
    _check_topk(oracle, ops, np.sort(ln(300_000)), 5_000, "ascending (lists overflow)")
    _check_topk(oracle, ops, np.sort(ln(300_000))[::-1].copy(), 5_000, "descending (lists overflow)")
    hot = ln(2_000_000)
    hot[777_000:780_000] += 1000.0
    _check_topk(oracle, ops, hot, 2_500, "one hot stretch (lists overflow)")
    _check_topk(oracle, ops, ln(2_000_000), 2_500, "same size, spread out (lists)")


def test_topk_without_the_sampled_hint(oracle):
    """GEAR_HIP_TOPK_HINT=0 (read at every call): uniform level-0 bins, no candidate lists for
    long inputs -- every level streams the priorities.  Same results."""
    import os
    from gear_amd import ops
    rng = np.random.default_rng(32)
    ln = lambda n: (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    old = os.environ.get("GEAR_HIP_TOPK_HINT")
    os.environ["GEAR_HIP_TOPK_HINT"] = "0"
    try:
        _check_topk(oracle, ops, ln(3_000_000), 65_536, "no hint, lognormal")
        _check_topk(oracle, ops, ln(3_000_000), 1, "no hint, k = 1")
        _check_topk(oracle, ops, rng.integers(0, 50, size=2_000_000).astype(np.float32), 100_000,
                    "no hint, ties")
        _check_topk(oracle, ops, rng.normal(size=1_500_000).astype(np.float32), 140_000,
                    "no hint, signed, radix-sorted output")
    finally:
        if old is None:
            os.environ.pop("GEAR_HIP_TOPK_HINT", None)
        else:
            os.environ["GEAR_HIP_TOPK_HINT"] = old


def test_topk_infinite_priorities(oracle):
    """The k-th largest priority is +inf (at least k of them), or the selection reaches down to
    -inf (k == n): the bins of the infinities border on keys that decode to NaN."""
    from gear_amd import ops
    rng = np.random.default_rng(61)
    w = (rng.lognormal(0, 1, size=200_000) ** 0.6).astype(np.float32)
    w[rng.permutation(200_000)[:5_000]] = np.inf
    _check_topk(oracle, ops, w, 3_000, "k-th largest is +inf")
    _check_topk(oracle, ops, w, 5_000, "exactly k +inf")
    _check_topk(oracle, ops, w, 5_001, "one below the +inf")
    v = rng.normal(size=70_000).astype(np.float32)
    v[rng.permutation(70_000)[:900]] = -np.inf
    v[rng.permutation(70_000)[:50]] = np.inf
    _check_topk(oracle, ops, v, 70_000, "k == n with -inf")
    _check_topk(oracle, ops, v, 69_500, "threshold is -inf")
    _check_topk(oracle, ops, np.full(5_000, -np.inf, np.float32), 100, "all -inf")
    _check_topk(oracle, ops, np.full(5_000, np.inf, np.float32), 4_999, "all +inf")


def test_topk_nan_priorities_stay_inside_the_outputs():
    """NaN is not a valid priority and the selection is then unspecified, but nothing may be
    written outside values_out[0:k) / indices_out[0:k)."""
    from gear_amd import _cabi
    import ctypes
    lib = _cabi.load()
    rng = np.random.default_rng(62)
    n = 300_000
    for frac, k in ((0.001, 4_096), (0.5, 4_096), (1.0, 4_096), (0.5, 20_000), (1.0, 20_000)):
        w = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
        nan = rng.random(n) < frac
        w[nan] = np.nan
        # NaNs of either sign next to infinities: a bin map laid out around NaN samples may take
        # the infinities for candidates whose bins lie below the bound's
        bits = w.view(np.uint32)
        bits[nan & (rng.random(n) < 0.5)] |= np.uint32(0x80000000)
        w[rng.permutation(n)[:2_000]] = np.inf
        w[rng.permutation(n)[:1_000]] = -np.inf
        dw = _dev(w)
        for by_value in (0, 1):
            vals = torch.full((k + 1024,), -7.0, dtype=torch.float32, device="cuda")
            idx = torch.full((k + 1024,), -7, dtype=torch.int64, device="cuda")
            ws = torch.empty(lib.gear_hip_topk_workspace_bytes(n, k), dtype=torch.uint8,
                             device="cuda")
            announce("topk with NaN fraction %g by_value=%d" % (frac, by_value))
            rc = lib.gear_hip_topk_f32(ctypes.c_void_p(dw.data_ptr()), n, k, by_value,
                                       ctypes.c_void_p(vals.data_ptr()),
                                       ctypes.c_void_p(idx.data_ptr()),
                                       ctypes.c_void_p(ws.data_ptr()), ws.numel(), None)
            assert rc == 0
            torch.cuda.synchronize()
            assert bool((vals[k:] == -7.0).all()) and bool((idx[k:] == -7).all())


def test_topk_value_order_paths(oracle):
    """Value order: large groups of equal priorities above the threshold (the segment sort goes
    down to the index bits), both sides of the k at which the radix sort takes over, and both
    sides of the input size from which a sample is drawn."""
    from gear_amd import ops
    rng = np.random.default_rng(81)
    ln = lambda n: (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    ties = ln(2_000_000)
    ties[rng.permutation(2_000_000)[:60_000]] = 100.0
    _check_topk(oracle, ops, ties, 65_536, "60 000 equal priorities above the threshold")
    _check_topk(oracle, ops, ties, 50_000, "threshold inside the equal priorities")
    three = rng.integers(0, 3, size=1_500_000).astype(np.float32)
    _check_topk(oracle, ops, three, 131_072, "three distinct values, k = 131072")
    big = ln(3_000_000)
    _check_topk(oracle, ops, big, 131_072, "largest k of the segment sort")
    _check_topk(oracle, ops, big, 131_073, "smallest k of the radix sort")
    _check_topk(oracle, ops, ln(262_144), 1_000, "smallest input with a sample")
    _check_topk(oracle, ops, ln(262_143), 1_000, "largest input without a sample")
    _check_topk(oracle, ops, ln(30_000_000), 65_536, "long input")
    # ~220 candidates per wave: the queues are ordered by the same-step neighbours
    _check_topk(oracle, ops, ln(60_000_000), 65_536, "longer input, long candidate queues")
    wide = (rng.normal(size=1_000_000) * np.exp(rng.normal(size=1_000_000) * 8)).astype(np.float32)
    _check_topk(oracle, ops, wide, 40_000, "priorities over many orders of magnitude, both signs")
    # candidates from 1e-38 to 100: the stretch of keys between the hint and the largest sample
    # is more than a quarter of all keys, and no level-0 bin may be wider than the two levels
    # below it can resolve (the index-ordered selection asks for few, wide bins there)
    tiny = (rng.random(10_000_000) * 1e-38).astype(np.float32)
    tiny[9_000_000:9_014_000] += np.float32(100.0)
    _check_topk(oracle, ops, tiny, 59_000, "denormals and a stretch of 100.0")
    tiny[rng.permutation(10_000_000)[:30_000]] = rng.random(30_000, dtype=np.float32) * 1e30
    _check_topk(oracle, ops, tiny, 59_000, "denormals up to 1e30")


def test_topk_value_order_small_inputs_and_narrow_key_ranges(oracle):
    """The table that says where every bin starts in value order is built by the workgroups of
    the launch together, however few they are (small inputs), for every k around the numbers of
    segments; and a segment whose keys lie on both sides of a power of two (where nearly every
    key bit differs between neighbours) is sorted like any other."""
    from gear_amd import ops
    rng = np.random.default_rng(83)
    ln = lambda n: (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    for n in (300, 5_000, 70_000, 300_000, 1_100_000):
        w = ln(n)
        for k in (1, 2, 253, 254, 255, 256, 257, 511, 512, 513, n // 3, n):
            if k <= min(n, 131_072):
                _check_topk(oracle, ops, w, k, "n=%d k=%d" % (n, k))
    around_one = (1.0 + rng.normal(size=2_000_000) * 1e-4).astype(np.float32)
    _check_topk(oracle, ops, around_one, 65_536, "priorities around 1.0")
    _check_topk(oracle, ops, around_one, 1_000_000, "priorities around 1.0, half of them")
    around_zero = (rng.normal(size=1_000_000) * 1e-30).astype(np.float32)
    _check_topk(oracle, ops, around_zero, 100_000, "priorities around 0, both signs")


def test_topk_value_order_with_thousands_of_equal_priorities(oracle):
    """Fresh transitions enter a replay buffer at the maximum priority: thousands of equal
    priorities above the threshold.  In value order they form one segment that does not fit the
    sort's LDS buffers (more than 8192 entries): scattered over the array, as one hot stretch of
    consecutive entries, next to other keys in the same segment, and two such groups."""
    from gear_amd import ops
    rng = np.random.default_rng(83)
    n, k = 3_000_000, 65_536
    base = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    top = np.float32(base.max())
    w = base.copy()
    w[rng.permutation(n)[:30_000]] = top
    _check_topk(oracle, ops, w, k, "30000 scattered entries at the maximum")
    w = base.copy()
    w[1_000_000:1_040_000] = np.float32(10.0)
    _check_topk(oracle, ops, w, k, "a stretch of 40000 equal entries above the threshold")
    w = base.copy()
    w[rng.permutation(n)[:20_000]] = np.float32(10.0)
    w[2_000_000:2_012_000] = np.float32(10.000001)
    _check_topk(oracle, ops, w, k, "two long groups of neighbouring keys")
    w = base.copy()
    w[rng.permutation(n)[:100_000]] = top
    _check_topk(oracle, ops, w, 131_072, "100000 entries at the maximum, k = 131072")


def _sample_size(n, k):
    """How many priorities the selection samples: 2, 8 or 32 per thread of one 1024-thread
    workgroup -- the fewest with which the entries above the hint are expected to fit a wave's
    candidate list with six standard deviations to spare, with strides of at least 128 elements."""
    def cdiv(a, b):
        return -(-a // b)

    wave_len = cdiv(cdiv(n, 4096), 256) * 256            # 256 workgroups of 16 waves, 256-element steps
    waves = cdiv(n, wave_len * 16) * 16
    cap = min(max(cdiv(8 * cdiv(k, waves), 64) * 64, 256), 1024, wave_len, 512)

    def rank(per):
        mu = per * 1024 * k / n
        return mu + 6.0 * mu ** 0.5 + 8.0

    def lists_hold(per):
        e = 1.6 * rank(per) / (per * 1024) * wave_len
        return e + 6.0 * e ** 0.5 <= cap

    per = 2
    while per < 32 and not lists_hold(per):
        per *= 4
    while per > 2 and n < 128 * per * 1024:
        per //= 4
    return per * 1024


def _sampled_positions(n, samples=2048):
    """Where the selection looks for its sample: one position per stride, at a hashed offset."""
    stride = n // samples
    s = np.arange(samples, dtype=np.uint64)
    off = (((s * np.uint64(2654435761)) & np.uint64(0xffffffff)) * np.uint64(stride)) >> np.uint64(32)
    return (s * np.uint64(stride) + off).astype(np.int64)


def test_topk_with_a_misleading_sample(oracle):
    """The sample only decides how the work is done: when it overstates the priorities (too few
    candidates: the first read is done again on uniform bins) or understates them (every entry a
    candidate: the lists overflow and the levels stream), the result is the same."""
    from gear_amd import ops
    rng = np.random.default_rng(71)
    n = 2_000_000
    base = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    for k, what in ((65_536, "sample overstates (redo)"),
                    (1_000, "sample overstates, k below the sampled entries")):
        pos = _sampled_positions(n, _sample_size(n, k))
        high = base.copy()
        high[pos] = 1000.0 + rng.random(pos.size, dtype=np.float32)
        _check_topk(oracle, ops, high, k, what)
    low = base.copy()
    low[_sampled_positions(n, _sample_size(n, 65_536))] = 1e-6
    _check_topk(oracle, ops, low, 65_536, "sample understates (lists overflow)")
    neg = -base
    _check_topk(oracle, ops, neg, 30_000, "all negative")


def test_topk_small_inputs_with_a_sample(oracle):
    """Inputs of a few hundred thousand priorities: a wave's list is as long as its range (it
    cannot overflow), and the sample still decides which entries are listed -- up to k = n / 8."""
    from gear_amd import ops
    rng = np.random.default_rng(97)
    for n, k in ((262_144, 1), (300_000, 37_500), (600_000, 65_536), (1_000_000, 125_000),
                 (1_000_000, 125_001)):
        base = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
        _check_topk(oracle, ops, base, k, "lognormal")
        ties = base.copy()
        ties[rng.permutation(n)[:max(1, k - k // 8)]] = np.float32(base.max())
        _check_topk(oracle, ops, ties, k, "most of the selection at the maximum")
        hot = base.copy()
        hot[n // 3:n // 3 + max(1, k // 2)] += np.float32(50.0)
        _check_topk(oracle, ops, hot, k, "a hot stretch")
        if k > 1:
            high = base.copy()
            pos = _sampled_positions(n, _sample_size(n, k))
            high[pos] = 1000.0 + rng.random(pos.size, dtype=np.float32)
            _check_topk(oracle, ops, high, k, "sample overstates")
    _check_topk(oracle, ops, np.full(500_000, 1.5, np.float32), 50_000, "all equal")


def _check_state(oracle, state, w, k, by_value, label):
    announce("warm topk %s n=%d k=%d by_value=%d" % (label, len(w), k, by_value))
    vals, idx = state.select(_dev(w), k, sorted_by_value=by_value)
    torch.cuda.synchronize()
    evals, eidx = oracle.topk_f32(w, k, by_value)
    assert np.array_equal(idx.cpu().numpy(), eidx), label
    assert np.array_equal(vals.cpu().numpy().view(np.uint32), w[eidx].view(np.uint32)), label


@pytest.mark.parametrize("by_value", [True, False])
def test_topk_warm_calls_follow_a_changing_array(oracle, by_value):
    """The warm form starts from the bound the call before it left in the workspace.  The bound
    only decides how the work is done: on an array that changes a little between calls (the
    replay buffer's priority updates), on one whose priorities all shrank (the stale bound is
    too high: fewer than k entries above it), on one whose priorities all grew (too low: the
    lists overflow), and after a call of another shape, the result is the oracle's."""
    from gear_amd import ops
    rng = np.random.default_rng(91)
    n, k = 2_000_000, 65_536
    w = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    state = ops.TopKState()
    _check_state(oracle, state, w, k, by_value, "first call (a sample)")
    for step in range(3):
        pos = rng.permutation(n)[:20_000]
        w[pos] = (rng.lognormal(0, 1, size=pos.size) ** 0.6).astype(np.float32)
        _check_state(oracle, state, w, k, by_value, "after updates %d" % step)
    small = (w * np.float32(0.01)).astype(np.float32)
    _check_state(oracle, state, small, k, by_value, "all priorities shrank (bound too high)")
    _check_state(oracle, state, small, k, by_value, "the call after the failed bound")
    _check_state(oracle, state, small, k, by_value, "and the one after that")
    big = (w * np.float32(100.0)).astype(np.float32)
    _check_state(oracle, state, big, k, by_value, "all priorities grew (bound too low)")
    _check_state(oracle, state, big, k, by_value, "the call after the overflow")
    _check_state(oracle, state, big, k, by_value, "and the one after that")
    _check_state(oracle, state, w[:1_500_000].copy(), 30_000, by_value, "another shape")
    _check_state(oracle, state, w[:1_500_000].copy(), 30_000, by_value, "the same shape again")
    # a bound just above most of the array: few candidates, the k-th largest far below it
    spike = w.copy()
    spike[rng.permutation(n)[:200_000]] += np.float32(50.0)
    _check_state(oracle, state, spike, 150_000 if not by_value else 100_000, by_value,
                 "a fifth of a million entries lifted")
    plain = w.copy()
    _check_state(oracle, state, plain, 150_000 if not by_value else 100_000, by_value,
                 "and dropped again (bound too high by far)")


def test_topk_warm_on_a_workspace_that_holds_something_else(oracle):
    """A warm call on a workspace that no top-k call has used (zeros, ones, the prefix sums of an
    earlier tenant) finds no mark and draws its sample like the plain form."""
    from gear_amd import ops, _cabi
    lib = _cabi.load()
    rng = np.random.default_rng(92)
    n, k = 1_000_000, 10_000
    w = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    nbytes = lib.gear_hip_topk_workspace_bytes(n, k)
    evals, eidx = oracle.topk_f32(w, k, True)
    for fill in ("zeros", "ones", "ramp"):
        announce("warm topk on a workspace of %s" % fill)
        if fill == "zeros":
            ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        elif fill == "ones":
            ws = torch.full((nbytes,), 255, dtype=torch.uint8, device="cuda")
        else:
            ws = torch.arange(nbytes // 8 + 1, dtype=torch.int64, device="cuda").view(torch.uint8)[:nbytes].clone()
        vals, idx = ops.topk(_dev(w), k, sorted_by_value=True, warm=True, workspace=ws)
        torch.cuda.synchronize()
        assert np.array_equal(idx.cpu().numpy(), eidx)
        assert np.array_equal(vals.cpu().numpy().view(np.uint32), evals.view(np.uint32))


def test_topk_config5_size(oracle):
    """Config 5's maintenance step at full size: top-65 536 of 10 000 000 lognormal^0.6."""
    from gear_amd import ops
    rng = np.random.default_rng(1005)
    w = (rng.lognormal(0, 1, size=10_000_000) ** 0.6).astype(np.float32)
    _check_topk(oracle, ops, w, 65_536, "config5")


def test_sort_i64(oracle):
    from gear_amd import ops
    rng = np.random.default_rng(41)
    for n, bits in ((1, 1), (2, 8), (255, 9), (256, 20), (1025, 20), (2048, 24), (4096, 31),
                    (4097, 17), (5000, 64), (65_536, 40), (131_072, 33), (131_073, 16),
                    (300_001, 63)):
        keys = rng.integers(0, 1 << min(bits, 62), size=n).astype(np.int64)
        keys[rng.integers(0, n, size=max(n // 3, 1))] = keys[0]  # duplicates: stability matters
        vals = rng.integers(-2**62, 2**62, size=n).astype(np.int64)
        announce("sort n=%d bits=%d" % (n, bits))
        ko, vo = ops.sort_i64(_dev(keys), _dev(vals), key_bits=bits)
        k2 = ops.sort_i64(_dev(keys), key_bits=bits)
        torch.cuda.synchronize()
        ek, ev = oracle.sort_i64(keys, vals)
        assert np.array_equal(ko.cpu().numpy(), ek)
        assert np.array_equal(vo.cpu().numpy(), ev)
        assert np.array_equal(k2.cpu().numpy(), ek)
        order = np.argsort(keys, kind="stable")
        assert np.array_equal(ek, keys[order]) and np.array_equal(ev, vals[order])


def test_scatter_unique_and_duplicates(oracle):
    from gear_amd import ops
    rng = np.random.default_rng(51)
    n = 1_000_000
    w0 = rng.random(n, dtype=np.float32)
    # unique indices: a seeded permutation prefix
    idx = rng.permutation(n)[:65_536].astype(np.int64)
    v = rng.random(65_536, dtype=np.float32)
    for unique in (True, False):
        announce("scatter unique input, unique_indices=%s" % unique)
        dw = _dev(w0)
        ops.scatter(dw, _dev(idx), _dev(v), unique_indices=unique)
        torch.cuda.synchronize()
        exp = oracle.scatter_f32(w0.copy(), idx, v)
        ref = w0.copy()
        ref[idx] = v
        assert np.array_equal(exp, ref)
        assert np.array_equal(dw.cpu().numpy(), exp)
    # duplicates (each index about 8 times) + out-of-range entries: last write wins
    idx = rng.integers(0, 8192, size=65_536).astype(np.int64)
    idx[::1000] = -1
    idx[1::1000] = n + 5
    announce("scatter with duplicates")
    dw = _dev(w0)
    ops.scatter(dw, _dev(idx), _dev(v), unique_indices=False)
    torch.cuda.synchronize()
    exp = oracle.scatter_f32(w0.copy(), idx, v)
    ref = w0.copy()
    for j in range(len(idx)):          # brute-force "last wins"
        if 0 <= idx[j] < n:
            ref[idx[j]] = v[j]
    assert np.array_equal(exp, ref)
    assert np.array_equal(dw.cpu().numpy(), exp)
