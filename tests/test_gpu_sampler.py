"""GPU parity of the weighted sampler: fp64 prefix sum (the chained, two-launch and three-launch
forms of the range scan), batched upper_bound
search, importance weights, through the C ABI against the CPU oracle."""
import os

import numpy as np
import pytest

from conftest import announce

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

# small sizes, then the sizes at which the range geometry, the staggered start, the streaming
# loads and the variant change (524 288, 2 097 152, 4 194 304, 16 777 216, 33 554 432, 67 108 864,
# 134 217 728)
SIZES = [1, 2, 3, 63, 64, 65, 255, 1023, 2047, 2048, 2049, 4095, 4096, 4097, 8191, 8192, 8193,
         100_000, 524_288, 524_289, 1_000_000, 2_097_153, 4_194_305, 10_000_003, 16_777_217,
         33_554_433, 34_000_001, 67_108_864, 67_108_865, 134_300_000]


@pytest.fixture(params=["two_launch", "single_pass"])
def scan_variant(request):
    """The library reads GEAR_HIP_SCAN_SINGLE_PASS at every call."""
    old = os.environ.get("GEAR_HIP_SCAN_SINGLE_PASS")
    os.environ["GEAR_HIP_SCAN_SINGLE_PASS"] = "1" if request.param == "single_pass" else "0"
    yield request.param
    if old is None:
        os.environ.pop("GEAR_HIP_SCAN_SINGLE_PASS", None)
    else:
        os.environ["GEAR_HIP_SCAN_SINGLE_PASS"] = old


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _priorities(n, seed):
    rng = np.random.default_rng(seed)
    return (rng.lognormal(0.0, 1.0, size=n) ** 0.6).astype(np.float32)


@pytest.mark.parametrize("n", SIZES)
def test_scan_integer_valued_is_bit_exact(oracle, n, scan_variant):
    """Integer-valued fp32 priorities: every partial sum is exact in fp64, so any summation order
    must reproduce the sequential oracle bit for bit."""
    from gear_amd import ops
    rng = np.random.default_rng(n)
    p = rng.integers(0, 1000, size=n).astype(np.float32)
    announce("scan integer-valued n=%d %s" % (n, scan_variant))
    got = ops.prefix_sum(_dev(p))
    torch.cuda.synchronize()
    exp = oracle.scan_f32_f64(p)
    assert np.array_equal(got.cpu().numpy(), exp)
    assert np.array_equal(exp, np.cumsum(p.astype(np.float64)))


@pytest.mark.parametrize("n", [1, 4097, 1_000_000, 10_000_003])
def test_scan_lognormal_close_to_sequential(oracle, n, scan_variant):
    """Random priorities: the parallel fp64 sum may differ from the sequential one in the last
    bits only: relative error <= 1e-12 (tolerance of the fp64 prefix), and it is monotone."""
    from gear_amd import ops
    p = _priorities(n, 1002)
    announce("scan lognormal n=%d %s" % (n, scan_variant))
    got = ops.prefix_sum(_dev(p)).cpu().numpy()
    exp = oracle.scan_f32_f64(p)
    rel = np.max(np.abs(got - exp) / exp)
    assert rel <= 1e-12, rel
    assert np.all(np.diff(got) >= 0)


def test_scan_repeated_runs_agree(oracle, scan_variant):
    """Range sums travel between workgroups through the workspace (between two launches, or
    published and polled inside one): 30 runs must all be exact (integer-valued input, reused
    workspace)."""
    from gear_amd import ops
    n = 10_000_000
    rng = np.random.default_rng(5)
    p = rng.integers(0, 64, size=n).astype(np.float32)
    exp = torch.from_numpy(np.cumsum(p.astype(np.float64))).cuda()
    dp = _dev(p)
    out = torch.empty(n, dtype=torch.float64, device="cuda")
    announce("scan repeated 30x n=%d %s" % (n, scan_variant))
    for it in range(30):
        out.fill_(-1.0)
        ops.prefix_sum(dp, out=out)
        assert torch.equal(out, exp), "run %d" % it


@pytest.mark.parametrize("n", [1, 2047, 2048, 2049, 100_000, 3_000_001])
def test_scan_i64_exact(oracle, n, scan_variant):
    from gear_amd import ops
    rng = np.random.default_rng(n + 1)
    w = rng.integers(0, 1001, size=n).astype(np.int64)
    announce("scan int64 n=%d %s" % (n, scan_variant))
    got = ops.prefix_sum_i64(_dev(w)).cpu().numpy()
    assert np.array_equal(got, oracle.scan_i64(w))
    assert np.array_equal(got, np.cumsum(w))


@pytest.mark.parametrize("n", [1, 5, 4096, 1_000_003])
def test_sum_f32(oracle, n):
    import math
    from gear_amd import ops
    p = _priorities(n, 3)
    announce("sum n=%d" % n)
    out64 = torch.zeros(1, dtype=torch.float64, device="cuda")
    out = ops.sum_f32(_dev(p), out_f64=out64)
    exact = math.fsum(float(x) for x in p)
    assert abs(out64.item() - exact) <= 1e-12 * exact
    assert abs(out64.item() - oracle.sum_f32(p)) <= 1e-12 * exact
    assert out.item() == np.float32(out64.item())


def _boundary_close(prefix, t, idx, rel=1e-9):
    """Draws within rel * total of a bucket boundary (the exemption the benchmark definition allows)."""
    total = prefix[-1]
    lo = np.where(idx > 0, prefix[np.maximum(idx - 1, 0)], 0.0)
    hi = prefix[idx]
    return np.minimum(np.abs(t - lo), np.abs(t - hi)) <= rel * total


def test_config2_prioritized_sampling(oracle):
    """benchmark config 2 at full size: 1e6 lognormal^0.6 priorities, 4096 fp32 draws in [0, sum),
    indices bit-exact vs the sequential fp64 oracle except boundary-close draws (< 1e-6 of the
    draws), importance weights (N p / sum)^-0.4 / max within 1 ulp of fp32."""
    from gear_amd import ops
    n, B = 1_000_000, 4096
    p = _priorities(n, 1002)
    rng = np.random.default_rng(1002)
    exp_prefix = oracle.scan_f32_f64(p)
    u = (rng.random(B, dtype=np.float32) * np.float32(exp_prefix[-1])).astype(np.float32)
    u = np.minimum(u, np.nextafter(np.float32(exp_prefix[-1]), np.float32(0)))
    dp, du = _dev(p), _dev(u)
    announce("config2 scan + search + weights")
    prefix = ops.prefix_sum(dp)
    idx, w = ops.upper_bound(prefix, du, priorities=dp, beta=0.4)
    torch.cuda.synchronize()
    got_prefix = prefix.cpu().numpy()
    got_idx = idx.cpu().numpy()
    # (a) search is exact on the prefix it was given
    assert np.array_equal(got_idx, oracle.upper_bound_f64(got_prefix, u))
    assert np.array_equal(got_idx,
                          np.minimum(np.searchsorted(got_prefix, u.astype(np.float64), "right"),
                                     n - 1))
    # (b) end to end vs the sequential fp64 prefix
    exp_idx = oracle.upper_bound_f64(exp_prefix, u)
    diff = got_idx != exp_idx
    close = _boundary_close(exp_prefix, u.astype(np.float64), exp_idx)
    assert not np.any(diff & ~close)
    assert diff.sum() <= max(1e-6 * B, 0) or diff.sum() == 0
    # (c) importance weights
    exp_w = oracle.is_weights(p, exp_prefix[-1], exp_idx, 0.4)
    got_w = w.cpu().numpy()
    same = ~diff
    ulp = np.spacing(np.abs(exp_w[same]).astype(np.float32))
    assert np.all(np.abs(got_w[same] - exp_w[same]) <= ulp)
    assert got_w.max() == 1.0
    # closed form of one weight, evaluated with Python floats
    j = int(np.argmin(got_w))
    wj = (n * float(p[exp_idx[j]]) / float(exp_prefix[-1])) ** -0.4
    wmax = max((n * float(p[i]) / float(exp_prefix[-1])) ** -0.4 for i in exp_idx)
    assert abs(got_w[j] - wj / wmax) <= 2e-7 * (wj / wmax)


def test_search_small_brute_force(oracle):
    """N <= 64: compare with a linear scan, including zero-weight entries (never selected unless
    the draw is clipped at the end) and draws equal to a boundary."""
    from gear_amd import ops
    rng = np.random.default_rng(9)
    for n in (1, 2, 7, 64):
        p = rng.integers(0, 4, size=n).astype(np.float32)
        p[rng.integers(0, n)] = 3.0
        prefix_np = np.cumsum(p.astype(np.float64))
        u = np.concatenate([prefix_np, prefix_np - 0.5, [0.0], rng.random(50) * prefix_np[-1]])
        u = np.clip(u, 0, None).astype(np.float32)
        announce("search brute force n=%d" % n)
        prefix = ops.prefix_sum(_dev(p))
        idx = ops.upper_bound(prefix, _dev(u)).cpu().numpy()
        brute = np.array([min(sum(1 for i in range(n) if prefix_np[i] <= float(t)), n - 1)
                          for t in u])
        assert np.array_equal(idx, brute)
        inside = u.astype(np.float64) < prefix_np[-1]
        assert np.all(p[idx[inside]] > 0)  # zero-weight entries are never drawn


def test_search_unit_uniforms(oracle):
    from gear_amd import ops
    n, B = 300_000, 2048
    p = _priorities(n, 12)
    u01 = np.random.default_rng(12).random(B, dtype=np.float32)
    announce("search unit uniforms")
    prefix = ops.prefix_sum(_dev(p))
    idx = ops.upper_bound(prefix, _dev(u01), unit_uniforms=True).cpu().numpy()
    pre = prefix.cpu().numpy()
    assert np.array_equal(idx, oracle.upper_bound_f64(pre, u01, unit_uniforms=True))
    t = u01.astype(np.float64) * pre[-1]
    assert np.array_equal(idx, np.minimum(np.searchsorted(pre, t, "right"), n - 1))


def test_config3_length_weighted_trajectory_sampling(oracle):
    """Config 3's sampler: 100 000 trajectory lengths as int64 weights, exact integer prefix,
    1024 draws; a trajectory is drawn with probability proportional to its length."""
    from gear_amd import ops
    rng = np.random.default_rng(1003)
    lens = rng.integers(200, 1001, size=100_000).astype(np.int64)
    u = rng.random(1024)
    announce("config3 int64 prefix + search")
    prefix = ops.prefix_sum_i64(_dev(lens))
    idx = ops.upper_bound_i64(prefix, _dev(u), unit_uniforms=True).cpu().numpy()
    pre = np.cumsum(lens)
    assert np.array_equal(prefix.cpu().numpy(), pre)
    t = np.floor(u * float(pre[-1])).astype(np.int64)
    assert np.array_equal(idx, np.minimum(np.searchsorted(pre, t, "right"), len(lens) - 1))
    assert np.array_equal(idx, oracle.upper_bound_i64(pre, u, unit_uniforms=True))
    t2 = rng.integers(0, pre[-1], size=1024).astype(np.int64)
    idx2 = ops.upper_bound_i64(prefix, _dev(t2), unit_uniforms=False).cpu().numpy()
    assert np.array_equal(idx2, np.searchsorted(pre, t2, "right"))


@pytest.mark.parametrize("num", [1, 100, 1024, 1025, 2048, 3000, 4096, 4097, 10_000])
def test_sample_sorted_equals_search_then_sort(oracle, num):
    """The one-call sampler (search + sort + split) returns exactly sort(upper_bound(draws)) and
    the divmod split of it; 4096 and 4097 draws straddle the one-workgroup / multi-kernel paths."""
    from gear_amd import ops
    n, T = 777_777, 1000
    p = _priorities(n, 77)
    u01 = np.random.default_rng(num).random(num, dtype=np.float32)
    announce("sample_sorted num=%d" % num)
    prefix = ops.prefix_sum(_dev(p))
    srt, idxs, tss, lens = ops.sample_sorted(prefix, _dev(u01), unit_uniforms=True,
                                             trajectory_length=T, modulo=500_000)
    plain = ops.sample_sorted(prefix, _dev(u01), unit_uniforms=True)
    torch.cuda.synchronize()
    pre = prefix.cpu().numpy()
    exp = np.sort(oracle.upper_bound_f64(pre, u01, unit_uniforms=True))
    assert np.array_equal(srt.cpu().numpy(), exp)
    assert np.array_equal(plain.cpu().numpy(), exp)
    f = exp % 500_000
    assert np.array_equal(idxs.cpu().numpy(), f // T)
    assert np.array_equal(tss.cpu().numpy(), f % T)
    assert np.array_equal(lens.cpu().numpy(), f % T + 1)


@pytest.mark.parametrize("num", [64, 65, 2048, 4096])
def test_sample_sorted_with_many_equal_indices(oracle, num):
    """Few buckets, many draws: nearly every found index repeats, so the ranking sort must place
    equal keys by position without gaps or collisions."""
    from gear_amd import ops
    n, T = 37, 5
    p = _priorities(n, 5)
    u01 = np.random.default_rng(num + 1).random(num, dtype=np.float32)
    announce("sample_sorted ties num=%d" % num)
    prefix = ops.prefix_sum(_dev(p))
    srt, idxs, tss, lens = ops.sample_sorted(prefix, _dev(u01), unit_uniforms=True,
                                             trajectory_length=T)
    torch.cuda.synchronize()
    exp = np.sort(oracle.upper_bound_f64(prefix.cpu().numpy(), u01, unit_uniforms=True))
    assert np.array_equal(srt.cpu().numpy(), exp)
    assert np.array_equal(idxs.cpu().numpy(), exp // T)
    assert np.array_equal(tss.cpu().numpy(), exp % T)
    assert np.array_equal(lens.cpu().numpy(), exp % T + 1)


@pytest.mark.parametrize("n", [5_000, 1_000_000, 10_000_003])
def test_rescan_from_first_changed_is_bit_identical(oracle, n):
    """gear_hip_rescan_f32_f64: after priorities[k:] changed, rescanning from k gives exactly the
    bits of a full scan of the changed array (the range sums before k are reused from the
    workspace), for k inside the first range, on range boundaries, at the end and beyond it."""
    from gear_amd import ops
    rng = np.random.default_rng(n)
    p = _priorities(n, 11)
    dp = _dev(p)
    state = ops.PrefixState()
    state.scan(dp)
    other = _dev(_priorities(70_000, 12))
    for k in (1, 2047, 2048, 4096, n // 3, n // 2 + 1, n - 1, n, n + 5):
        if k < n:
            m = min(n - k, 1000)
            pos = k + rng.integers(0, n - k, size=m)
            pos[0] = k
            p[pos] = (rng.lognormal(0, 1, size=m) ** 0.6).astype(np.float32)
            dp.copy_(torch.from_numpy(p))
        ops.prefix_sum(other)                      # scans of other arrays do not disturb the state
        announce("rescan n=%d first_changed=%d" % (n, k))
        got = state.scan(dp, first_changed=k)
        full = ops.prefix_sum(dp)
        torch.cuda.synchronize()
        assert torch.equal(got, full), "first_changed=%d" % k
    exp = oracle.scan_f32_f64(p)
    assert np.max(np.abs(got.cpu().numpy() - exp) / exp) <= 1e-12


def test_rescan_integer_valued_matches_oracle_exactly(oracle):
    from gear_amd import ops
    n = 3_000_017
    rng = np.random.default_rng(8)
    p = rng.integers(0, 100, size=n).astype(np.float32)
    dp = _dev(p)
    state = ops.PrefixState()
    state.scan(dp)
    for k in (2_999_000, 1_500_000, 77):
        p[k:k + 500] = rng.integers(0, 100, size=500).astype(np.float32)
        dp.copy_(torch.from_numpy(p))
        announce("integer rescan first_changed=%d" % k)
        got = state.scan(dp, first_changed=k).cpu().numpy()
        assert np.array_equal(got, oracle.scan_f32_f64(p))


def test_split_step_index():
    """flat step index -> (trajectory, timestep, length = timestep + 1), optionally modulo the
    number of steps in the table (benchmark config 5 draws from 1e7 priorities over a 2e6-step
    table)."""
    from gear_amd import ops
    rng = np.random.default_rng(4)
    flat = rng.integers(0, 10_000_000, size=5000).astype(np.int64)
    for T, modulo in ((1000, 0), (1000, 2_000_000), (7, 0), (1, 13)):
        announce("split T=%d modulo=%d" % (T, modulo))
        idxs, tss, lens = ops.split_step_index(_dev(flat), T, modulo)
        torch.cuda.synchronize()
        f = flat % modulo if modulo else flat
        assert np.array_equal(idxs.cpu().numpy(), f // T)
        assert np.array_equal(tss.cpu().numpy(), f % T)
        assert np.array_equal(lens.cpu().numpy(), f % T + 1)


@pytest.mark.parametrize("n", [4097, 100_000, 3_000_001])
def test_scan_i64_signed_weights_with_range_sums_of_minus_one(oracle, n, scan_variant):
    """int64 weights of either sign whose range sums are -1 (the all-ones word): the int64 scan
    never takes a kernel that marks unpublished sums with that word, whatever the environment
    selects, and stays exact."""
    from gear_amd import ops
    rng = np.random.default_rng(n)
    w = rng.integers(-5, 6, size=n).astype(np.int64)
    # make every 2048-element stretch (the smallest range) sum to -1, and so every larger range
    # of 2^k of them sum to -2^k; a second array makes the larger ranges sum to -1 as well
    for width in (2048, 4096, 8192, 16384):
        v = w.copy()
        for s in range(0, n - width + 1, width):
            v[s + width - 1] -= v[s:s + width].sum() + 1
        announce("scan int64 signed n=%d range width %d %s" % (n, width, scan_variant))
        got = ops.prefix_sum_i64(_dev(v)).cpu().numpy()
        assert np.array_equal(got, np.cumsum(v))
        assert np.array_equal(got, oracle.scan_i64(v))


def test_scans_of_more_ranges_than_a_workgroup_adds_up():
    """Beyond 16384 ranges (134 M fp32 / 67 M int64 elements) a launch in between scans the range
    sums: same bits on every run and for the rescan of a suffix, exact on integers, int64 sums of
    -1 included."""
    from gear_amd import ops
    n = (1 << 27) + 5001
    g = torch.Generator(device="cuda").manual_seed(11)
    announce("scan f32->f64 n=%d (three launches)" % n)
    w = torch.randint(0, 1000, (n,), device="cuda", generator=g).float()
    got = ops.prefix_sum(w).clone()
    assert torch.equal(got, torch.cumsum(w.double(), 0))          # integers: exact in any order
    w = torch.rand(n, device="cuda", generator=g)
    first = ops.prefix_sum(w).clone()
    again = ops.prefix_sum(w).clone()
    assert torch.equal(first, again)
    ref = torch.cumsum(w.double(), 0)
    assert float((first - ref).abs().max() / ref[-1]) <= 1e-12
    del ref, again
    state = ops.PrefixState()
    state.scan(w)
    for k in (1, 8191, 50_000_000, n - 1):
        w[k:] = torch.rand(n - k, device="cuda", generator=g)
        announce("rescan n=%d from %d (three launches)" % (n, k))
        got = state.scan(w, first_changed=k)
        full = ops.prefix_sum(w)
        torch.cuda.synchronize()
        assert torch.equal(got, full)
    del w, got, full, first, state
    n = (1 << 26) + 4097
    announce("scan int64 n=%d (three launches)" % n)
    v = torch.randint(-5, 6, (n,), device="cuda", generator=g, dtype=torch.int64)
    v[4095::4096] -= v.view(-1)[: (n // 4096) * 4096].view(-1, 4096).sum(1) + 1   # every range sums to -1
    assert torch.equal(ops.prefix_sum_i64(v), torch.cumsum(v, 0))


def test_chained_scan_ignores_what_the_workspace_held():
    """A workspace need not be initialised, and what memory holds is rarely random: words left by
    index arrays, counts and their sums are small integers, as are the tags 1, 2, 3 ... that a
    launch counter would hand out.  The chained kernel must not take any of it for a range sum
    published in its own launch."""
    import ctypes
    from gear_amd import _cabi
    lib = _cabi.load()
    g = torch.Generator(device="cuda").manual_seed(5)
    n = 5_852_911
    w = torch.rand(n, device="cuda", generator=g)
    nbytes = int(lib.gear_hip_scan_workspace_bytes(n))
    ws = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    out = torch.empty(n, dtype=torch.float64, device="cuda")

    def scan():
        rc = lib.gear_hip_scan_f32_f64(ctypes.c_void_p(w.data_ptr()), ctypes.c_void_p(out.data_ptr()),
                                       n, ctypes.c_void_p(ws.data_ptr()), ws.numel(),
                                       ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
        assert rc == 0
        torch.cuda.synchronize()
        return out.clone()

    expect = scan()                                     # zeroed workspace
    words = ws.view(torch.int64)
    sums = torch.cumsum(torch.randint(0, 1 << 20, (words.numel(),), device="cuda", generator=g,
                                      dtype=torch.int64), 0)
    patterns = {
        "running sums of small integers": sums,
        "0, 1, 2, ...": torch.arange(words.numel(), device="cuda", dtype=torch.int64),
        "tags 1, 2, 3 ... of an earlier process": (torch.arange(words.numel(), device="cuda",
                                                                dtype=torch.int64) // 3 % 64 + 1) << 22,
        "all ones": torch.full((words.numel(),), -1, device="cuda", dtype=torch.int64),
    }
    for what, fill in patterns.items():
        for rep in range(8):                            # several launches: several tags
            words.copy_(fill)
            announce("chained scan, workspace holds %s (%d)" % (what, rep))
            assert torch.equal(scan(), expect), what


@pytest.mark.parametrize("n", [4097, 1_000_000, 3_000_001, 40_000_001])
def test_chained_scan_with_no_patience_sums_the_missing_ranges_itself(oracle, n):
    """The chained kernel waits a bounded number of polls for an earlier range's sum and then sums
    that range itself.  With a limit of 0 polls (forced from the host) every workgroup takes
    that path for whatever is not published yet: the kernel ends and the prefix is bit-identical
    to the two-launch result, for fp64 and int64."""
    from gear_amd import ops
    rng = np.random.default_rng(n)
    p = _priorities(n, 12)
    w = rng.integers(-3, 1000, size=n).astype(np.int64)
    dp, dw = _dev(p), _dev(w)
    old = {k: os.environ.get(k) for k in ("GEAR_HIP_SCAN_SINGLE_PASS", "GEAR_HIP_SCAN_SPIN_LIMIT")}
    try:
        os.environ["GEAR_HIP_SCAN_SINGLE_PASS"] = "0"
        ref = ops.prefix_sum(dp).clone()
        ref_i = ops.prefix_sum_i64(dw).clone()
        os.environ["GEAR_HIP_SCAN_SINGLE_PASS"] = "1"
        os.environ["GEAR_HIP_SCAN_SPIN_LIMIT"] = "0"
        announce("chained scan, spin limit 0, n=%d" % n)
        got = ops.prefix_sum(dp).clone()
        got_i = ops.prefix_sum_i64(dw).clone()
        os.environ["GEAR_HIP_SCAN_SPIN_LIMIT"] = "3"
        got3 = ops.prefix_sum(dp).clone()
        torch.cuda.synchronize()
    finally:
        for k, v in old.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v
    assert torch.equal(got, ref) and torch.equal(got3, ref)
    assert torch.equal(got_i, ref_i)
    assert np.array_equal(got_i.cpu().numpy(), np.cumsum(w))


def test_scan_under_graph_capture_replays_correctly(oracle):
    """A captured scan must not bake a one-time tag into the graph: every replay (with changed
    priorities in between) equals the eager result."""
    from gear_amd import ops
    n = 300_000
    rng = np.random.default_rng(9)
    dp = _dev(_priorities(n, 9))
    out = torch.empty(n, dtype=torch.float64, device="cuda")
    ops.prefix_sum(dp, out=out)                      # warm-up: workspace exists before capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops.prefix_sum(dp, out=out)                  # workspace of the capture stream
    torch.cuda.synchronize()
    with torch.cuda.graph(g, stream=side):
        ops.prefix_sum(dp, out=out)
    for it in range(4):
        dp.copy_(_dev(_priorities(n, 100 + it)))
        announce("graph replay %d of a captured scan" % it)
        g.replay()
        torch.cuda.synchronize()
        eager = ops.prefix_sum(dp)
        torch.cuda.synchronize()
        assert torch.equal(out, eager), it


def test_chained_scans_on_two_streams_next_to_a_busy_gpu():
    """Workgroups of the chained kernel wait for sums that other workgroups of the same launch
    publish.  With two such launches in flight on two streams and a third stream keeping every CU
    busy, late workgroups start when a slot frees: every result must still equal the two-launch
    result bit for bit (each stream has a workspace of its own)."""
    from gear_amd import ops
    rng = np.random.default_rng(17)
    sizes = [10_000_000, 4_300_000, 1_000_000]
    pri = [_dev((rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)) for n in sizes]
    old = os.environ.get("GEAR_HIP_SCAN_SINGLE_PASS")
    os.environ["GEAR_HIP_SCAN_SINGLE_PASS"] = "0"
    try:
        ref = [ops.prefix_sum(p).clone() for p in pri]
        torch.cuda.synchronize()
    finally:
        if old is None:
            os.environ.pop("GEAR_HIP_SCAN_SINGLE_PASS", None)
        else:
            os.environ["GEAR_HIP_SCAN_SINGLE_PASS"] = old
    s1, s2, s3 = torch.cuda.Stream(), torch.cuda.Stream(), torch.cuda.Stream()
    busy = torch.ones(1 << 27, dtype=torch.float32, device="cuda")
    outs = [[torch.empty_like(r) for r in ref] for _ in range(2)]
    announce("chained scans on two streams, 25 rounds")
    for _ in range(25):
        with torch.cuda.stream(s3):
            busy.mul_(1.0001)
            busy.add_(1.0)
        for si, st in enumerate((s1, s2)):
            with torch.cuda.stream(st):
                for j, p in enumerate(pri):
                    ops.prefix_sum(p, out=outs[si][j])
        torch.cuda.synchronize()
        for si in range(2):
            for j in range(len(pri)):
                assert torch.equal(outs[si][j], ref[j])


def test_select_with_lookups_equals_the_separate_calls(oracle):
    """gear_hip_sample_lookup_f64 / gear_hip_sort_lookup_i64 / gear_hip_lookup_i64 against the
    chain they fold (search -> sort -> indices[p] -> - offset -> timesteps[local]) on both sides
    of the 4096-entry ranking sort, with an index offset, and against numpy."""
    from gear_amd import ops
    rng = np.random.default_rng(1234)
    for n, num, offset in ((1, 1, 0), (5_000, 257, 0), (300_000, 1024, 3), (300_000, 1025, 3),
                           (100_000, 4096, 1_000_000), (100_000, 4097, 77), (1_000_000, 20_000, 5)):
        announce("select + look-ups n=%d num=%d offset=%d" % (n, num, offset))
        pri = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
        if n > 10:
            pri[rng.integers(0, n, size=n // 7)] = 0.0           # never drawn
        pri[0] = max(pri[0], 0.5)
        lengths = rng.integers(1, 1001, size=n).astype(np.int64)
        indices = np.arange(n, dtype=np.int64) + offset          # ascending, as a loader's are
        u = rng.random(num, dtype=np.float32)
        dpri, dlen, dind, du = _dev(pri), _dev(lengths), _dev(indices), _dev(u)
        prefix = ops.prefix_sum(dpri)
        sampled, local, lens = ops.sample_lookup(prefix, du, index_table=dind, index_offset=offset,
                                                 lengths_table=dlen)
        pos = ops.sample_sorted(prefix, du, unit_uniforms=True)
        torch.cuda.synchronize()
        hpos = pos.cpu().numpy()
        exp_pos = np.sort(oracle.upper_bound_f64(prefix.cpu().numpy(), u, unit_uniforms=True))
        assert np.array_equal(hpos, exp_pos)
        assert np.array_equal(sampled.cpu().numpy(), indices[exp_pos])
        assert np.array_equal(local.cpu().numpy(), exp_pos)
        assert np.array_equal(lens.cpu().numpy(), lengths[exp_pos])
        # identity index table, only the lengths asked for
        s2, l2, n2 = ops.sample_lookup(prefix, du, lengths_table=dlen)
        torch.cuda.synchronize()
        assert np.array_equal(s2.cpu().numpy(), exp_pos) and np.array_equal(n2.cpu().numpy(), lengths[exp_pos])
        # uniform draws: positions given, with duplicates
        draws = rng.integers(0, n, size=num).astype(np.int64)
        s3, l3, n3 = ops.sort_lookup(_dev(draws), n, index_table=dind, index_offset=offset,
                                     lengths_table=dlen)
        torch.cuda.synchronize()
        sd = np.sort(draws)
        assert np.array_equal(s3.cpu().numpy(), indices[sd])
        assert np.array_equal(l3.cpu().numpy(), sd) and np.array_equal(n3.cpu().numpy(), lengths[sd])
        # positions in their own order (a top-k's selection), entries outside the tables read 0
        order = draws.copy()
        order[::97] = n + 3
        s4, l4, n4 = ops.lookup(_dev(order), index_table=dind, index_offset=offset, lengths_table=dlen)
        torch.cuda.synchronize()
        inside = order < n
        exp_s = np.where(inside, indices[np.minimum(order, n - 1)], 0)
        exp_l = exp_s - offset
        ok_l = (exp_l >= 0) & (exp_l < n)
        exp_n = np.where(ok_l, lengths[np.clip(exp_l, 0, n - 1)], 0)
        assert np.array_equal(s4.cpu().numpy(), exp_s) and np.array_equal(l4.cpu().numpy(), exp_l)
        assert np.array_equal(n4.cpu().numpy(), exp_n)


def test_select_over_an_int64_prefix_with_window_starts(oracle):
    """gear_hip_sample_lookup_i64: trajectories drawn by length (int64 prefix, float64 uniforms or
    int64 targets), sorted, with their lengths and the start of a window inside each --
    floor(v * (length - window + 1)) -- against the oracle's search and numpy, on both sides of
    the 4096 draws of the ranking sort."""
    from gear_amd import ops
    rng = np.random.default_rng(4242)
    for n, num, window in ((1, 1, 1), (100_000, 1024, 20), (100_000, 1025, 20), (7_777, 333, 1),
                           (250_000, 4096, 64), (250_000, 5000, 200)):
        announce("int64 select + look-ups n=%d num=%d window=%d" % (n, num, window))
        lengths = rng.integers(1, 1001, size=n).astype(np.int64)
        if n > 10:
            lengths[rng.integers(0, n, size=n // 9)] = 0          # never drawn
        lengths[0] = max(lengths[0], 1)
        u = rng.random(num)
        v = rng.random(num)
        dlen = _dev(lengths)
        prefix = ops.prefix_sum_i64(dlen)
        hp = prefix.cpu().numpy()
        assert np.array_equal(hp, np.cumsum(lengths))
        traj, local, lens, starts = ops.sample_lookup(prefix, _dev(u), lengths_table=dlen,
                                                      start_uniforms=_dev(v), window=window)
        torch.cuda.synchronize()
        exp = np.sort(oracle.upper_bound_i64(hp, u, unit_uniforms=True))
        assert np.array_equal(traj.cpu().numpy(), exp)
        assert np.array_equal(local.cpu().numpy(), exp)
        assert np.array_equal(lens.cpu().numpy(), lengths[exp])
        room = lengths[exp] - (window - 1)
        exp_starts = np.where(room > 0, np.floor(v * room.astype(np.float64)).astype(np.int64), 0)
        assert np.array_equal(starts.cpu().numpy(), exp_starts)
        assert np.all(exp_starts + np.minimum(window, lengths[exp]) <= lengths[exp])
        # int64 targets instead of uniforms, no starts
        t = rng.integers(0, hp[-1], size=num).astype(np.int64)
        traj2, _, lens2 = ops.sample_lookup(prefix, _dev(t), unit_uniforms=False, lengths_table=dlen)
        torch.cuda.synchronize()
        exp2 = np.sort(np.minimum(np.searchsorted(hp, t, side="right"), n - 1))
        assert np.array_equal(traj2.cpu().numpy(), exp2)
        assert np.array_equal(lens2.cpu().numpy(), lengths[exp2])
    with pytest.raises(ValueError):
        ops.sample_lookup(ops.prefix_sum(_dev(np.ones(8, np.float32))), _dev(np.zeros(2, np.float32)),
                          lengths_table=_dev(np.ones(8, np.int64)),
                          start_uniforms=_dev(np.zeros(2)), window=2)


def test_staggered_start_of_the_chained_scan_changes_no_bit():
    """GEAR_HIP_SCAN_STAGGER_PS (read at every call): workgroups of the chained kernel's first
    wave start a little after one another above 512 ranges.  Off, at the default and four times
    as long, the prefix has the same bits."""
    from gear_amd import ops
    rng = np.random.default_rng(4321)
    pri = _dev((rng.lognormal(0, 1, size=10_000_003) ** 0.6).astype(np.float32))
    old = os.environ.get("GEAR_HIP_SCAN_STAGGER_PS")
    try:
        outs = []
        for ps in ("0", None, "20000"):
            if ps is None:
                os.environ.pop("GEAR_HIP_SCAN_STAGGER_PS", None)
            else:
                os.environ["GEAR_HIP_SCAN_STAGGER_PS"] = ps
            announce("chained scan, stagger %s ps" % ps)
            outs.append(ops.prefix_sum(pri).clone())
        torch.cuda.synchronize()
        assert torch.equal(outs[0], outs[1]) and torch.equal(outs[1], outs[2])
    finally:
        if old is None:
            os.environ.pop("GEAR_HIP_SCAN_STAGGER_PS", None)
        else:
            os.environ["GEAR_HIP_SCAN_STAGGER_PS"] = old
