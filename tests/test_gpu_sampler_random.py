"""Randomised differential test of the sampler-side entry points (prefix sums, incremental
rescan, search, one-call batch sampler, top-k, sort, scatter) against the CPU oracle: random
sizes, value distributions, tie densities and batch sizes, seeded."""
import numpy as np
import pytest

from conftest import announce

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _values(rng, n):
    """fp32 priorities from one of several distributions, some with masses of ties or zeros."""
    kind = int(rng.integers(0, 6))
    if kind == 0:
        v = rng.lognormal(0.0, 1.0, size=n) ** 0.6
    elif kind == 1:
        v = rng.integers(0, int(rng.integers(2, 50)), size=n).astype(np.float64)   # heavy ties
    elif kind == 2:
        v = rng.random(n) * (rng.random(n) < 0.3)                                 # 70 % zeros
    elif kind == 3:
        v = np.sort(rng.random(n))                                                # ascending
    elif kind == 4:
        v = np.full(n, 1.5)                                                       # all equal
    else:
        v = rng.random(n) * 1e-38                                                 # denormals
    v = v.astype(np.float32)
    if not v.any():
        v[int(rng.integers(0, n))] = 1.0      # a sampler needs a positive total
    return kind, v


@pytest.mark.parametrize("seed", list(range(16)))
def test_random_scan_search_sample(oracle, seed):
    from gear_amd import ops
    rng = np.random.default_rng(7000 + seed)
    n = int(rng.integers(1, 3_000_000)) if seed % 4 else int(rng.integers(1, 5000))
    kind, p = _values(rng, n)
    num = int(rng.integers(1, 6000))
    u01 = rng.random(num, dtype=np.float32)
    announce("random sampler seed=%d n=%d kind=%d draws=%d" % (seed, n, kind, num))
    dp = _dev(p)
    state = ops.PrefixState()
    prefix = state.scan(dp)
    exp_prefix = oracle.scan_f32_f64(p)
    got_prefix = prefix.cpu().numpy()
    assert np.all(np.abs(got_prefix - exp_prefix) <= 1e-12 * np.maximum(exp_prefix, 1e-300))
    # searches are checked against the prefix the GPU produced (bit-exact index parity)
    idx = ops.upper_bound(prefix, _dev(u01), unit_uniforms=True)
    exp_idx = oracle.upper_bound_f64(got_prefix, u01, unit_uniforms=True)
    assert np.array_equal(idx.cpu().numpy(), exp_idx)
    T = int(rng.integers(1, 2000))
    srt, idxs, tss, lens = ops.sample_sorted(prefix, _dev(u01), unit_uniforms=True,
                                             trajectory_length=T)
    torch.cuda.synchronize()
    es = np.sort(exp_idx)
    assert np.array_equal(srt.cpu().numpy(), es)
    assert np.array_equal(idxs.cpu().numpy(), es // T)
    assert np.array_equal(tss.cpu().numpy(), es % T)
    assert np.array_equal(lens.cpu().numpy(), es % T + 1)
    # change a tail of the priorities and rescan from there: the bits of a full scan
    k = int(rng.integers(0, n))
    p[k:] = _values(rng, n - k)[1]
    dp.copy_(torch.from_numpy(p))
    got = state.scan(dp, first_changed=k)
    full = ops.prefix_sum(dp)
    torch.cuda.synchronize()
    assert torch.equal(got, full)


@pytest.mark.parametrize("seed", list(range(16)))
def test_random_topk_sort_scatter(oracle, seed):
    from gear_amd import ops
    rng = np.random.default_rng(9000 + seed)
    n = int(rng.integers(1, 2_000_000)) if seed % 4 else int(rng.integers(1, 9000))
    kind, w = _values(rng, n)
    if seed % 3 == 0:
        w = (w - np.float32(0.5)).astype(np.float32)          # negative values as well
    k = int(rng.integers(1, min(n, 70_000) + 1))
    announce("random top-k seed=%d n=%d kind=%d k=%d" % (seed, n, kind, k))
    dw = _dev(w)
    vals, idx = ops.topk(dw, k, sorted_by_value=True)
    _, uidx = ops.topk(dw, k, sorted_by_value=False, want_values=False)
    torch.cuda.synchronize()
    evals, eidx = oracle.topk_f32(w, k, True)
    assert np.array_equal(idx.cpu().numpy(), eidx)
    assert np.array_equal(vals.cpu().numpy().view(np.uint32), evals.view(np.uint32))
    assert np.array_equal(uidx.cpu().numpy(), oracle.topk_f32(w, k, False)[1])
    # sort with payload, random key width
    m = int(rng.integers(1, 200_000))
    bits = int(rng.integers(1, 64))
    keys = rng.integers(0, 1 << min(bits, 62), size=m).astype(np.int64)
    pay = rng.integers(-2**62, 2**62, size=m).astype(np.int64)
    announce("random sort seed=%d m=%d bits=%d" % (seed, m, bits))
    ko, vo = ops.sort_i64(_dev(keys), _dev(pay), key_bits=bits)
    torch.cuda.synchronize()
    ek, ev = oracle.sort_i64(keys, pay)
    assert np.array_equal(ko.cpu().numpy(), ek) and np.array_equal(vo.cpu().numpy(), ev)
    # priority update with duplicates and out-of-range entries: last write wins
    q = int(rng.integers(1, 100_000))
    uidx_np = rng.integers(-3, n + 3, size=q).astype(np.int64)
    uval = rng.random(q, dtype=np.float32)
    announce("random scatter seed=%d updates=%d" % (seed, q))
    ops.scatter(dw, _dev(uidx_np), _dev(uval), unique_indices=False)
    torch.cuda.synchronize()
    assert np.array_equal(dw.cpu().numpy(), oracle.scatter_f32(w.copy(), uidx_np, uval))


def _tied_values(rng, n, k):
    """Priorities with masses of equal or nearly equal entries around and above the k-th largest:
    one to five groups of 500 to 120 000 entries -- above everything, around the threshold, a
    few ulps from another group, or anywhere in the selection -- scattered or as one stretch of
    consecutive entries; or integers from a small range."""
    if int(rng.integers(0, 4)) == 3:
        return rng.integers(0, int(rng.integers(2, 3000)), size=n).astype(np.float32)
    w = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    srt = np.sort(w)
    thr = srt[n - k]
    vals = []
    for _ in range(int(rng.integers(1, 6))):
        c = int(rng.integers(0, 4))
        if c == 0:
            v = np.float32(srt[-1] * rng.uniform(1.0, 3.0))
        elif c == 1:
            v = np.float32(thr * rng.uniform(0.98, 1.3))
        elif c == 2 and vals:
            v = (np.nextafter(vals[-1], np.float32(np.inf), dtype=np.float32) if rng.random() < 0.5
                 else np.float32(vals[-1] * (1 + 1e-6 * rng.integers(1, 50))))
        else:
            v = np.float32(rng.uniform(thr, srt[-1]))
        vals.append(np.float32(v))
        size = int(rng.integers(500, min(120_000, n // 3)))
        if rng.random() < 0.5:
            w[rng.integers(0, n, size=size)] = v
        else:
            a = int(rng.integers(0, n - size))
            w[a:a + size] = v
    return w


@pytest.mark.parametrize("seed", list(range(12)))
def test_random_topk_with_masses_of_ties(oracle, seed):
    """Value order sorts by segments; a segment of thousands of equal priorities does not fit its
    LDS buffers and takes the paths that keep index order instead of sorting by index."""
    from gear_amd import ops
    rng = np.random.default_rng(7000 + seed)
    n = int(rng.integers(262_144, 4_000_000))
    k = int(rng.integers(9_000, min(131_072, n // 8) + 1))
    w = _tied_values(rng, n, k)
    announce("random top-k with ties seed=%d n=%d k=%d" % (seed, n, k))
    dw = _dev(w)
    for by_value in (True, False):
        vals, idx = ops.topk(dw, k, sorted_by_value=by_value)
        torch.cuda.synchronize()
        _, eidx = oracle.topk_f32(w, k, by_value)
        assert np.array_equal(idx.cpu().numpy(), eidx)
        assert np.array_equal(vals.cpu().numpy().view(np.uint32), w[eidx].view(np.uint32))
    ref = np.argsort(-w.astype(np.float64), kind="stable")[:k]     # independent statement
    assert np.array_equal(oracle.topk_f32(w, k, True)[1], ref)


@pytest.mark.parametrize("seed", [3, 8, 13])
def test_random_entry_points_with_workspaces_full_of_leftovers(oracle, seed, monkeypatch):
    """No entry point may depend on what its workspace held: every shared workspace is refilled
    before each use with what recycled memory typically holds (running sums of small integers,
    all ones, 0 1 2 ..., random words)."""
    from gear_amd import ops
    plain_get = ops._ws.get
    uses = [0]

    def leftover_get(tag, nbytes, device):
        buf = plain_get(tag, nbytes, device)
        words = buf[: buf.numel() // 8 * 8].view(torch.int64)
        kind = uses[0] % 4
        uses[0] += 1
        if kind == 0:
            words.copy_(torch.cumsum(torch.randint(0, 1 << 20, (words.numel(),), device=buf.device,
                                                   dtype=torch.int64), 0))
        elif kind == 1:
            words.fill_(-1)
        elif kind == 2:
            words.copy_(torch.arange(words.numel(), device=buf.device, dtype=torch.int64))
        else:
            words.copy_(torch.randint(-2**62, 2**62, (words.numel(),), device=buf.device,
                                      dtype=torch.int64))
        return buf

    monkeypatch.setattr(ops._ws, "get", leftover_get)
    test_random_scan_search_sample(oracle, seed)
    test_random_topk_sort_scatter(oracle, seed)
    assert uses[0] > 0
