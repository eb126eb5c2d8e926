"""GPU tests of the drop-in layer: libgear.core kernel bindings, samplers and OfflineLoader,
through the reference's own call patterns, checked against the CPU oracle."""
import os

import numpy as np
import pytest

from conftest import announce

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def _mpu():
    from gear_amd.mpu import ModelParallelismUnit
    return ModelParallelismUnit(device=torch.device("cuda:0"))


def _dataset(placement, capacity=48, T=40, seed=0):
    """obs fp32[11], actions fp32[3], done uint8 with per-trajectory lengths in [1, T]."""
    from gear_amd.dataset import SharedDataset
    from gear_amd.specs import TableSpec
    tspec = TableSpec.create(trajectory_length=T, capacity=capacity, column_specs=[
        {"shape": [11], "dtype": torch.float32, "name": "observations"},
        {"shape": [3], "dtype": torch.float32, "name": "actions"},
        {"shape": [], "dtype": torch.uint8, "name": "done"}])
    ds = SharedDataset.create(tspec, key=os.getpid() + seed, placement=placement)
    g = torch.Generator().manual_seed(seed)
    raw = {"observations": [], "actions": [], "done": [], "len": []}
    for i in range(capacity):
        n = int(torch.randint(1, T + 1, (1,), generator=g))
        obs = torch.zeros((T, 11))
        act = torch.zeros((T, 3))
        done = torch.zeros(T, dtype=torch.uint8)
        obs[:n] = torch.randn((n, 11), generator=g)
        act[:n] = torch.randn((n, 3), generator=g)
        done[n - 1] = 1
        ds[i] = (float(torch.rand(1, generator=g)) + 0.01, n, [obs, act, done])
        raw["observations"].append(obs[:n]); raw["actions"].append(act[:n])
        raw["done"].append(done[:n]); raw["len"].append(n)
    return ds, raw


PATTERNS = [{"name": "observations", "offset": -40, "length": 40, "pad": "tail"},
            {"name": "actions", "offset": -40, "length": 40, "pad": "head"},
            {"name": "done", "offset": -5, "length": 5, "pad": "head"}]


@pytest.mark.parametrize("placement", ["pinned", "device"])
def test_data_integrity_invariant(placement):
    """examples/offline/single-node/misc.py:5-31 of the reference: gather every trajectory and
    compare with the raw data, for a host-resident (zero-copy) and an HBM-resident table."""
    from gear_amd.loader import OfflineLoader
    announce("loader integrity placement=%s" % placement)
    ds, raw = _dataset(placement)
    loader = OfflineLoader(ds, 16, _mpu(), "Uniform", PATTERNS)
    indices = torch.arange(48, dtype=torch.long)
    loaded = loader.exposed_fused_iterate(indices)
    torch.cuda.synchronize()
    for tid in range(48):
        n = raw["len"][tid]
        obs = loaded[0][tid].cpu()
        assert torch.equal(obs[:n], raw["observations"][tid]) and not obs[n:].any()
        act = loaded[1][tid].cpu()
        assert torch.equal(act[40 - n:], raw["actions"][tid]) and not act[:40 - n].any()
        done = loaded[2][tid].cpu()
        k = min(n, 5)
        assert torch.equal(done[5 - k:], raw["done"][tid][n - k:]) and not done[:5 - k].any()
    # the host sub() + vcopy path of the reference gives the same batch
    tss, low = loader.exposed_low_level_controlled_iterate(indices)
    torch.cuda.synchronize()
    assert tss.tolist() == raw["len"]
    for a, b in zip(loaded, low):
        assert torch.equal(a, b)


@pytest.mark.parametrize("method", ["Uniform", "Weighted", "Topk"])
def test_next_loader_batches(oracle, method):
    from gear_amd.loader import OfflineLoader
    from gear_amd import sampler as smp
    announce("next(loader) sampling=%s" % method)
    ds, raw = _dataset("pinned", seed=3)
    loader = OfflineLoader(ds, 32 if method != "Topk" else 16, _mpu(),
                           "TopK" if method == "Topk" else method, PATTERNS, with_mask=True)
    B = loader._batch_size
    # what the sampler will return, restated with the oracle from the same seeded draws
    gen = torch.Generator("cuda:0").manual_seed(42)
    w = ds.weights.numpy().copy()
    if method == "Uniform":
        draws = torch.randint(0, 48, (B,), generator=gen, dtype=torch.long, device="cuda:0")
        expect = np.sort(draws.cpu().numpy())
    elif method == "Weighted":
        u = torch.rand(B, generator=gen, dtype=torch.float32, device="cuda:0").cpu().numpy()
        expect = np.sort(oracle.upper_bound_f64(oracle.scan_f32_f64(w), u, unit_uniforms=True))
    else:
        expect = oracle.topk_f32(w, B, False)[1]
    timesteps, batch = next(loader)
    torch.cuda.synchronize()
    lens = np.array(raw["len"])[expect]
    assert timesteps.tolist() == lens.tolist()
    for i, tid in enumerate(expect):
        n = raw["len"][tid]
        assert torch.equal(batch[0][i, :n].cpu(), raw["observations"][tid])
        assert torch.equal(batch[1][i, 40 - n:].cpu(), raw["actions"][tid])
        m = loader.last_masks[0][i].cpu()
        assert int(m.sum()) == n and bool(m[:n].all())
    assert batch[0].shape == (B, 40, 11) and batch[2].dtype == torch.uint8
    assert isinstance(loader._sampler, getattr(smp, type(loader._sampler).__name__))


def test_samplers_against_oracle(oracle):
    from gear_amd.sampler import TopKSampler, UniformSampler, WeightedSampler
    mpu = _mpu()
    n, B = 200_000, 2048
    rng = np.random.default_rng(8)
    w = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    indices = torch.arange(n, dtype=torch.long, device="cuda:0") + 1000   # shard offset 1000
    dw = torch.from_numpy(w)
    announce("samplers vs oracle")
    got = WeightedSampler(mpu, seed=42).sync_sample(indices, dw, B).cpu().numpy()
    gen = torch.Generator("cuda:0").manual_seed(42)
    u = torch.rand(B, generator=gen, dtype=torch.float32, device="cuda:0").cpu().numpy()
    pos = oracle.upper_bound_f64(oracle.scan_f32_f64(w), u, unit_uniforms=True)
    assert np.array_equal(got, np.sort(pos) + 1000)
    got = TopKSampler(mpu).sync_sample(indices, dw, 500).cpu().numpy()
    assert np.array_equal(got, oracle.topk_f32(w, 500, False)[1] + 1000)
    got = UniformSampler(mpu, seed=7).sync_sample(indices, dw, B).cpu().numpy()
    gen = torch.Generator("cuda:0").manual_seed(7)
    draws = torch.randint(0, n, (B,), generator=gen, dtype=torch.long, device="cuda:0").cpu().numpy()
    assert np.array_equal(got, np.sort(draws) + 1000)
    # importance weights in draw order
    idx, isw = WeightedSampler(mpu, seed=5).sample_with_importance(indices, dw, 512, beta=0.4)
    gen = torch.Generator("cuda:0").manual_seed(5)
    u = torch.rand(512, generator=gen, dtype=torch.float32, device="cuda:0").cpu().numpy()
    prefix = oracle.scan_f32_f64(w)
    pos = oracle.upper_bound_f64(prefix, u, unit_uniforms=True)
    assert np.array_equal(idx.cpu().numpy(), pos + 1000)
    exp = oracle.is_weights(w, prefix[-1], pos, 0.4)
    assert np.all(np.abs(isw.cpu().numpy() - exp) <= np.spacing(exp))


def test_weighted_sampler_distribution():
    """Closed form: with priorities (1, 2, 3, 4) the draw frequencies approach 0.1 .. 0.4."""
    from gear_amd.sampler import WeightedSampler
    s = WeightedSampler(_mpu(), seed=123)
    idx = torch.arange(4, dtype=torch.long, device="cuda:0")
    w = torch.tensor([1.0, 2.0, 3.0, 4.0])
    counts = np.zeros(4)
    for _ in range(20):
        got = s.sync_sample(idx, w, 4096).cpu().numpy()
        counts += np.bincount(got, minlength=4)
    freq = counts / counts.sum()
    assert np.all(np.abs(freq - np.array([0.1, 0.2, 0.3, 0.4])) < 0.01)


def test_libgear_kernel_bindings(oracle):
    """The reference's tests/test_copy.py and tests/test_sub.py flows through libgear.core."""
    from gear_amd.libgear import core as glibc
    device = torch.device("cuda:0")
    announce("libgear.core.copy_debug (reference tests/test_copy.py)")
    data = torch.ones((32, 100, 4, 3, 2), dtype=torch.float32, device="cpu", pin_memory=True)
    copied = torch.zeros((10, 4, 3, 2), dtype=torch.float32, device=device)
    src_offset = torch.zeros(1, dtype=torch.long, device=device)
    dst_offset = torch.zeros(1, dtype=torch.long, device=device)
    stride = copied.numel() * copied.element_size() * torch.ones(1, dtype=torch.long, device=device)
    glibc.copy_debug(data, copied, src_offset, dst_offset, stride, int(stride[0]))
    torch.cuda.synchronize()
    assert torch.all(copied)

    announce("handler.sub + vcopy from a device tensor (reference tests/test_sub.py)")
    cspecs = [glibc.ColumnSpec([1, 2, 3, 4], glibc.float32, "x")]
    tspec = glibc.TableSpec(0, 1, 100, 32, 1, cspecs)
    table = glibc.TrajectoryTable(tspec, 7, True, "host")
    handler = glibc.get_cpu_handler(table, 32, glibc.Range(0, 0), glibc.Range(0, 32))
    handler.set([0], [glibc.SubscribePattern(-1, 100, glibc.SubscribePattern.PadOption.head)])
    indices = torch.arange(10, dtype=torch.long)
    lengths = torch.ones(10, dtype=torch.long) * 10
    so, do, cl = (torch.zeros(10, dtype=torch.long) for _ in range(3))
    handler.sub(indices, indices.clone(), lengths, 0, so, do, cl)
    mock_src = torch.randn((32, 100, 1, 2, 3, 4), dtype=torch.float32, device=device)
    dst = torch.zeros((10, 100, 1, 2, 3, 4), dtype=torch.float32, device=device)
    glibc.vcopy(glibc.MemoryPtr(mock_src.data_ptr()), dst, so.to(device), do.to(device),
                cl.to(device), 100 * 96)
    torch.cuda.synchronize()
    for i in range(10):
        start = max(i - 1, 0)
        assert torch.equal(dst[i, 100 - (10 - start):], mock_src[i, start:10])
        assert not dst[i, :100 - (10 - start)].any()

    announce("libgear.core.sum / prefix_sum / copy")
    rng = np.random.default_rng(2)
    p = (rng.lognormal(0, 1, size=100_001) ** 0.6).astype(np.float32)
    dp = torch.from_numpy(p).to(device)
    out = torch.zeros(1, dtype=torch.float32, device=device)
    glibc.sum(dp, out, 1)
    assert abs(out.item() - oracle.sum_f32(p)) <= 1e-6 * oracle.sum_f32(p)
    pre64 = torch.empty(len(p), dtype=torch.float64, device=device)
    pre32 = torch.empty(len(p), dtype=torch.float32, device=device)
    glibc.prefix_sum(dp, pre64)
    glibc.prefix_sum(dp, pre32)
    exp = oracle.scan_f32_f64(p)
    assert np.max(np.abs(pre64.cpu().numpy() - exp) / exp) <= 1e-12
    assert np.array_equal(pre32.cpu().numpy(), pre64.cpu().numpy().astype(np.float32))
    src = torch.arange(4096, dtype=torch.uint8, device=device)
    d2 = torch.zeros(64, dtype=torch.uint8, device=device)
    glibc.copy(glibc.MemoryPtr(src.data_ptr()), d2,
               torch.tensor([5, 300], device=device), torch.tensor([0, 32], device=device), 32)
    torch.cuda.synchronize()
    assert torch.equal(d2[:32], src[5:37]) and torch.equal(d2[32:], src[300:332])

    announce("subcopy on a table the GPU cannot see is refused")
    with pytest.raises(RuntimeError, match="not visible to the GPU"):
        z = torch.zeros(10, dtype=torch.long, device=device)
        table.connect()
        handler.subcopy(z, z, z, 0, dst)


def test_update_priorities_then_topk(oracle):
    from gear_amd.loader import OfflineLoader
    ds, raw = _dataset("pinned", seed=5)
    loader = OfflineLoader(ds, 8, _mpu(), "TopK", PATTERNS)
    w = ds.weights.numpy().copy()
    idx = torch.tensor([3, 7, 3, 40, 7])
    val = torch.tensor([9.0, 8.0, 7.5, 6.0, 9.5])
    announce("priority update through the loader, then a top-k batch")
    loader.update_priorities(idx, val)
    oracle.scatter_f32(w, idx.numpy(), val.numpy())
    assert np.array_equal(loader._device_weights.cpu().numpy(), w)
    timesteps, batch = next(loader)
    expect = oracle.topk_f32(w, 8, False)[1]
    assert set([3, 7, 40]).issubset(set(expect.tolist()))
    assert timesteps.tolist() == [raw["len"][i] for i in expect]


def test_cached_weight_updates_reach_the_device(oracle):
    """Online path: pending updates (deduplicated on the host, last write wins) are scattered into
    the device priorities and lengths, then sampled from."""
    from gear_amd.libgear import core as glibc
    from gear_amd.loader import OfflineLoader
    ds, raw = _dataset("pinned", seed=9)
    loader = OfflineLoader(ds, 8, _mpu(), "TopK", PATTERNS)
    w = ds.weights.numpy().copy()
    ts = ds.timesteps.numpy().copy()
    cache = glibc.CachedRequest(48)
    rng = np.random.default_rng(9)
    for _ in range(100):
        i = int(rng.integers(0, 48))
        t = int(rng.integers(1, 41))
        x = float(rng.random()) + 5.0
        cache.warr.update(i, t, x)
        w[i], ts[i] = np.float32(x), t
    announce("apply cached weight updates")
    n = loader.apply_cached_updates(cache)
    torch.cuda.synchronize()
    assert n == len(set(np.nonzero(w >= 5.0)[0].tolist()))
    assert np.array_equal(loader._device_weights.cpu().numpy(), w)
    assert np.array_equal(loader._device_timesteps.cpu().numpy(), ts)
    assert np.array_equal(ds.weights.numpy(), w) and np.array_equal(ds.timesteps.numpy(), ts)
    timesteps, _ = next(loader)
    expect = oracle.topk_f32(w, 8, False)[1]
    assert timesteps.tolist() == ts[expect].tolist()
    # int64 scatter with duplicates: last write wins
    from gear_amd import ops
    tab = torch.zeros(100, dtype=torch.int64, device="cuda")
    idx = torch.tensor([5, 7, 5, 99, 7, 5], device="cuda")
    val = torch.tensor([1, 2, 3, 4, 5, 6], device="cuda")
    ops.scatter(tab, idx, val, unique_indices=False)
    assert tab[5].item() == 6 and tab[7].item() == 5 and tab[99].item() == 4


def test_weighted_loader_rescans_from_the_first_updated_priority(oracle):
    """Online path with the weighted sampler: after priority updates whose indices are known on the
    host, the next batch rescans the prefix from the smallest updated index only; the prefix it
    samples from must equal a full scan of the updated priorities bit for bit, and a batch without
    updates in between must not change it."""
    from gear_amd import ops
    from gear_amd.loader import OfflineLoader
    ds, raw = _dataset("pinned", seed=11)
    loader = OfflineLoader(ds, 8, _mpu(), "Weighted", PATTERNS)
    next(loader)
    w = ds.weights.numpy().copy()
    rng = np.random.default_rng(11)
    for rnd in range(4):
        idx = torch.from_numpy(rng.integers(5 * rnd + 3, 48, size=6))
        val = torch.from_numpy(rng.random(6).astype(np.float32) + 0.5)
        announce("weighted loader update round %d" % rnd)
        loader.update_priorities(idx, val)
        oracle.scatter_f32(w, idx.numpy(), val.numpy())
        assert loader._dirty_from == int(idx.min())
        timesteps, _ = next(loader)
        torch.cuda.synchronize()
        assert loader._dirty_from == 48
        full = ops.prefix_sum(loader._device_weights)
        assert torch.equal(loader._sampler._prefix, full)
        assert np.array_equal(loader._device_weights.cpu().numpy(), w)
        next(loader)                                   # nothing changed: no rescan, same prefix
        torch.cuda.synchronize()
        assert torch.equal(loader._sampler._prefix, full)


@pytest.mark.parametrize("method", ["Uniform", "Weighted", "Topk"])
def test_graph_loader_equals_eager_loader(method):
    """use_graph=True captures select + length look-up + gather once and replays it per batch;
    with the same seed every batch must equal the eager loader's, also after a priority update."""
    from gear_amd.loader import OfflineLoader
    name = {"Topk": "TopK"}.get(method, method)
    ds, raw = _dataset("device", seed=21)
    eager = OfflineLoader(ds, 16, _mpu(), name, PATTERNS, timesteps_on_device=True)
    graph = OfflineLoader(ds, 16, _mpu(), name, PATTERNS, timesteps_on_device=True,
                          use_graph=True)
    with pytest.raises(ValueError):
        OfflineLoader(ds, 16, _mpu(), name, PATTERNS, use_graph=True)
    for it in range(6):
        if it == 3:
            idx = torch.tensor([1, 17, 30, 44])
            val = torch.tensor([50.0, 40.0, 30.0, 20.0])
            eager.update_priorities(idx, val)
            graph.update_priorities(idx, val)
        announce("graph loader %s iteration %d" % (method, it))
        ts_e, b_e = next(eager)
        ts_g, b_g = next(graph)
        torch.cuda.synchronize()
        assert torch.equal(ts_e, ts_g), "iteration %d" % it
        for a, b in zip(b_e, b_g):
            assert torch.equal(a, b), "iteration %d" % it


@pytest.mark.parametrize("placement", ["pinned", "device"])
def test_handler_subcopy_ignores_indices_outside_the_table(placement):
    """handler.subcopy under the reference's own name (src/storage/pybind.cc:140-146) takes the
    checked launch: a negative or too large trajectory index gathers nothing (its rows keep the
    caller's zeros, as the reference's pre-zeroed batch does) instead of reading outside the
    table; the windows with valid indices are what they were."""
    ds, raw = _dataset(placement, seed=31)
    handler = ds._handler
    from gear_amd.libgear import core as glibc
    handler.set([0], [glibc.SubscribePattern(-40, 40, glibc.SubscribePattern.PadOption.tail)])
    idx = torch.tensor([0, -1, 47, 48, 5, 1 << 40, -(1 << 50), 13], device="cuda")
    good = [0, 2, 4, 7]
    lens = torch.tensor([raw["len"][i] if 0 <= i < 48 else 40 for i in idx.tolist()],
                        device="cuda")
    announce("handler.subcopy with indices outside the table, placement=%s" % placement)
    for zero_fill in (False, True):
        dst = torch.zeros((8, 40, 11), dtype=torch.float32, device="cuda") if not zero_fill \
            else torch.full((8, 40, 11), 7.0, dtype=torch.float32, device="cuda")
        handler.subcopy(idx, lens, lens, 0, dst, zero_fill=zero_fill)
        torch.cuda.synchronize()
        out = dst.cpu()
        for row in range(8):
            if row in good:
                tid = int(idx[row])
                n = raw["len"][tid]
                assert torch.equal(out[row, :n], raw["observations"][tid])
                assert not out[row, n:].any()
            else:
                assert not out[row].any()


def test_two_cached_update_flushes_back_to_back(oracle):
    """Two apply_cached_updates calls with no synchronisation in between reuse the same pinned
    staging buffers: the second flush must wait for the first one's uploads.  Device state after
    both equals the host restatement (last write wins inside a flush, later flush wins)."""
    from gear_amd.libgear import core as glibc
    from gear_amd.loader import OfflineLoader
    ds, raw = _dataset("pinned", capacity=4096, T=4, seed=33)
    loader = OfflineLoader(ds, 8, _mpu(), "TopK", PATTERNS_SHORT, timesteps_on_device=True)
    w = ds.weights.numpy().copy()
    ts = ds.timesteps.numpy().copy()
    rng = np.random.default_rng(33)
    cache = glibc.CachedRequest(4096)
    announce("two flushes of cached updates back to back")
    for flush in range(6):
        for _ in range(3000):
            i = int(rng.integers(0, 4096))
            t = int(rng.integers(1, 5))
            x = float(np.float32(rng.random() + 1.0 + flush))
            cache.warr.update(i, t, x)
            w[i], ts[i] = np.float32(x), t
        assert loader.apply_cached_updates(cache) > 0     # no synchronize between flushes
    torch.cuda.synchronize()
    assert np.array_equal(loader._device_weights.cpu().numpy(), w)
    assert np.array_equal(loader._device_timesteps.cpu().numpy(), ts)
    assert np.array_equal(ds.weights.numpy(), w) and np.array_equal(ds.timesteps.numpy(), ts)


PATTERNS_SHORT = [{"name": "observations", "offset": -4, "length": 4, "pad": "tail"}]


@pytest.mark.parametrize("src_placement,dst_placement", [("device", "pinned"), ("pinned", "device"),
                                                         ("device", "device")])
def test_checkpoint_round_trip_between_placements(tmp_path, src_placement, dst_placement):
    """SharedDataset.checkpoint / load (gear/dataset/shared_dataset.py:179-258) with the table in
    HBM or in pinned host memory: the table pickle (src/storage/pybind.cc:178-204) reads a device
    table back through the library, the loaded copy lands in the other placement, and both
    datasets gather byte-identical batches.  The index state travels as the reference's PACKED
    blob -- timesteps int64[n] directly followed by weights fp32[n] at byte 8n, not at the
    128-byte-rounded offset the live index set uses (include/index/set.h:158-181,
    src/index/pybind.cc:15-50)."""
    from gear_amd.dataset import SharedDataset
    from gear_amd.loader import OfflineLoader
    cap = 50                                          # 8 * 50 = 400 is not a multiple of 128
    ds, raw = _dataset(src_placement, capacity=cap, seed=41)
    assert ds._table.placement == src_placement
    path = tmp_path / "ckpt" / "ds.pt"
    announce("checkpoint %s table, load as %s" % (src_placement, dst_placement))
    ds.checkpoint(path)
    state = ds._iset.get_state().__getstate__()
    blob = np.asarray(state[3]).view(np.uint8)
    assert blob.size == 8 * cap + 4 * cap
    assert np.array_equal(blob[:8 * cap].view(np.int64), ds.timesteps.numpy())
    assert np.array_equal(blob[8 * cap:].view(np.float32), ds.weights.numpy())
    os.environ["GEAR_TABLE_PLACEMENT"] = dst_placement
    try:
        ds2 = SharedDataset().load(path, key=os.getpid() + 4100)
    finally:
        del os.environ["GEAR_TABLE_PLACEMENT"]
    assert ds2._table.placement == dst_placement
    assert torch.equal(ds2.weights, ds.weights) and torch.equal(ds2.timesteps, ds.timesteps)
    # the table bytes, read back through the handler of each placement
    nbytes = int(ds._table.get_table_spec().size())
    a = torch.empty(nbytes, dtype=torch.uint8)
    b = torch.empty(nbytes, dtype=torch.uint8)
    ds._handler.raw(0, nbytes).copy_to(a)
    ds2._handler.raw(0, nbytes).copy_to(b)
    assert torch.equal(a, b) and bool(a.any())
    # and what the gather makes of them
    indices = torch.arange(cap, dtype=torch.long)
    l1 = OfflineLoader(ds, 16, _mpu(), "Uniform", PATTERNS)
    l2 = OfflineLoader(ds2, 16, _mpu(), "Uniform", PATTERNS)
    b1 = l1.exposed_fused_iterate(indices)
    b2 = l2.exposed_fused_iterate(indices)
    torch.cuda.synchronize()
    for x, y in zip(b1, b2):
        assert torch.equal(x, y)
    for tid in range(cap):
        n = raw["len"][tid]
        assert torch.equal(b2[0][tid, :n].cpu(), raw["observations"][tid])
    # same sampler seed, same batches from both
    w1 = OfflineLoader(ds, 8, _mpu(), "Weighted", PATTERNS)
    w2 = OfflineLoader(ds2, 8, _mpu(), "Weighted", PATTERNS)
    for _ in range(3):
        t1, x1 = next(w1)
        t2, x2 = next(w2)
        torch.cuda.synchronize()
        assert torch.equal(t1, t2)
        for x, y in zip(x1, x2):
            assert torch.equal(x, y)
