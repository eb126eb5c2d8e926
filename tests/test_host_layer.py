"""CPU tests of the host layer: the pybind `libgear.core` surface and the `gear` Python API,
written after the reference's own tests (tests/test_specs.py, test_table.py, test_sub.py)."""
import json
import os
import pickle as pkl
import random

import numpy as np
import pytest
import torch

import gear_amd
from gear_amd.dtypes import CVT_DTYPES_GEAR_TO_TORCH as CVT_GTT
from gear_amd.libgear import core as glibc
from gear_amd.specs import ColumnSpec, TableSpec

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.mark.parametrize(
    "shape, dtype, name",
    [
        ((3,), torch.bool, "bool"),
        ((3, 4), torch.uint8, "uint8"),
        ((3, 4, 5), torch.int8, "int8"),
        ((3, 4, 5, 6), torch.int32, "int32"),
        ((3, 4, 5, 6, 7), torch.int64, "int64"),
        ((3, 4, 5, 6, 7, 8), torch.float32, "float32"),
        ((3, 4, 5, 6, 7, 8, 9), torch.float64, "float64"),
    ],
)
class TestColumnSpec:
    """tests/test_specs.py:10-34 of the reference, unchanged in what it asserts."""

    def test_column_spec_build(self, shape, dtype, name):
        cspec = ColumnSpec.create(shape, dtype, name)
        assert tuple(cspec.shape) == shape
        assert CVT_GTT[cspec.dtype] == dtype
        assert cspec.name == name
        assert cspec.size() == int(np.prod(shape)) * torch.empty(0, dtype=dtype).element_size()

    def test_column_spec_pickle(self, shape, dtype, name):
        cspec = ColumnSpec.create(shape, dtype, name)
        rec = pkl.loads(pkl.dumps(cspec))
        assert cspec.shape == rec.shape and cspec.dtype == rec.dtype and cspec.name == rec.name


def _table_spec():
    return TableSpec.create(rank=0, worldsize=1, trajectory_length=100, capacity=1000,
                            column_specs=[{"shape": [3, 32], "dtype": glibc.float32, "name": "a"},
                                          {"shape": [1], "dtype": glibc.int32, "name": "b"}])


def test_dtype_enum_values_and_sizes():
    with open(os.path.join(GOLD, "reference_tests.json")) as f:
        sizes = json.load(f)["dtype_sizes"]
    for name, nbytes in sizes.items():
        assert glibc.sizeof_dtype(getattr(glibc, name)) == nbytes
    # integer values of the reference's enum (include/common/dtypes.h:18-28)
    assert [int(glibc.bool), int(glibc.int8), int(glibc.uint8), int(glibc.int16), int(glibc.int32),
            int(glibc.int64), int(glibc.float16), int(glibc.float32), int(glibc.float64)] == list(range(9))
    assert glibc.short == glibc.int16 and glibc.long == glibc.int64 and glibc.double == glibc.float64
    with pytest.raises(RuntimeError, match="Unsupported type"):
        glibc.ColumnSpec([2], glibc.float16, "h").size()


def test_table_spec_and_layout():
    tspec = _table_spec()
    assert tspec.size() == 38_800_000 and tspec.num_columns == 2
    assert tspec.index("b") == 1 and tspec.index("missing") == -1
    rec = pkl.loads(pkl.dumps(tspec))
    assert rec.size() == tspec.size() and rec.column_specs[0].name == "a"
    with pytest.raises(RuntimeError, match="mismatch"):
        glibc.TableSpec(0, 1, 10, 10, 3, [glibc.ColumnSpec([1], glibc.int32, "x")])
    table = glibc.TrajectoryTable(tspec, 7, True, "host")
    assert table.trajectory_stride == 38_800 and table.ncolumns == 2
    assert table.column_stride(0) == 384 and table.column_base(1) == 38_400


def test_table_pickle_round_trip():
    """tests/test_table.py of the reference: fill one view, pickle the table."""
    tspec = TableSpec.create(trajectory_length=10, capacity=8,
                             column_specs=[{"shape": [3, 2], "dtype": glibc.float32},
                                           {"shape": [1], "dtype": glibc.int32}])
    table = glibc.TrajectoryTable(tspec, 7, True, "host")
    assert table.connect() == tspec.size()
    handler = glibc.get_cpu_handler(table, 8, glibc.Range(0, 0), glibc.Range(0, 8))
    handler.view(0, 0).tensor().fill_(16)
    handler.view(5, 1).cast_tensor(glibc.int32).copy_(torch.arange(10, dtype=torch.int32))
    state = pkl.dumps(table)
    os.environ["GEAR_TABLE_PLACEMENT"] = "host"
    try:
        table2 = pkl.loads(state)
    finally:
        del os.environ["GEAR_TABLE_PLACEMENT"]
    h2 = glibc.get_cpu_handler(table2, 8, glibc.Range(0, 0), glibc.Range(0, 8))
    assert bool(torch.all(h2.view(0, 0).tensor() == 16))
    assert h2.view(5, 1).cast_tensor(glibc.int32).tolist() == list(range(10))
    assert not h2.view(1, 0).tensor().any()


def test_handler_sub_reference_vector():
    """tests/test_sub.py:10-28 of the reference through the bindings."""
    with open(os.path.join(GOLD, "reference_tests.json")) as f:
        v = json.load(f)["test_sub"]
    cspecs = [glibc.ColumnSpec([1, 2, 3, 4], glibc.float32, "x")]
    tspec = glibc.TableSpec(0, 1, 100, 32, 1, cspecs)
    table = glibc.TrajectoryTable(tspec, 7, True, "host")
    handler = glibc.get_cpu_handler(table, 32, glibc.Range(0, 0), glibc.Range(0, 32))
    handler.set([0], [glibc.SubscribePattern(-1, 100, glibc.SubscribePattern.PadOption.head)])
    indices = torch.arange(10, dtype=torch.long)
    lengths = torch.ones(10, dtype=torch.long) * 10
    so, do, cl = (torch.zeros(10, dtype=torch.long) for _ in range(3))
    ret = handler.sub(indices, indices.clone(), lengths, 0, so, do, cl)
    assert ret == v["expected_return"]
    assert so.tolist() == v["src_offsets"] and do.tolist() == v["dst_offsets"]
    assert cl.tolist() == v["copy_lens"]
    # explicit spans and sub_ give the same
    so2, do2, cl2 = (torch.zeros(10, dtype=torch.long) for _ in range(3))
    handler.sub_(indices, indices.clone(), lengths, 0, so2, do2, cl2)
    assert so2.tolist() == so.tolist()
    S = glibc.Int64Span.from_tensor
    handler.sub(S(indices), S(indices), S(lengths), 0, S(so2), S(do2), S(cl2))
    assert cl2.tolist() == cl.tolist()
    with pytest.raises(RuntimeError, match="SubscribePattern"):
        glibc.get_cpu_handler(table, 32, glibc.Range(0, 0), glibc.Range(0, 32)).sub(
            indices, indices, lengths, 0, so, do, cl)


def test_pattern_defaults_and_pickle():
    p = glibc.SubscribePattern(-3, 7)
    assert p.pad_option == glibc.SubscribePattern.PadOption.tail and p.offset == -3 and p.length == 7
    q = pkl.loads(pkl.dumps(glibc.SubscribePattern(1, 2, glibc.SubscribePattern.PadOption.head)))
    assert q.pad_option == glibc.SubscribePattern.PadOption.head
    assert "offset -3" in repr(p)


def test_spans():
    t = torch.arange(12, dtype=torch.float32)
    s = glibc.Float32Span.from_tensor(t)
    assert s.size == 12 and s.as_uint8().size == 48 and s.as_float64().size == 6
    assert torch.equal(s.tensor(), t)
    s.as_int32().tensor()[0] = 0x3F800000
    assert t[0] == 1.0                               # views alias the tensor's memory
    s.copy(torch.full((5,), 7.0))
    assert t[:5].tolist() == [7.0] * 5 and t[5] == 5.0
    assert glibc.Uint8Span.Tensor(s.as_uint8()).dtype == torch.uint8
    assert s.as_uint8().cast_tensor(glibc.int16).dtype == torch.int16


def test_indexset_state_layout():
    iset = glibc.Indexset(20, 10, 5)
    assert (iset.global_capacity, iset.local_capacity, iset.index_offset) == (20, 10, 5)
    iset.timesteps[:] = torch.arange(10) * 3
    iset.weights[:] = torch.arange(10, dtype=torch.float32) / 4
    iset.set_weight(2, 9.5)
    state = iset.get_state()
    off, local, glob, blob = state.__getstate__()
    assert (off, local, glob) == (5, 10, 20)
    blob = np.asarray(blob)
    assert blob.size == 10 * 12                    # timesteps int64[n] || weights fp32[n], packed
    assert blob[:80].view(np.int64).tolist() == [3 * i for i in range(10)]
    assert blob[80:].view(np.float32)[2] == 9.5
    rec = glibc.Indexset.load_state(pkl.loads(pkl.dumps(state)), False, 0, False)
    assert torch.equal(rec.timesteps, iset.timesteps) and torch.equal(rec.weights, iset.weights)
    with pytest.raises(IndexError):
        iset.set_weight(10, 1.0)


def test_shared_memory_attach_failure_returns_minus_one():
    key = random.Random(os.getpid()).randint(1 << 20, 1 << 30)
    shm = glibc.SharedMemory(key, 4096, False)      # nobody created it
    assert shm.alloc() == -1
    tspec = TableSpec.create(trajectory_length=4, capacity=2,
                             column_specs=[{"shape": [1], "dtype": glibc.int32}])
    assert glibc.TrajectoryTable(tspec, key, False, "shm").connect() == -1


def test_shared_dataset_items_and_checkpoint(tmp_path):
    from gear_amd.dataset import SharedDataset
    tspec = TableSpec.create(trajectory_length=6, capacity=5,
                             column_specs=[{"shape": [3], "dtype": torch.float32, "name": "obs"},
                                           {"shape": [], "dtype": torch.uint8, "name": "done"}])
    ds = SharedDataset.create(tspec, key=os.getpid(), placement="host")
    rng = torch.Generator().manual_seed(1)
    for i in range(5):
        obs = torch.rand((6, 3), generator=rng)
        done = torch.zeros(6, dtype=torch.uint8)
        done[i] = 1
        ds[i] = (0.5 + i, i + 1, [obs, done])
    e = ds[3]
    assert e.weight == 3.5 and e.timestep == 4 and e.column0.shape == (6, 3)
    assert e.column1.tolist() == [0, 0, 0, 1, 0, 0]
    path = tmp_path / "ckpt" / "ds.pt"
    ds.checkpoint(path)
    os.environ["GEAR_TABLE_PLACEMENT"] = "host"
    try:
        ds2 = SharedDataset().load(path, key=os.getpid() + 1)
    finally:
        del os.environ["GEAR_TABLE_PLACEMENT"]
    for i in range(5):
        a, b = ds[i], ds2[i]
        assert a.weight == b.weight and a.timestep == b.timestep
        assert torch.equal(a.column0, b.column0) and torch.equal(a.column1, b.column1)


def test_install_as_gear_aliases():
    import sys
    gear_amd.install_as_gear()
    import gear
    import libgear.core as lg
    from gear.sampler import TopKSampler, UniformSampler, WeightedSampler  # noqa: F401
    from gear.loader import OfflineLoader  # noqa: F401
    assert lg is glibc and gear is gear_amd and "gear.dataset" in sys.modules


def test_multi_rank_entry_points_refuse():
    tspec = TableSpec.create(trajectory_length=4, capacity=2,
                             column_specs=[{"shape": [1], "dtype": glibc.int32}])
    table = glibc.TrajectoryTable(tspec, 1, True, "host")
    h = glibc.get_cpu_handler(table, 2, glibc.Range(0, 0), glibc.Range(0, 2))
    with pytest.raises(RuntimeError, match="single-GPU"):
        h.connect(0, 2, b"x")
    with pytest.raises(RuntimeError, match="single-GPU"):
        h.subsend(1)


def test_checkpoint_stream_uses_reference_class_paths(tmp_path):
    """A checkpoint names `libgear.core.*` / `gear.dataset.shared_dataset.*` classes with the
    reference's state tuples (storage/pybind.cc:178-204, index/pybind.cc:15-50), so files written
    by either side unpickle on the other; a stream assembled by hand from those tuples loads."""
    import pickletools
    from gear_amd.dataset import SharedDataset
    gear_amd.install_as_gear()
    tspec = TableSpec.create(trajectory_length=4, capacity=3,
                             column_specs=[{"shape": [2], "dtype": torch.float32, "name": "x"}])
    ds = SharedDataset.create(tspec, key=4242, placement="host")
    for i in range(3):
        ds[i] = (1.0 + i, i + 1, [torch.full((4, 2), float(i))])
    path = tmp_path / "ref_style.pt"
    ds.checkpoint(path)
    names = set()
    with open(path, "rb") as f:
        data = f.read()
    for op, arg, _ in pickletools.genops(data):
        if op.name in ("GLOBAL", "STACK_GLOBAL") and arg:
            names.add(arg)
        if op.name in ("SHORT_BINUNICODE", "BINUNICODE") and isinstance(arg, str) and (
                arg.startswith("libgear") or arg.startswith("gear")):
            names.add(arg)
    assert "libgear.core" in names and "gear.dataset.shared_dataset" in names
    assert not any(n.startswith("gear_amd") for n in names)

    # hand-built stream in the reference's layout: meta, table 5-tuple, index-state 4-tuple
    import io
    table_bytes = np.arange(tspec.size(), dtype=np.uint8)
    ts = np.array([4, 3, 2], np.int64)
    w = np.array([0.5, 0.25, 2.0], np.float32)
    blob = np.concatenate([ts.view(np.uint8), w.view(np.uint8)])

    def from_state(cls, state):              # what unpickling does: __new__, then __setstate__
        obj = cls.__new__(cls)
        obj.__setstate__(state)
        return obj

    from gear_amd.dataset.shared_dataset import IndexMeta, SharedDatasetMeta
    os.environ["GEAR_TABLE_PLACEMENT"] = "host"
    try:
        table = from_state(glibc.TrajectoryTable, (tspec, 1234, int(tspec.size()), True, table_bytes))
    finally:
        del os.environ["GEAR_TABLE_PLACEMENT"]
    state = from_state(glibc.IndexsetState, (0, 3, 3, blob))
    buf = io.BytesIO()
    pk = pkl.Pickler(buf, protocol=2)
    pk.dump(SharedDatasetMeta(tspec, IndexMeta(3, 3, 0, False, 99)))
    pk.dump(table)
    pk.dump(state)
    p2 = tmp_path / "handmade.pt"
    p2.write_bytes(buf.getvalue())
    os.environ["GEAR_TABLE_PLACEMENT"] = "host"
    try:
        loaded = SharedDataset().load(p2, key=777)
    finally:
        del os.environ["GEAR_TABLE_PLACEMENT"]
    assert loaded.timesteps.tolist() == [4, 3, 2] and loaded.weights.tolist() == [0.5, 0.25, 2.0]
    assert loaded._handler.raw(0, int(tspec.size())).tensor().tolist() == table_bytes.tolist()


def test_weight_update_requests_dedupe_last_wins():
    """request.cc:41-75: one pending update per index (the last one), in order of first
    appearance; continuous() packs (index, timestep at +capacity, weight) and clears."""
    cache = glibc.CachedRequest(16)
    model = {}
    order = []
    rng = random.Random(3)
    for _ in range(60):
        i, ts, w = rng.randrange(16), rng.randrange(100), rng.random()
        cache.warr.update(i, ts, w)
        if i not in model:
            order.append(i)
        model[i] = (ts, np.float32(w))
    assert cache.warr.count == len(order)
    idxs = torch.zeros(32, dtype=torch.long)
    weights = torch.zeros(16, dtype=torch.float32)
    num = cache.continuous(idxs, weights)
    assert num == len(order)
    assert idxs[:num].tolist() == order
    assert idxs[16:16 + num].tolist() == [model[i][0] for i in order]
    assert weights[:num].tolist() == [float(model[i][1]) for i in order]
    assert cache.warr.count == 0 and cache.continuous(idxs, weights) == 0
    assert not any(cache.warr.updated_element_view(i) for i in range(16))
    with pytest.raises(RuntimeError, match="less space"):
        cache.warr.update(1, 1, 1.0)
        cache.continuous(torch.zeros(3, dtype=torch.long), weights)
    cache.iarr.insert(2, 7, 11)
    assert cache.iarr.count == 1 and cache.iarr.index_element_view(0) == 7
    assert cache.iarr.timestep_tensor_view().tolist() == [11]


def test_loader_partition_and_rank_order_on_one_rank():
    """OfflineLoader.partition_indices / generate_rank_comm_order
    (gear/loader/offline_loader.py:123-153) at a data-parallel world of 1: one slice with the
    whole batch, one shard, peer order [0]; indices outside the shard are dropped."""
    from gear_amd.dataset import SharedDataset
    from gear_amd.loader import OfflineLoader
    from gear_amd.loader.offline_loader import BasicLoader
    from gear_amd.mpu import ModelParallelismUnit
    tspec = TableSpec.create(trajectory_length=4, capacity=6,
                             column_specs=[{"shape": [2], "dtype": torch.float32, "name": "obs"}])
    ds = SharedDataset.create(tspec, key=os.getpid() + 77, placement="host")
    for i in range(6):
        ds[i] = (1.0, 4, [torch.full((4, 2), float(i))])
    loader = OfflineLoader(ds, 3, ModelParallelismUnit(device="cpu"), "Uniform",
                           [{"name": "obs", "offset": 0, "length": 4}])
    assert isinstance(loader, BasicLoader)
    # the base hooks are no-ops as in gear/loader/basic_loader.py:8-14, and OfflineLoader does
    # not override checkpoint: it returns None instead of raising
    assert loader.checkpoint() is None
    assert BasicLoader(3).__next__() is None
    parts = loader.partition_indices(torch.tensor([0, 5, 2, 9, -1, 3]))
    assert len(parts) == 1 and len(parts[0]) == 1
    assert parts[0][0].tolist() == [0, 5, 2, 3]
    assert loader.generate_rank_comm_order() == [0]
    gear_amd.install_as_gear()
    from gear.loader.basic_loader import BasicLoader as B2
    assert B2 is BasicLoader
    # the spelling the loader documents, "Topk" (gear/loader/offline_loader.py:44,61), finds the
    # top-k sampler through the "<method>Sampler" look-up (:102-104)
    import gear.sampler
    assert gear.sampler.TopkSampler is gear.sampler.TopKSampler
    topk_loader = OfflineLoader(ds, 3, ModelParallelismUnit(device="cpu"), "Topk",
                                [{"name": "obs", "offset": 0, "length": 4}])
    assert isinstance(topk_loader._sampler, gear.sampler.TopKSampler)


def test_host_code_is_clean_under_address_and_ub_sanitizers(request):
    """The host C++ layer and the oracle rebuilt with -fsanitize=address,undefined and run under
    the CPU tests of this directory (tests/host_sanitizers.py); opt-in: pytest --host-sanitizers."""
    if not request.config.getoption("--host-sanitizers"):
        pytest.skip("run with --host-sanitizers (rebuilds the host code with ASan + UBSan)")
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "tests", "host_sanitizers.py")],
                       cwd=root, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert r.returncode == 0, r.stdout[-4000:]
