"""Randomised differential test of the gather entry points: random schemas (1..16 columns, odd
byte sizes), window patterns, batch sizes and destination strides, against the numpy gather."""
import numpy as np
import pytest

from conftest import announce
from helpers import Schema, fill_random, numpy_window_gather

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

DTYPES = [("uint8", 1), ("int16", 2), ("float32", 4), ("int64", 8)]


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("seed", list(range(12)))
def test_random_schemas_and_patterns(oracle, seed):
    from gear_amd import ops
    rng = np.random.default_rng(1000 + seed)
    ncol = int(rng.integers(1, 17))
    cols = []
    for c in range(ncol):
        name, _ = DTYPES[int(rng.integers(0, len(DTYPES)))]
        shape = tuple(int(x) for x in rng.integers(1, 6, size=int(rng.integers(0, 3))))
        cols.append(("c%d" % c, name, shape))
    T = int(rng.integers(1, 60))
    cap = int(rng.integers(1, 40))
    schema = Schema(cols, T, cap)
    table = fill_random(schema, seed)
    B = int(rng.integers(1, 700))
    idxs = rng.integers(0, cap, size=B).astype(np.int64)
    lens = rng.integers(0, T + 1, size=B).astype(np.int64)
    tss = rng.integers(0, T + 2, size=B).astype(np.int64)
    tdev, di, dt, dl = _dev(table), _dev(idxs), _dev(tss), _dev(lens)
    descs, expect = [], []
    for c in range(ncol):
        span = int(rng.integers(1, T + 3))
        ofst = int(rng.integers(-T - 2, 4))
        pad_head = bool(rng.integers(0, 2))
        sb = schema.step_bytes[c]
        dst = torch.full((B, span * sb), 0xA5, dtype=torch.uint8, device="cuda")
        mask = torch.full((B, span), 5, dtype=torch.uint8, device="cuda")
        descs.append(dict(dst=dst, mask_out=mask, ofst=ofst, span=span, step_bytes=sb,
                          col_base=schema.col_base(c), pad_head=pad_head))
        expect.append(numpy_window_gather(schema, table, c, idxs, tss, lens, ofst, span, pad_head))
    announce("random gather seed=%d ncol=%d T=%d cap=%d B=%d" % (seed, ncol, T, cap, B))
    ops.subcopy_multi(tdev, di, dt, dl, schema.traj_stride, descs)
    torch.cuda.synchronize()
    for c in range(ncol):
        assert np.array_equal(descs[c]["dst"].cpu().numpy(), expect[c][0]), "column %d" % c
        assert np.array_equal(descs[c]["mask_out"].cpu().numpy(), expect[c][1]), "mask %d" % c
    # per-column entry point without zero fill, into a wider destination stride
    c = int(rng.integers(0, ncol))
    d = descs[c]
    extra = int(rng.integers(0, 40))
    stride = d["span"] * d["step_bytes"] + extra
    dst = torch.full((B, stride), 0x3C, dtype=torch.uint8, device="cuda")
    ops.subcopy(tdev, dst, di, dt, dl, pad_head=d["pad_head"], ofst=d["ofst"], span=d["span"],
                traj_stride=schema.traj_stride, step_bytes=d["step_bytes"],
                col_base=d["col_base"], zero_fill=False, dst_stride=stride)
    torch.cuda.synchronize()
    pre = np.full((B, stride), 0x3C, np.uint8)
    exp, _ = oracle.subcopy(table, idxs, tss, lens, d["pad_head"], d["ofst"], d["span"],
                            schema.traj_stride, d["step_bytes"], d["col_base"],
                            dst_stride=stride, zero_fill=False, dst=pre)
    assert np.array_equal(dst.cpu().numpy(), exp)


def test_offsets_beyond_32_bits():
    """Trajectory offsets above 2^31 and 2^32 (the reference's kernel keeps them in `int`)."""
    from gear_amd import ops
    free, _ = torch.cuda.mem_get_info()
    if free < (7 << 30):
        pytest.skip("needs 6 GiB of free HBM")
    sb, T = 4096, 64                     # 256 KiB per trajectory
    cap = 5 * 4096                       # 5 GiB table
    table = torch.empty(cap * T * sb, dtype=torch.uint8, device="cuda")
    probe = [0, 8191, 8192, 16383, 16384, cap - 1]   # around 2 GiB and 4 GiB
    for i in probe:
        table[i * T * sb:(i + 1) * T * sb] = torch.arange(T * sb, device="cuda").to(torch.uint8) + (i % 251)
    idxs = torch.tensor(probe, dtype=torch.int64, device="cuda")
    tss = torch.tensor([0, 3, 60, 63, 10, 1], dtype=torch.int64, device="cuda")
    lens = torch.full((6,), T, dtype=torch.int64, device="cuda")
    dst = torch.empty((6, 2 * sb), dtype=torch.uint8, device="cuda")
    announce("gather with 64-bit offsets")
    ops.subcopy(table, dst, idxs, tss, lens, pad_head=False, ofst=0, span=2, traj_stride=T * sb,
                step_bytes=sb, col_base=0)
    torch.cuda.synchronize()
    for g, i in enumerate(probe):
        t0 = int(tss[g])
        steps = min(2, T - t0)
        a = i * T * sb + t0 * sb
        assert torch.equal(dst[g, :steps * sb], table[a:a + steps * sb])
        assert not dst[g, steps * sb:].any()
