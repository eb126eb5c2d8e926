"""benchmark config 3 end to end: length-weighted int64 sampler -> length look-up -> start offsets
-> 5-column window gather with a uint8 attention mask (Decision-Transformer windows).

  * full size: 100 000 variable-length trajectories (T = 1000, 104 bytes per step, 10.4 GB in HBM);
    the drawn trajectories are checked against the oracle's sampler and every gathered window
    against torch indexing of the same table on the device;
  * the padding edge: start offsets up to len - 1 (windows that run past the trajectory's end are
    tail-padded with zeros, their mask 0 there), 1000 trajectories, every byte against the oracle.
"""
import numpy as np
import pytest

from conftest import announce
from helpers import Schema

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

CFG3 = [("obs", "float32", (17,)), ("act", "float32", (6,)), ("rew", "float32", ()),
        ("rtg", "float32", ()), ("ts", "int32", ())]
B, SPAN = 1024, 20


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _chain(ops, table, lengths, u1, u2, schema, dsts, mask, full_windows):
    """The device-side chain of one batch; returns (traj, start, lens) tensors."""
    prefix = ops.prefix_sum_i64(lengths)
    traj = ops.sort_i64(ops.upper_bound_i64(prefix, u1, unit_uniforms=True), key_bits=17)
    lens = ops.take_i64(lengths, traj)
    room = (lens - (SPAN - 1)) if full_windows else lens      # start in [0, len-20] or [0, len-1]
    start = (u2 * room.double()).long()
    cols = [dict(dst=dsts[c], ofst=0, span=SPAN, step_bytes=schema.step_bytes[c],
                 col_base=schema.col_base(c), pad_head=False, zero_fill=True,
                 mask_out=mask if c == 0 else None) for c in range(5)]
    ops.subcopy_multi(table, traj, start, lens, schema.traj_stride, cols)
    return traj, start, lens


def test_config3_full_size_chain(oracle):
    from gear_amd import ops
    schema = Schema(CFG3, T=1000, capacity=100_000)
    free, _ = torch.cuda.mem_get_info()
    if free < schema.nbytes + (4 << 30):
        pytest.skip("not enough free HBM for the 10.4 GB table")
    announce("config3 full size: building the 10.4 GB table")
    g = torch.Generator(device="cuda")
    g.manual_seed(1003)
    table = torch.empty(schema.nbytes, dtype=torch.uint8, device="cuda")
    piece = 1 << 30
    for o in range(0, schema.nbytes, piece):
        n = min(piece, schema.nbytes - o)
        table[o:o + n] = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    rng = np.random.default_rng(1003)
    lengths_h = rng.integers(200, 1001, size=schema.capacity).astype(np.int64)
    lengths = _dev(lengths_h)
    dsts = [torch.empty((B, SPAN * sb), dtype=torch.uint8, device="cuda")
            for sb in schema.step_bytes]
    mask = torch.empty((B, SPAN), dtype=torch.uint8, device="cuda")
    for it in range(3):
        u1, u2 = rng.random(B), rng.random(B)
        for d in dsts:
            d.fill_(0x5A)
        mask.fill_(7)
        announce("config3 full size: batch %d" % it)
        traj, start, lens = _chain(ops, table, lengths, _dev(u1), _dev(u2), schema, dsts, mask,
                                   full_windows=True)
        torch.cuda.synchronize()
        # the sampler: exact integer prefix, exact search, sorted
        pre = oracle.scan_i64(lengths_h)
        assert np.array_equal(pre, np.cumsum(lengths_h))
        e_traj = np.sort(oracle.upper_bound_i64(pre, u1, unit_uniforms=True))
        assert np.array_equal(traj.cpu().numpy(), e_traj)
        e_len = lengths_h[e_traj]
        assert np.array_equal(lens.cpu().numpy(), e_len)
        e_start = (u2 * (e_len - (SPAN - 1)).astype(np.float64)).astype(np.int64)
        assert np.array_equal(start.cpu().numpy(), e_start)
        assert (e_start + SPAN <= e_len).all() and (e_start >= 0).all()
        # every window of every column against the table itself
        for c in range(5):
            sb = schema.step_bytes[c]
            first = traj * schema.traj_stride + schema.col_base(c) + start * sb
            want = table[first[:, None] + torch.arange(SPAN * sb, device="cuda")[None, :]]
            assert torch.equal(dsts[c], want), "batch %d column %d" % (it, c)
        assert bool((mask == 1).all())


def test_config3_padding_edge_against_the_oracle(oracle):
    from gear_amd import ops
    schema = Schema(CFG3, T=1000, capacity=1000)
    rng = np.random.default_rng(3003)
    table_h = rng.integers(0, 256, size=schema.nbytes, dtype=np.uint8)
    lengths_h = rng.integers(200, 1001, size=schema.capacity).astype(np.int64)
    table, lengths = _dev(table_h), _dev(lengths_h)
    dsts = [torch.empty((B, SPAN * sb), dtype=torch.uint8, device="cuda")
            for sb in schema.step_bytes]
    mask = torch.empty((B, SPAN), dtype=torch.uint8, device="cuda")
    u1, u2 = rng.random(B), rng.random(B)
    u2[:8] = [0.0, 0.999999999, 0.9999, 0.98, 0.5, 0.97, 0.99, 0.995]   # starts at both ends
    for d in dsts:
        d.fill_(0x5A)
    mask.fill_(7)
    announce("config3 padding edge: starts up to len - 1")
    traj, start, lens = _chain(ops, table, lengths, _dev(u1), _dev(u2), schema, dsts, mask,
                               full_windows=False)
    torch.cuda.synchronize()
    e_traj = np.sort(oracle.upper_bound_i64(oracle.scan_i64(lengths_h), u1, unit_uniforms=True))
    e_len = lengths_h[e_traj]
    e_start = (u2 * e_len.astype(np.float64)).astype(np.int64)
    assert np.array_equal(traj.cpu().numpy(), e_traj)
    assert np.array_equal(start.cpu().numpy(), e_start)
    short = e_start + SPAN > e_len
    assert short.sum() >= 8                      # windows that run past the end exist
    for c in range(5):
        exp, emask = oracle.subcopy(table_h, e_traj, e_start, e_len, False, 0, SPAN,
                                    schema.traj_stride, schema.step_bytes[c], schema.col_base(c),
                                    want_mask=True)
        assert np.array_equal(dsts[c].cpu().numpy(), exp), "column %d" % c
        if c == 0:
            assert np.array_equal(mask.cpu().numpy(), emask)
            steps = np.minimum(e_len - e_start, SPAN)
            assert np.array_equal(emask.sum(axis=1), steps)
            assert not exp.reshape(B, SPAN, -1)[short][:, -1].any()   # last step of a short window is padding
