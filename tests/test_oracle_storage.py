"""CPU tests: the oracle's table layout, sub() arithmetic and gathers against the vectors that
the reference's own tests imply (tests/golden/reference_tests.json) and independent numpy code."""
import itertools
import json
import os

import numpy as np
import pytest

from helpers import Schema, fill_random, numpy_window_gather

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def ref():
    with open(os.path.join(GOLD, "reference_tests.json")) as f:
        return json.load(f)


def test_layout_matches_reference_table_test(oracle, ref):
    t = ref["test_table"]
    accu, stride, total = oracle.layout(t["step_bytes"], t["trajectory_length"], t["capacity"])
    assert list(accu) == t["accu"]
    assert stride == t["traj_stride"] == 38800
    assert total == t["table_bytes"] == 38_800_000


def test_layout_brute_force_addresses(oracle):
    """Write a distinct tag per (trajectory, column, step) through the address formula and read it
    back through an independent numpy view of the same bytes."""
    cols = [("a", "float32", (3,)), ("b", "uint8", ()), ("c", "int64", (2,)), ("d", "int16", (5,))]
    schema = Schema(cols, T=7, capacity=5)
    accu, stride, total = oracle.layout(schema.step_bytes, 7, 5)
    assert total == schema.nbytes and stride == schema.traj_stride
    table = np.zeros(total, np.uint8)
    for i, c, t in itertools.product(range(5), range(4), range(7)):
        a = i * stride + accu[c] * 7 + t * schema.step_bytes[c]
        assert np.all(table[a:a + schema.step_bytes[c]] == 0)      # never written twice
        table[a:a + schema.step_bytes[c]] = 1 + (i * 28 + c * 7 + t) % 255
    assert np.all(table != 0)                                       # no gaps, no padding
    for c in range(4):
        rows, _, _ = schema.column_view(table, c)
        sb = schema.step_bytes[c]
        for i, t in itertools.product(range(5), range(7)):
            assert np.all(rows[i, t * sb:(t + 1) * sb] == 1 + (i * 28 + c * 7 + t) % 255)


def test_sub_reference_hand_vector(oracle, ref):
    v = ref["test_sub"]
    so, do, cl, exp = oracle.sub(v["indices"], v["timesteps"], v["lengths"], v["pad"] == "head",
                                 v["offset"], v["length"], v["traj_stride"], v["step_bytes"], 0)
    assert exp == v["expected_return"]
    assert list(cl) == v["copy_lens"]
    assert list(so) == v["src_offsets"]
    assert list(do) == v["dst_offsets"]


def test_sub_brute_force_small(oracle):
    """Every (ts, len, offset, span, pad) on T <= 8, against list slicing of the step range."""
    T, sb, col_base, stride = 8, 5, 24, 8 * 11
    for pad_head in (False, True):
        for ofst in range(-10, 4):
            for span in range(1, 10):
                cases = [(i % 3, ts, ln) for i, (ts, ln) in
                         enumerate(itertools.product(range(0, 10), range(0, T + 1)))]
                idx = [c[0] for c in cases]
                tss = [c[1] for c in cases]
                lens = [c[2] for c in cases]
                so, do, cl, exp = oracle.sub(idx, tss, lens, pad_head, ofst, span, stride, sb,
                                             col_base)
                assert exp == span * sb
                for g, (i, ts, ln) in enumerate(cases):
                    steps = list(range(ln))[max(ts + ofst, 0):][:span]
                    assert cl[g] == len(steps) * sb
                    if steps:
                        assert so[g] == i * stride + col_base + steps[0] * sb
                    want = g * span * sb + ((span - len(steps)) * sb if pad_head else 0)
                    assert do[g] == want


def test_subcopy_equals_sub_plus_vcopy_on_zeroed_batch(oracle):
    """handler.subcopy == handler.sub + vcopy into a torch.zeros batch (the two loader paths of
    gear/loader/offline_loader.py:155-204 and :206-278 must agree)."""
    cols = [("obs", "float32", (17,)), ("done", "uint8", ())]
    schema = Schema(cols, T=20, capacity=11)
    table = fill_random(schema, 3)
    rng = np.random.default_rng(3)
    B = 64
    idxs = rng.integers(0, 11, size=B)
    lens = rng.integers(0, 21, size=B)
    tss = rng.integers(0, 22, size=B)
    for c, pad_head, ofst, span in itertools.product(range(2), (False, True), (-4, 0, 2), (1, 6)):
        sb = schema.step_bytes[c]
        fused, _ = oracle.subcopy(table, idxs, tss, lens, pad_head, ofst, span,
                                  schema.traj_stride, sb, schema.col_base(c))
        so, do, cl, exp = oracle.sub(idxs, tss, lens, pad_head, ofst, span, schema.traj_stride,
                                     sb, schema.col_base(c))
        two_step = oracle.vcopy(table, np.zeros(B * exp, np.uint8), so, do, cl).reshape(B, exp)
        assert np.array_equal(fused, two_step)
        ref, _ = numpy_window_gather(schema, table, c, idxs, tss, lens, ofst, span, pad_head)
        assert np.array_equal(fused, ref)


def test_gather_fixture(oracle):
    z = np.load(os.path.join(GOLD, "gather_small.npz"))
    sb = z["step_bytes"]
    T = int(z["T"])
    accu = np.concatenate([[0], np.cumsum(sb)])
    stride = int(accu[-1]) * T
    for ci, (ofst, span, pad_head) in enumerate(z["cases"]):
        for c in range(len(sb)):
            dst, mask = oracle.subcopy(z["table"], z["idxs"], z["tss"], z["lens"], bool(pad_head),
                                       int(ofst), int(span), stride, int(sb[c]), int(accu[c]) * T,
                                       want_mask=True)
            assert np.array_equal(dst, z["dst_%d_%d" % (ci, c)])
            assert np.array_equal(mask, z["mask_%d_%d" % (ci, c)])


def test_integrity_invariant_of_reference_example(oracle):
    """examples/offline/single-node/misc.py:16-29: gathering every trajectory with pattern
    (offset=-L, length=L) and timestep == length returns gathered[i][:len_i] == raw[i][:len_i]
    for tail padding... with head padding the data sits at the end: gathered[i][L-len_i:]."""
    cols = [("observations", "float32", (11,)), ("actions", "float32", (3,))]
    L = 30
    schema = Schema(cols, T=L, capacity=16)
    table = fill_random(schema, 5)
    rng = np.random.default_rng(5)
    lens = rng.integers(1, L + 1, size=16)
    idxs = np.arange(16)
    for c in range(2):
        sb = schema.step_bytes[c]
        rows, _, _ = schema.column_view(table, c)
        tail, _ = oracle.subcopy(table, idxs, lens, lens, False, -L, L, schema.traj_stride, sb,
                                 schema.col_base(c))
        head, _ = oracle.subcopy(table, idxs, lens, lens, True, -L, L, schema.traj_stride, sb,
                                 schema.col_base(c))
        for i in range(16):
            n = int(lens[i]) * sb
            assert np.array_equal(tail[i, :n], rows[i, :n]) and not tail[i, n:].any()
            assert np.array_equal(head[i, L * sb - n:], rows[i, :n]) and not head[i, :L * sb - n].any()


def test_reference_copy_test_ones(oracle):
    """tests/test_copy.py: ones[32,100,4,3,2] fp32, one 960-byte slice at offset 0 -> all ones."""
    data = np.ones((32, 100, 4, 3, 2), np.float32)
    dst = np.zeros(10 * 24, np.float32)
    oracle.vcopy(data.view(np.uint8).reshape(-1), dst.view(np.uint8), [0], [0], [960])
    assert np.all(dst == 1.0)


def test_zero_fill_flag(oracle):
    schema = Schema([("x", "uint8", (3,))], T=6, capacity=4)
    table = fill_random(schema, 8)
    pre = np.full((3, 12), 0xEE, np.uint8)
    dst, _ = oracle.subcopy(table, [0, 1, 2], [0, 5, 9], [6, 6, 6], True, 0, 4, schema.traj_stride,
                            3, 0, zero_fill=False, dst=pre.copy())
    ref, mask = numpy_window_gather(schema, table, 0, [0, 1, 2], [0, 5, 9], [6, 6, 6], 0, 4, True)
    keep = np.repeat(mask, 3, axis=1).astype(bool)
    assert np.array_equal(dst[keep], ref[keep])
    assert np.all(dst[~keep] == 0xEE)


def test_subcopy_threads_equal_single_thread(oracle):
    """The all-cores leg of the CPU baseline splits the windows over threads: same bytes, same mask."""
    rng = np.random.default_rng(77)
    T, cap, sb = 16, 9, 7
    stride = T * (sb + 3)
    table = rng.integers(0, 256, size=cap * stride, dtype=np.uint8)
    n = 37
    idxs = rng.integers(0, cap, size=n).astype(np.int64)
    lens = rng.integers(0, T + 1, size=n).astype(np.int64)
    tss = rng.integers(0, T, size=n).astype(np.int64)
    for pad_head in (False, True):
        a, ma = oracle.subcopy(table, idxs, tss, lens, pad_head, -3, 6, stride, sb, 0, want_mask=True)
        for threads in (2, 5, 64):
            b, mb = oracle.subcopy(table, idxs, tss, lens, pad_head, -3, 6, stride, sb, 0,
                                   want_mask=True, threads=threads)
            assert np.array_equal(a, b) and np.array_equal(ma, mb)
