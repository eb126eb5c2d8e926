"""GPU parity against the committed golden fixtures (tests/golden/*.npz), through the C ABI."""
import os

import numpy as np
import pytest

from conftest import announce

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_gather_fixture_on_gpu():
    from gear_amd import ops
    z = np.load(os.path.join(GOLD, "gather_small.npz"))
    sb = z["step_bytes"]
    T = int(z["T"])
    accu = np.concatenate([[0], np.cumsum(sb)])
    stride = int(accu[-1]) * T
    table = _dev(z["table"])
    di, dt, dl = _dev(z["idxs"]), _dev(z["tss"]), _dev(z["lens"])
    B = len(z["idxs"])
    for ci, (ofst, span, pad_head) in enumerate(z["cases"]):
        announce("golden gather case %d" % ci)
        dsts, masks, cols = [], [], []
        for c in range(len(sb)):
            dsts.append(torch.full((B, int(span) * int(sb[c])), 0x77, dtype=torch.uint8, device="cuda"))
            masks.append(torch.full((B, int(span)), 3, dtype=torch.uint8, device="cuda"))
            cols.append(dict(dst=dsts[c], mask_out=masks[c], ofst=int(ofst), span=int(span),
                             step_bytes=int(sb[c]), col_base=int(accu[c]) * T,
                             pad_head=bool(pad_head)))
        ops.subcopy_multi(table, di, dt, dl, stride, cols)
        torch.cuda.synchronize()
        for c in range(len(sb)):
            assert np.array_equal(dsts[c].cpu().numpy(), z["dst_%d_%d" % (ci, c)])
            assert np.array_equal(masks[c].cpu().numpy(), z["mask_%d_%d" % (ci, c)])


def test_sampler_fixture_on_gpu():
    from gear_amd import ops
    z = np.load(os.path.join(GOLD, "sampler_small.npz"))
    announce("golden scan/search/weights")
    dp = _dev(z["p"])
    prefix = ops.prefix_sum(dp)
    got = prefix.cpu().numpy()
    assert np.max(np.abs(got - z["prefix"]) / np.maximum(z["prefix"], 1e-300)) <= 1e-12
    assert np.array_equal(ops.prefix_sum(_dev(z["pint"])).cpu().numpy(), z["pint_prefix"])
    idx, w = ops.upper_bound(prefix, _dev(z["u"]), priorities=dp, beta=0.4)
    assert np.array_equal(idx.cpu().numpy(), z["idx"])
    ulp = np.spacing(z["is_weights"])
    assert np.all(np.abs(w.cpu().numpy() - z["is_weights"]) <= ulp)
    announce("golden top-k / sort / scatter")
    vals, tidx = ops.topk(dp, int(z["topk_k"]))
    assert np.array_equal(tidx.cpu().numpy(), z["topk_idx"])
    assert np.array_equal(vals.cpu().numpy(), z["topk_val"])
    _, tidx = ops.topk(_dev(z["ties"]), 1500)
    assert np.array_equal(tidx.cpu().numpy(), z["ties_idx"])
    ko, vo = ops.sort_i64(_dev(z["sort_keys"]), _dev(z["sort_vals"]), key_bits=20)
    assert np.array_equal(ko.cpu().numpy(), z["sorted_keys"])
    assert np.array_equal(vo.cpu().numpy(), z["sorted_vals"])
    w0 = _dev(z["scatter_w0"])
    ops.scatter(w0, _dev(z["scatter_idx"]), _dev(z["scatter_val"]), unique_indices=False)
    assert np.array_equal(w0.cpu().numpy(), z["scatter_w1"])
