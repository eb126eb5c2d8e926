"""The whole sample -> gather step captured into a HIP graph and replayed: every kernel of the
path (descriptor init kernels instead of memsets, tickets, agent-scope descriptor polling) must
give the eager result on every replay, with eager work between the replays."""
import numpy as np
import pytest

from conftest import announce
from helpers import Schema, fill_random

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu


def test_step_graph_replays_match_eager(oracle):
    from gear_amd import ops
    schema = Schema([("obs", "uint8", (4, 21, 21)), ("act", "int32", ()), ("done", "uint8", ())],
                    T=100, capacity=200)
    table_np = fill_random(schema, 77)
    table = torch.from_numpy(table_np).cuda()
    n = 200 * 100
    rng = np.random.default_rng(77)
    pri_np = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    pri = torch.from_numpy(pri_np).cuda()
    B, span = 512, 30
    u = torch.empty(B, dtype=torch.float32, device="cuda")
    prefix = torch.empty(n, dtype=torch.float64, device="cuda")
    flat, idxs, tss, lens = (torch.empty(B, dtype=torch.int64, device="cuda") for _ in range(4))
    dsts = [torch.empty((B, span * sb), dtype=torch.uint8, device="cuda") for sb in schema.step_bytes]
    cols = [dict(dst=dsts[c], ofst=-29, span=span, step_bytes=schema.step_bytes[c],
                 col_base=schema.col_base(c), pad_head=True) for c in range(3)]
    topv = torch.empty(64, dtype=torch.float32, device="cuda")

    def step():
        ops.prefix_sum(pri, out=prefix)
        ops.sample_sorted(prefix, u, unit_uniforms=True, sorted_out=flat, trajectory_length=100,
                          idxs=idxs, tss=tss, lens=lens)
        ops.subcopy_multi(table, idxs, tss, lens, schema.traj_stride, cols)
        v, _ = ops.topk(pri, 64, sorted_by_value=True)
        topv.copy_(v)

    side = torch.cuda.Stream()
    with torch.cuda.stream(side):          # warm-up on the capture stream: workspaces get allocated
        u.uniform_()
        step()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    announce("capturing the step")
    with torch.cuda.graph(graph, stream=side):
        step()
    for it in range(4):
        u.copy_(torch.from_numpy(rng.random(B, dtype=np.float32)))
        if it == 2:                         # the priorities change between replays too
            pri.mul_(torch.from_numpy(rng.random(n, dtype=np.float32) + 0.5).cuda())
        for d in dsts:
            d.fill_(0xEE)                   # eager work between the replays
        torch.cuda.synchronize()
        announce("replay %d" % it)
        graph.replay()
        torch.cuda.synchronize()
        p_now = pri.cpu().numpy()
        pre = prefix.cpu().numpy()
        exp_pre = oracle.scan_f32_f64(p_now)
        assert np.max(np.abs(pre - exp_pre) / exp_pre) <= 1e-12
        exp_flat = np.sort(oracle.upper_bound_f64(pre, u.cpu().numpy(), unit_uniforms=True))
        assert np.array_equal(flat.cpu().numpy(), exp_flat)
        ti, tt = exp_flat // 100, exp_flat % 100
        for c in range(3):
            exp, _ = oracle.subcopy(table_np, ti, tt, tt + 1, True, -29, span, schema.traj_stride,
                                    schema.step_bytes[c], schema.col_base(c))
            assert np.array_equal(dsts[c].cpu().numpy(), exp), "replay %d column %d" % (it, c)
        assert np.array_equal(topv.cpu().numpy(), oracle.topk_f32(p_now, 64, True)[0])
