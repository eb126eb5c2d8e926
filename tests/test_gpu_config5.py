"""benchmark config 5 as a workload, bit-exact against the CPU oracle for three consecutive steps:

    scatter 65 536 new priorities into a 10 000 000-entry array  (src/index/request.cc:41-51)
    -> value-ordered top-65 536                                   (global_sampler.py:195-199)
    -> full fp64 rescan -> 2048 seeded draws, sorted, folded onto the table's steps
    -> (-29, 30, head) gather of all four Atari-shape columns THROUGH THE DEVICE ALIAS OF A
       PINNED HOST TABLE: the kernel reads host memory in place, which is the reference's default
       placement (src/memory/shared_memory.cc:35-63 + src/storage/handler.cc:133-154).

The table holds 128 trajectories of 1000 steps (3.61 GB of the 56.5 GB the config names: the
kernels do not depend on the table's size, the host link does the same work per window)."""
import ctypes

import numpy as np
import pytest

from conftest import announce

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

STEP_BYTES = [4 * 84 * 84, 4, 4, 1]       # obs uint8[4,84,84], action int32, reward fp32, done uint8
T, CAP, B, SPAN, OFST = 1000, 128, 2048, 30, -29
NPRI, K, M = 10_000_000, 65_536, 65_536


def _fill_host_table(lib, host, rng):
    """Typed content per column as the config states; obs bytes come from a seeded device
    generator in 512 MiB pieces (host-side generation of 3.6 GB would dominate the test)."""
    from gear_amd import _cabi
    row = sum(STEP_BYTES)
    S = row * T
    g = torch.Generator(device="cuda")
    g.manual_seed(5005)
    obs_bytes = STEP_BYTES[0] * T
    per_piece = 16                                    # trajectories per device piece
    for i0 in range(0, CAP, per_piece):
        piece = torch.randint(0, 256, (per_piece * obs_bytes,), dtype=torch.uint8, device="cuda",
                              generator=g)
        for j in range(per_piece):
            dst = host.ctypes.data + (i0 + j) * S
            _cabi.call("gear_hip_memcpy", ctypes.c_void_p(dst),
                       ctypes.c_void_p(piece.data_ptr() + j * obs_bytes), obs_bytes)
    torch.cuda.synchronize()
    traj = host.reshape(CAP, S)
    o = obs_bytes
    traj[:, o:o + 4 * T] = rng.integers(0, 18, size=(CAP, T), dtype=np.int32).view(np.uint8)
    o += 4 * T
    traj[:, o:o + 4 * T] = rng.integers(-1, 2, size=(CAP, T)).astype(np.float32).view(np.uint8)
    o += 4 * T
    traj[:, o:o + T] = (rng.random((CAP, T)) < 0.001).astype(np.uint8)


def test_config5_workload_three_steps_against_the_oracle(oracle):
    from gear_amd import _cabi, ops
    lib = _cabi.load()
    row = sum(STEP_BYTES)
    S = row * T
    nbytes = S * CAP
    accu = np.concatenate([[0], np.cumsum(STEP_BYTES)])
    host_ptr, dev_ptr = ctypes.c_void_p(), ctypes.c_void_p()
    announce("config 5: pinning a %.2f GB host table" % (nbytes / 1e9))
    assert lib.gear_hip_host_alloc(nbytes, ctypes.byref(host_ptr), ctypes.byref(dev_ptr)) == 0
    try:
        host = np.ctypeslib.as_array(ctypes.cast(host_ptr, ctypes.POINTER(ctypes.c_uint8)),
                                     shape=(nbytes,))
        rng = np.random.default_rng(1005)
        _fill_host_table(lib, host, rng)
        pri_host = (rng.lognormal(0, 1, size=NPRI) ** 0.6).astype(np.float32)
        pri = torch.from_numpy(pri_host.copy()).cuda()
        prefix = torch.empty(NPRI, dtype=torch.float64, device="cuda")
        dsts = [torch.empty((B, SPAN * sb), dtype=torch.uint8, device="cuda") for sb in STEP_BYTES]
        cols = [dict(dst=dsts[c], ofst=OFST, span=SPAN, step_bytes=STEP_BYTES[c],
                     col_base=int(accu[c]) * T, pad_head=True, zero_fill=True) for c in range(4)]
        near_edge = 0
        selection = ops.TopKState()      # steps after the first start from the last step's bound
        for step in range(3):
            upd_idx = rng.permutation(NPRI)[:M].astype(np.int64)        # unique indices
            upd_val = (rng.lognormal(0, 1, size=M) ** 0.6).astype(np.float32)
            u01 = rng.random(B, dtype=np.float32)
            for d in dsts:
                d.fill_(0xA5)                                           # no stale zeros to hide behind
            announce("config 5 step %d: scatter -> top-k -> rescan -> draw -> host-table gather" % step)
            ops.scatter(pri, torch.from_numpy(upd_idx).cuda(), torch.from_numpy(upd_val).cuda(),
                        unique_indices=True)
            vals, tidx = selection.select(pri, K, sorted_by_value=True)
            ops.prefix_sum(pri, out=prefix)
            flat, idxs, tss, lens = ops.sample_sorted(prefix, torch.from_numpy(u01).cuda(),
                                                      unit_uniforms=True, trajectory_length=T,
                                                      modulo=T * CAP)
            ops.subcopy_multi(dev_ptr.value, idxs, tss, lens, S, cols)
            torch.cuda.synchronize()

            # priorities after the update
            oracle.scatter_f32(pri_host, upd_idx, upd_val)
            assert np.array_equal(pri.cpu().numpy(), pri_host)
            # value-ordered top-k: values bit for bit, indices with the smaller-index tie rule
            evals, eidx = oracle.topk_f32(pri_host, K, True)
            assert np.array_equal(tidx.cpu().numpy(), eidx)
            assert np.array_equal(vals.cpu().numpy().view(np.uint32), evals.view(np.uint32))
            # fp64 prefix: within 1e-12 of the sequential sum
            got_prefix = prefix.cpu().numpy()
            seq = oracle.scan_f32_f64(pri_host)
            assert np.max(np.abs(got_prefix - seq) / seq) <= 1e-12
            # draws: exact against the search of the same prefix, and against the sequential
            # prefix except for draws within 1e-9 (relative to the total) of a bucket edge
            exp_flat = np.sort(oracle.upper_bound_f64(got_prefix, u01, unit_uniforms=True))
            assert np.array_equal(flat.cpu().numpy(), exp_flat)
            seq_flat = np.sort(oracle.upper_bound_f64(seq, u01, unit_uniforms=True))
            differ = exp_flat != seq_flat
            if differ.any():
                t = u01.astype(np.float64) * seq[-1]
                edge = np.minimum(np.abs(seq[np.minimum(seq_flat, NPRI - 1)] - np.sort(t)),
                                  np.abs(seq[np.maximum(seq_flat - 1, 0)] - np.sort(t)))
                assert np.all(edge[differ] <= 1e-9 * seq[-1])
                near_edge += int(differ.sum())
            # split onto the table's steps
            f = exp_flat % (T * CAP)
            e_idx, e_ts, e_len = f // T, f % T, f % T + 1
            assert np.array_equal(idxs.cpu().numpy(), e_idx)
            assert np.array_equal(tss.cpu().numpy(), e_ts)
            assert np.array_equal(lens.cpu().numpy(), e_len)
            assert (e_ts < 29).any()                      # some windows are head-padded
            # every gathered byte, read by the oracle from the same host memory
            for c in range(4):
                exp, _ = oracle.subcopy(host, e_idx, e_ts, e_len, True, OFST, SPAN, S,
                                        STEP_BYTES[c], int(accu[c]) * T, threads=8)
                assert np.array_equal(dsts[c].cpu().numpy(), exp), "step %d column %d" % (step, c)
        assert near_edge <= 1                             # < 1e-6 of draws in any realistic run
    finally:
        torch.cuda.synchronize()
        assert lib.gear_hip_host_free(host_ptr) == 0


def test_config5_full_size_host_table_window_by_window():
    """Config 5's table at its full size: 2 000 trajectories x 1000 steps of the Atari schema,
    56.5 GB of pinned, mapped host memory, filled from a seeded device generator.  2048 windows
    drawn by priority over the 2 000 000 steps are gathered, all four columns, through the device
    alias of the host pointer (offsets far beyond 32 bits), and every window is compared with
    numpy slicing of the SAME host memory.  Skipped with the reason where the box cannot pin that
    much."""
    from gear_amd import _cabi, ops
    lib = _cabi.load()
    cap = 2000
    row = sum(STEP_BYTES)
    S = row * T
    nbytes = S * cap
    accu = np.concatenate([[0], np.cumsum(STEP_BYTES)])
    host_ptr, dev_ptr = ctypes.c_void_p(), ctypes.c_void_p()
    announce("config 5 full size: pinning a %.1f GB host table" % (nbytes / 1e9))
    rc = lib.gear_hip_host_alloc(nbytes, ctypes.byref(host_ptr), ctypes.byref(dev_ptr))
    if rc != 0:
        pytest.skip("this box does not pin %.1f GB of host memory (gear_hip_host_alloc: %s)"
                    % (nbytes / 1e9, lib.gear_hip_error_string(rc).decode()))
    try:
        g = torch.Generator(device="cuda")
        g.manual_seed(5505)
        piece_bytes = 1 << 30
        announce("config 5 full size: filling the table from the device")
        for o in range(0, nbytes, piece_bytes):
            nb = min(piece_bytes, nbytes - o)
            piece = torch.randint(0, 256, (nb,), dtype=torch.uint8, device="cuda", generator=g)
            _cabi.call("gear_hip_memcpy", ctypes.c_void_p(host_ptr.value + o),
                       ctypes.c_void_p(piece.data_ptr()), nb)
        del piece
        host = np.ctypeslib.as_array(ctypes.cast(host_ptr, ctypes.POINTER(ctypes.c_uint8)),
                                     shape=(nbytes,))
        rng = np.random.default_rng(5505)
        pri = (rng.lognormal(0, 1, size=T * cap) ** 0.6).astype(np.float32)
        u01 = rng.random(B, dtype=np.float32)
        prefix = ops.prefix_sum(torch.from_numpy(pri).cuda())
        flat, idxs, tss, lens = ops.sample_sorted(prefix, torch.from_numpy(u01).cuda(),
                                                  unit_uniforms=True, trajectory_length=T)
        dsts = [torch.full((B, SPAN * sb), 0xA5, dtype=torch.uint8, device="cuda")
                for sb in STEP_BYTES]
        cols = [dict(dst=dsts[c], ofst=OFST, span=SPAN, step_bytes=STEP_BYTES[c],
                     col_base=int(accu[c]) * T, pad_head=True, zero_fill=True) for c in range(4)]
        announce("config 5 full size: gather of 2048 windows x 4 columns from host memory")
        ops.subcopy_multi(dev_ptr.value, idxs, tss, lens, S, cols)
        torch.cuda.synchronize()
        hi, ht = idxs.cpu().numpy(), tss.cpu().numpy()
        assert np.array_equal(lens.cpu().numpy(), ht + 1)
        assert hi.max() * S > 2 ** 35 and (ht < SPAN - 1).any() and hi.max() < cap
        announce("config 5 full size: checking every window against the host bytes")
        for c in range(4):
            sb = STEP_BYTES[c]
            got = dsts[c].cpu().numpy()
            for w in range(B):
                first = max(int(ht[w]) + 1 - SPAN, 0)
                steps = int(ht[w]) + 1 - first
                a = int(hi[w]) * S + int(accu[c]) * T + first * sb
                assert np.array_equal(got[w, (SPAN - steps) * sb:], host[a:a + steps * sb]), (c, w)
                assert not got[w, :(SPAN - steps) * sb].any(), (c, w)
    finally:
        torch.cuda.synchronize()
        assert lib.gear_hip_host_free(host_ptr) == 0
