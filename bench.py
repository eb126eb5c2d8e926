#!/usr/bin/env python3
"""Benchmark of the replay-sampling hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one pass of the hot path over one batch: prefix sum of the per-step priorities, search
of the batch's seeded uniforms, sort of the drawn indices, split into (trajectory, timestep) and
the gather of all columns of the windows into contiguous batch tensors.  The default workload is
benchmark config 4 (Atari-shape table resident in HBM, 2048 windows of 30 steps).  Rank 0 prints
ONE JSON line; other workloads (--workload) print the same kind of line for that config.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth
# HBM bytes per gather launch on config 4, from the two rocprofv3 --pmc runs (FETCH_SIZE, then
# WRITE_SIZE, each scaled by a 1 GiB plain copy in the same run) summarised in
# profiles/subcopy_multi_kernel_config4_hbm_traffic.txt
MEASURED_GATHER_TRAFFIC_BYTES = 3486579262


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


class AtariTable:
    """benchmark config 4 / 5 schema: obs uint8[4,84,84], action int32, reward fp32, done uint8."""
    step_bytes = [4 * 84 * 84, 4, 4, 1]
    names = ["obs", "action", "reward", "done"]

    def __init__(self, T, capacity):
        self.T, self.capacity = T, capacity
        self.accu = [0]
        for b in self.step_bytes:
            self.accu.append(self.accu[-1] + b)
        self.traj_stride = self.accu[-1] * T
        self.nbytes = self.traj_stride * capacity

    def col_base(self, c):
        return self.accu[c] * self.T


def fill_device_table(torch, nbytes, seed):
    """Uniform random bytes written in 1 GiB pieces (values of the typed columns do not matter
    for a byte gather; the typed generators of the config are used by the parity tests)."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    table = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    piece = 1 << 30
    for o in range(0, nbytes, piece):
        n = min(piece, nbytes - o)
        table[o:o + n] = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    return table


def run_config4(args):
    import numpy as np
    import torch
    from gear_amd import ops

    torch.cuda.set_device(0)
    ops.set_device(0)
    T, cap, B, span, ofst = 1000, args.trajectories, 2048, 30, -29
    tab = AtariTable(T, cap)
    nsteps_total = T * cap
    log("building %.1f GB table in HBM" % (tab.nbytes / 1e9))
    table = fill_device_table(torch, tab.nbytes, 1004)
    rng = np.random.default_rng(1004)
    pri = (rng.lognormal(0.0, 1.0, size=nsteps_total) ** 0.6).astype(np.float32)
    dpri = torch.from_numpy(pri).cuda()
    total_iters = args.warmup + args.steps
    g = torch.Generator(device="cuda")
    g.manual_seed(2004)
    u01 = torch.rand((total_iters, B), dtype=torch.float32, device="cuda", generator=g)

    prefix = torch.empty(nsteps_total, dtype=torch.float64, device="cuda")
    flat = torch.empty(B, dtype=torch.int64, device="cuda")
    idxs = torch.empty(B, dtype=torch.int64, device="cuda")
    tss = torch.empty(B, dtype=torch.int64, device="cuda")
    lens = torch.empty(B, dtype=torch.int64, device="cuda")
    dsts = [torch.empty((B, span * sb), dtype=torch.uint8, device="cuda") for sb in tab.step_bytes]
    cols = [dict(dst=dsts[c], ofst=ofst, span=span, step_bytes=tab.step_bytes[c],
                 col_base=tab.col_base(c), pad_head=True, zero_fill=True) for c in range(4)]
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(args.steps)]

    def step(i, timed_slot=None):
        ops.prefix_sum(dpri, out=prefix)
        ops.sample_sorted(prefix, u01[i], unit_uniforms=True, sorted_out=flat,
                          trajectory_length=T, idxs=idxs, tss=tss, lens=lens)
        if timed_slot is not None:
            ev[timed_slot][0].record()
        ops.subcopy_multi(table, idxs, tss, lens, tab.traj_stride, cols)
        if timed_slot is not None:
            ev[timed_slot][1].record()

    if args.calibrate_copy:
        # a plain copy of known size through the generic slice kernel: the yardstick that the
        # FETCH_SIZE / WRITE_SIZE counters of the gather are scaled by
        nb = 1 << 30
        cdst = torch.empty(nb, dtype=torch.uint8, device="cuda")
        zero = torch.zeros(1, dtype=torch.int64, device="cuda")
        for _ in range(3):
            ops.copy(table, cdst, zero, zero, nb)
        torch.cuda.synchronize()
        del cdst

    for i in range(args.warmup):
        step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(args.warmup + i, i)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    launch_ms = sorted(a.elapsed_time(b) for a, b in ev)
    gather_ms = sum(launch_ms) / args.steps
    pct = lambda q: launch_ms[min(len(launch_ms) - 1, int(q * len(launch_ms)))]

    # The same K steps again with the sampler of batch i+1 enqueued on a second stream while
    # batch i is being gathered (what a prefetching loader does); reported next to the serial
    # figure, never instead of it.
    s_sample, s_gather = torch.cuda.Stream(), torch.cuda.Stream()
    bufs = [tuple(torch.empty(B, dtype=torch.int64, device="cuda") for _ in range(4))
            for _ in range(2)]
    torch.cuda.synchronize()

    def run_pipelined(first, count):
        sampled = [torch.cuda.Event() for _ in range(count)]
        gathered = [torch.cuda.Event() for _ in range(count)]
        for j in range(count):
            fl, ix, ts, ln = bufs[j % 2]
            with torch.cuda.stream(s_sample):
                if j >= 2:
                    s_sample.wait_event(gathered[j - 2])
                ops.prefix_sum(dpri, out=prefix)
                ops.sample_sorted(prefix, u01[first + j], unit_uniforms=True, sorted_out=fl,
                                  trajectory_length=T, idxs=ix, tss=ts, lens=ln)
                sampled[j].record(s_sample)
            with torch.cuda.stream(s_gather):
                s_gather.wait_event(sampled[j])
                ops.subcopy_multi(table, ix, ts, ln, tab.traj_stride, cols)
                gathered[j].record(s_gather)

    ms_pipelined = None
    if not args.no_pipelined:
        run_pipelined(0, args.warmup)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_pipelined(args.warmup, args.steps)
        torch.cuda.synchronize()
        ms_pipelined = (time.perf_counter() - t0) * 1e3 / args.steps

    payload = B * span * sum(tab.step_bytes)
    # Every byte of the batch is written once; a window that starts before its trajectory does
    # (ts < span - 1) reads only the steps that exist, the rest is zero padding.  The read side is
    # counted from the windows of the timed steps (same seeded draws, sampled again after timing).
    copied_steps, counted = 0, min(args.steps, 16)
    for i in range(counted):
        ops.prefix_sum(dpri, out=prefix)
        ops.sample_sorted(prefix, u01[args.warmup + i], unit_uniforms=True, sorted_out=flat,
                          trajectory_length=T, idxs=idxs, tss=tss, lens=lens)
        copied_steps += int(torch.clamp(tss + 1, max=span).sum().item())
    read_frac = copied_steps / float(counted * B * span)
    alg_bytes = payload * (1.0 + read_frac)
    achieved = alg_bytes / (gather_ms * 1e-3) / 1e9

    # Yardsticks of the same run: the batch payload moved as ONE contiguous piece, by the library's
    # slice kernel and by torch's device-to-device copy.  What a plain copy reaches on this box is
    # the practical ceiling of the gather; the roofline stays priced against the nominal peak.
    yard = None
    if not args.no_pipelined:
        ydst = torch.empty(payload, dtype=torch.uint8, device="cuda")
        ysrc = table[:payload]
        zero = torch.zeros(1, dtype=torch.int64, device="cuda")

        def timed_ms(fn, reps=20):
            for _ in range(3):
                fn()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(reps):
                fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / reps

        ms_lib = timed_ms(lambda: ops.copy(table, ydst, zero, zero, payload))
        ms_torch = timed_ms(lambda: ydst.copy_(ysrc))
        # one-directional streams through torch's own kernels: a fill (write only) and a sum
        # (read only) over the same number of bytes
        n8 = payload // 8
        y64 = ydst[:n8 * 8].view(torch.int64)
        ms_fill = timed_ms(lambda: y64.fill_(1))
        ms_sum = timed_ms(lambda: y64.sum())
        yard = {"contiguous_copy_slice_kernel_GBps": 2 * payload / (ms_lib * 1e-3) / 1e9,
                "contiguous_copy_torch_GBps": 2 * payload / (ms_torch * 1e-3) / 1e9,
                "write_only_torch_fill_GBps": n8 * 8 / (ms_fill * 1e-3) / 1e9,
                "read_only_torch_sum_GBps": n8 * 8 / (ms_sum * 1e-3) / 1e9,
                "gather_vs_contiguous_copy": ms_lib / gather_ms,
                "what": "%d bytes read + written as one contiguous piece, same run" % payload}
        del ydst
    result = {
        "metric": "sampled windows/sec + gather GB/s (% of HBM peak) at batch 2048, 1 MI355X",
        "value": B / (ms_per_step * 1e-3),
        "unit": "windows/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": "config4: Atari-shape table in HBM, %d steps (%d traj x %d), "
                               "priority-sampled batch of %d windows x %d steps, 4 columns"
                               % (nsteps_total, cap, T, B, span),
                   "table_bytes": tab.nbytes, "batch_payload_bytes": payload,
                   "step": "scan(1e6 f32->f64) + [search(2048) + sort + split] + gather(4 columns)"},
        "pipelined": None if ms_pipelined is None else {
            "ms_per_step": ms_pipelined, "value": B / (ms_pipelined * 1e-3),
            "frac_of_hbm_peak": alg_bytes / (ms_pipelined * 1e-3) / 1e9 / HBM_PEAK_GBPS,
            "what": "same steps, sampler of batch i+1 on a second stream during gather i"},
        "yardsticks": yard,
        "step_GBps": alg_bytes / (ms_per_step * 1e-3) / 1e9,
        "step_frac_of_hbm_peak": alg_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "roofline": {"bound": "hbm", "kernel": "subcopy_multi_kernel", "achieved": achieved,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "avg_launch_ms": gather_ms, "launch_ms_p10_p50_p90": [pct(0.1), pct(0.5), pct(0.9)],
                     "algorithmic_bytes": alg_bytes,
                     "algorithmic_bytes_if_no_window_were_padded": 2 * payload,
                     "steps_read_per_step_written": read_frac,
                     "traffic": args.traffic_bytes if args.traffic_bytes is not None else
                     (MEASURED_GATHER_TRAFFIC_BYTES if cap == 1000 else None),
                     "traffic_source": "--traffic-bytes" if args.traffic_bytes is not None else
                     ("profiles/subcopy_multi_kernel_config4_hbm_traffic.txt (rocprofv3 --pmc "
                      "FETCH_SIZE and WRITE_SIZE of this command, scaled by a 1 GiB copy; not "
                      "re-measured in this run)" if cap == 1000 else None)},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_config4(np, torch, tab, table, pri, B, span, ofst)
    if not args.no_hostlink:
        # after everything the line is made of has been measured: the same batch shape gathered
        # from a pinned host table (config 5's zero-copy path) against the host link
        del table
        torch.cuda.empty_cache()
        try:
            result["config5_hostlink"] = config5_hostlink(np, torch, ops, args.hostlink_trajectories)
        except Exception as exc:  # a refused pin or anything else here never fails the bench
            log("config-5 host-link sub-record skipped: %r" % (exc,))
            result["config5_hostlink"] = None
    return result


def config5_hostlink(np, torch, ops, cap):
    """Bounded sub-record of the config-4 line: config 5's gather -- 2048 windows x 30 steps x 4
    columns read by the GPU in place from a pinned, mapped host table -- next to a pinned
    hipMemcpyAsync host-to-device copy of the same number of bytes in the same run (the method of
    the reference's own benchmark, examples/offline/single-node/misc.py:34-46, on the path of
    src/storage/handler.cc:148-153).  The table is smaller than config 5's 56 GB: what the link
    delivers does not depend on the size of the table the windows are spread over."""
    import ctypes
    from gear_amd import _cabi
    lib = _cabi.load()
    T, B, span, ofst = 1000, 2048, 30, -29
    tab = AtariTable(T, cap)
    host_ptr, dev_ptr = ctypes.c_void_p(), ctypes.c_void_p()
    log("pinning %.1f GB of host memory for the host-link sub-record" % (tab.nbytes / 1e9))
    rc = lib.gear_hip_host_alloc(tab.nbytes, ctypes.byref(host_ptr), ctypes.byref(dev_ptr))
    if rc != 0:
        raise RuntimeError("gear_hip_host_alloc(%d) returned %d" % (tab.nbytes, rc))
    try:
        g = torch.Generator(device="cuda")
        g.manual_seed(1005)
        piece = torch.randint(0, 256, (1 << 28,), dtype=torch.uint8, device="cuda", generator=g)
        for o in range(0, tab.nbytes, piece.numel()):
            nb = min(piece.numel(), tab.nbytes - o)
            _cabi.call("gear_hip_memcpy", ctypes.c_void_p(host_ptr.value + o),
                       ctypes.c_void_p(piece.data_ptr()), nb)
        del piece
        flat = torch.sort(torch.randint(0, T * cap, (B,), dtype=torch.int64, device="cuda",
                                        generator=g)).values
        idxs, tss = flat // T, flat % T
        lens = tss + 1
        dsts = [torch.empty((B, span * sb), dtype=torch.uint8, device="cuda")
                for sb in tab.step_bytes]
        cols = [dict(dst=dsts[c], ofst=ofst, span=span, step_bytes=tab.step_bytes[c],
                     col_base=tab.col_base(c), pad_head=True, zero_fill=True) for c in range(4)]
        payload = B * span * sum(tab.step_bytes)
        read_bytes = int(torch.clamp(tss + 1, max=span).sum().item()) * sum(tab.step_bytes)

        def timed_ms(fn, warm, reps):
            for _ in range(warm):
                fn()
            torch.cuda.synchronize()
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(reps):
                fn()
            b.record()
            torch.cuda.synchronize()
            return a.elapsed_time(b) / reps

        gather_ms = timed_ms(lambda: ops.subcopy_multi(dev_ptr.value, idxs, tss, lens,
                                                       tab.traj_stride, cols), 3, 10)
        # a window is checked against the host bytes it came from
        w = B // 2
        i, ts = int(idxs[w].item()), int(tss[w].item())
        n = min(ts + 1, span)
        for c in (0, 3):
            sb = tab.step_bytes[c]
            off = i * tab.traj_stride + tab.col_base(c) + (ts + 1 - n) * sb
            src = np.ctypeslib.as_array(ctypes.cast(host_ptr.value + off,
                                                    ctypes.POINTER(ctypes.c_uint8)), shape=(n * sb,))
            got = dsts[c][w].cpu().numpy()
            if not (np.array_equal(got[(span - n) * sb:], src) and not got[:(span - n) * sb].any()):
                raise RuntimeError("host-table gather does not match the host bytes")
        pin = torch.empty(read_bytes, dtype=torch.uint8, pin_memory=True)
        dev = torch.empty(read_bytes, dtype=torch.uint8, device="cuda")
        h2d_ms = timed_ms(lambda: dev.copy_(pin, non_blocking=True), 2, 5)
        achieved = read_bytes / (gather_ms * 1e-3) / 1e9
        peak = read_bytes / (h2d_ms * 1e-3) / 1e9
        return {"bound": "host-link", "kernel": "subcopy_multi_kernel (source in pinned host memory)",
                "achieved": achieved, "peak": peak, "unit": "GB/s", "frac": achieved / peak,
                "peak_source": "pinned hipMemcpyAsync host-to-device copy of the same bytes, same run",
                "table_bytes": tab.nbytes, "bytes_over_the_link_per_launch": read_bytes,
                "batch_payload_bytes": payload,
                "parts_ms": {"gather": gather_ms, "h2d_copy": h2d_ms},
                "windows_per_s": B / (gather_ms * 1e-3),
                "what": "10 zero-copy gathers of 2048 windows x 30 steps x 4 columns from a %d-"
                        "trajectory (%.2f GB) Atari-shape table in pinned host memory; 5 pinned "
                        "host-to-device copies of the bytes those windows read"
                        % (cap, tab.nbytes / 1e9)}
    finally:
        lib.gear_hip_host_free(host_ptr)


def cpu_baseline_config4(np, torch, tab, table, pri, B, span, ofst):
    """The CPU oracle (a single-threaded C restatement of the reference's host path) on a bounded
    sample: the same priorities and batch shape, the table restricted to its first trajectories."""
    from oracle import oracle as orc
    keep = min(64, tab.capacity)
    host = table[:keep * tab.traj_stride].cpu().numpy()
    T = tab.T
    rng = np.random.default_rng(3004)
    dsts = [np.zeros((B, span * sb), np.uint8) for sb in tab.step_bytes]

    def one_step(threads):
        u01 = rng.random(B, dtype=np.float32)
        t0 = time.perf_counter()
        prefix = orc.scan_f32_f64(pri, threads=threads)
        flat = orc.upper_bound_f64(prefix, u01, unit_uniforms=True, threads=threads)
        flat = orc.sort_i64(flat)
        idxs = (flat // T) % keep
        tss = flat % T
        lens = tss + 1
        for c in range(4):
            orc.subcopy(host, idxs, tss, lens, True, ofst, span, tab.traj_stride,
                        tab.step_bytes[c], tab.col_base(c), zero_fill=True, dst=dsts[c],
                        threads=threads)
        return time.perf_counter() - t0

    def timed(threads, budget):
        nrun, t_total = 0, 0.0
        while nrun < 3 or (t_total < budget and nrun < 400):
            t_total += one_step(threads)
            nrun += 1
        return nrun, t_total

    nrun, t_total = timed(1, 10.0)
    # the same step over the host's share of cores (two-level chunked scan, draws and windows split
    # over threads; the sort of 2048 keys stays sequential): 16 threads at most, the CPU share of a
    # one-GPU box
    cores = max(1, min(16, os.cpu_count() or 1))
    one_step(cores)
    nrun_mt, t_mt = timed(cores, 5.0)
    return {"value": B * nrun / t_total, "unit": "windows/s", "cores": 1, "kind": "port",
            "ms_per_step": t_total / nrun * 1e3,
            "all_cores": {"value": B * nrun_mt / t_mt, "unit": "windows/s", "cores": cores,
                          "ms_per_step": t_mt / nrun_mt * 1e3},
            "cpu_model": cpu_model(),
            "sample": "%d steps of the same pipeline (fp64 scan of 1e6 priorities, 2048 searches, "
                      "sort, 4-column gather with memset+memcpy per window) on the first %d of %d "
                      "trajectories (%.1f GB of the table, trajectory index taken modulo %d); "
                      "host has %d logical cores; value uses 1, all_cores runs a chunked scan and "
                      "splits draws and windows over %d threads (%d steps)"
                      % (nrun, keep, tab.capacity, keep * tab.traj_stride / 1e9, keep,
                         os.cpu_count() or 0, cores, nrun_mt)}


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


class GenericTable:
    def __init__(self, step_bytes, T, capacity):
        self.step_bytes = list(step_bytes)
        self.T, self.capacity = T, capacity
        self.accu = [0]
        for b in self.step_bytes:
            self.accu.append(self.accu[-1] + b)
        self.traj_stride = self.accu[-1] * T
        self.nbytes = self.traj_stride * capacity

    def col_base(self, c):
        return self.accu[c] * self.T


def _time_steps(torch, step, steps, warmup, events=None):
    """Wall time per step of `steps` steps after `warmup` untimed ones, then the same steps once
    more with the HIP events that bracket the kernels (step(i, slot) records them when slot is
    not None): in these small steps two event records cost as much as a kernel launch, so they
    stay out of the timed pass."""
    for i in range(warmup):
        step(i, None)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(warmup + i, None)
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / steps
    for i in range(steps):
        step(warmup + i, i)
    torch.cuda.synchronize()
    return ms


def _time_graph(torch, body, feed, steps, warmup):
    """The same steps replayed from a HIP graph (what a launch-bound loop wants): body() reads
    static input buffers, feed(i) copies step i's inputs into them (eager, one small launch)."""
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):   # warm-up on the capture stream: workspaces get allocated
        feed(0)
        body()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        body()
    for i in range(warmup):
        feed(i)
        graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        feed(warmup + i)
        graph.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def _graph_extra(B, unit, gms_):
    return {"graph_replay": {"ms_per_step": gms_, "value": B / (gms_ * 1e-3), "unit": unit,
                             "what": "same steps: inputs copied into static buffers, then one "
                                     "replay of the captured step"}}


def _line(metric_value, unit, args, ms, workload, roofline, extra=None):
    d = {"metric": "sampled windows/sec + gather GB/s (% of HBM peak) at batch 2048, 1 MI355X",
         "value": metric_value, "unit": unit, "n_gpus": 1, "steps": args.steps,
         "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True, "scaling": "weak",
         "vs_baseline": None, "dtype": "u8", "data": "synthetic",
         "config": {"workload": workload}, "roofline": roofline}
    if extra:
        d.update(extra)
    return d


def run_config1(args):
    """Uniform sampling + full-trajectory gather, 4096 x 64 table, batch 256."""
    import numpy as np
    import torch
    from gear_amd import ops
    from oracle import oracle as orc
    tab = GenericTable([68, 24, 4, 1], 64, 4096)
    table = fill_device_table(torch, tab.nbytes, 1001)
    B = 256
    g = torch.Generator(device="cuda")
    g.manual_seed(1001)
    draws = torch.randint(0, 4096, (args.warmup + args.steps, B), dtype=torch.int64, device="cuda",
                          generator=g)
    tss = torch.zeros(B, dtype=torch.int64, device="cuda")
    lens = torch.full((B,), 64, dtype=torch.int64, device="cuda")
    dsts = [torch.empty((B, 64 * sb), dtype=torch.uint8, device="cuda") for sb in tab.step_bytes]
    cols = [dict(dst=dsts[c], ofst=0, span=64, step_bytes=tab.step_bytes[c],
                 col_base=tab.col_base(c), pad_head=False) for c in range(4)]
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(args.steps)]

    # the loader's step after the draws, in two calls: ascending sort of the drawn trajectories
    # with the look-up of their recorded lengths (all 64 here) in the same launch, then the
    # gather of all columns through a plan made once (same batch tensors every step)
    lengths_table = torch.full((4096,), 64, dtype=torch.int64, device="cuda")
    idx = torch.empty(B, dtype=torch.int64, device="cuda")
    loc = torch.empty(B, dtype=torch.int64, device="cuda")
    plan = ops.GatherPlan(table, tab.traj_stride, cols, B)

    def select(d):
        ops.sort_lookup(d, 4096, lengths_table=lengths_table, sampled_out=idx, local_out=loc,
                        lens_out=lens)

    def step(i, slot):
        select(draws[i])
        if slot is not None:
            ev[slot][0].record()
        plan.run(idx, tss, lens)
        if slot is not None:
            ev[slot][1].record()

    ms = _time_steps(torch, step, args.steps, args.warmup)
    gms = sum(a.elapsed_time(b) for a, b in ev) / args.steps
    cur = torch.empty(B, dtype=torch.int64, device="cuda")

    def body():
        select(cur)
        plan.run(idx, tss, lens)

    ms_graph = _time_graph(torch, body, lambda i: cur.copy_(draws[i]), args.steps, args.warmup)
    alg = 2 * B * tab.traj_stride
    host = table.cpu().numpy()
    hd = [np.zeros((B, 64 * sb), np.uint8) for sb in tab.step_bytes]
    rng = np.random.default_rng(1)
    t0 = time.perf_counter()
    n = 0
    while time.perf_counter() - t0 < 3.0:
        idx = np.sort(rng.integers(0, 4096, size=B))
        for c in range(4):
            orc.subcopy(host, idx, np.zeros(B, np.int64), np.full(B, 64, np.int64), False, 0, 64,
                        tab.traj_stride, tab.step_bytes[c], tab.col_base(c), dst=hd[c])
        n += 1
    cpu_ms = (time.perf_counter() - t0) * 1e3 / n
    cores = max(1, min(16, os.cpu_count() or 1))
    t0 = time.perf_counter()
    nmt = 0
    while time.perf_counter() - t0 < 2.0:
        idx = np.sort(rng.integers(0, 4096, size=B))
        for c in range(4):
            orc.subcopy(host, idx, np.zeros(B, np.int64), np.full(B, 64, np.int64), False, 0, 64,
                        tab.traj_stride, tab.step_bytes[c], tab.col_base(c), dst=hd[c], threads=cores)
        nmt += 1
    mt_ms = (time.perf_counter() - t0) * 1e3 / nmt
    return _line(B / (ms * 1e-3), "trajectories/s", args, ms,
                 "config1: 4096 x 64 table (obs f32[17], act f32[6], rew f32, done u8), uniform "
                 "batch of 256 full trajectories, sort + 4-column gather",
                 {"bound": "hbm", "kernel": "subcopy_multi_kernel", "achieved": alg / (gms * 1e-3) / 1e9,
                  "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": alg / (gms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                  "avg_launch_ms": gms, "algorithmic_bytes": alg, "traffic": None},
                 dict(_graph_extra(B, "trajectories/s", ms_graph),
                      cpu_baseline={"value": B / (cpu_ms * 1e-3), "unit": "trajectories/s",
                                    "cores": 1, "kind": "port", "ms_per_step": cpu_ms,
                                    "all_cores": {"value": B / (mt_ms * 1e-3),
                                                  "unit": "trajectories/s", "cores": cores,
                                                  "ms_per_step": mt_ms, "steps": nmt},
                                    "cpu_model": cpu_model(),
                                    "sample": "%d steps of sort + 4-column memset+memcpy gather "
                                              "(all_cores: windows split over threads)" % n}))


def run_config2(args):
    """Prioritized sampling: 1e6 priorities, 4096 draws, importance weights."""
    import numpy as np
    import torch
    from gear_amd import ops
    from oracle import oracle as orc
    n, B = 1_000_000, 4096
    rng = np.random.default_rng(1002)
    pri = (rng.lognormal(0.0, 1.0, size=n) ** 0.6).astype(np.float32)
    dpri = torch.from_numpy(pri).cuda()
    g = torch.Generator(device="cuda")
    g.manual_seed(1002)
    u01 = torch.rand((args.warmup + args.steps, B), dtype=torch.float32, device="cuda", generator=g)
    prefix = torch.empty(n, dtype=torch.float64, device="cuda")
    idx = torch.empty(B, dtype=torch.int64, device="cuda")
    w = torch.empty(B, dtype=torch.float32, device="cuda")
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(args.steps)]

    def step(i, slot):
        if slot is not None:
            ev[slot][0].record()
        ops.prefix_sum(dpri, out=prefix)
        if slot is not None:
            ev[slot][1].record()
        ops.upper_bound(prefix, u01[i], unit_uniforms=True, idx_out=idx, priorities=dpri, beta=0.4,
                        weights_out=w)

    ms = _time_steps(torch, step, args.steps, args.warmup)
    sms = sum(a.elapsed_time(b) for a, b in ev) / args.steps
    ucur = torch.empty(B, dtype=torch.float32, device="cuda")

    def body():
        ops.prefix_sum(dpri, out=prefix)
        ops.upper_bound(prefix, ucur, unit_uniforms=True, idx_out=idx, priorities=dpri, beta=0.4,
                        weights_out=w)

    ms_graph = _time_graph(torch, body, lambda i: ucur.copy_(u01[i]), args.steps, args.warmup)
    alg = 12 * n
    t0 = time.perf_counter()
    k = 0
    while time.perf_counter() - t0 < 3.0:
        uu = rng.random(B, dtype=np.float32)
        pre = orc.scan_f32_f64(pri)
        ii = orc.upper_bound_f64(pre, uu, unit_uniforms=True)
        orc.is_weights(pri, pre[-1], ii, 0.4)
        k += 1
    cpu_ms = (time.perf_counter() - t0) * 1e3 / k
    cores = max(1, min(16, os.cpu_count() or 1))
    t0 = time.perf_counter()
    kmt = 0
    while time.perf_counter() - t0 < 2.0:
        uu = rng.random(B, dtype=np.float32)
        pre = orc.scan_f32_f64(pri, threads=cores)
        ii = orc.upper_bound_f64(pre, uu, unit_uniforms=True, threads=cores)
        orc.is_weights(pri, pre[-1], ii, 0.4)
        kmt += 1
    mt_ms = (time.perf_counter() - t0) * 1e3 / kmt
    return _line(B / (ms * 1e-3), "draws/s", args, ms,
                 "config2: 1e6 fp32 priorities -> fp64 prefix (one chained single-pass launch), 4096 "
                 "draws, importance weights",
                 {"bound": "hbm", "kernel": "scan_ranges_kernel<float, double, double, G, kChained> (one launch: the chained prefix sum)", "achieved": alg / (sms * 1e-3) / 1e9,
                  "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": alg / (sms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                  "avg_launch_ms": sms, "algorithmic_bytes": alg, "traffic": None},
                 dict(_graph_extra(B, "draws/s", ms_graph),
                      cpu_baseline={"value": B / (cpu_ms * 1e-3), "unit": "draws/s", "cores": 1,
                                    "kind": "port", "ms_per_step": cpu_ms,
                                    "all_cores": {"value": B / (mt_ms * 1e-3), "unit": "draws/s",
                                                  "cores": cores, "ms_per_step": mt_ms, "steps": kmt},
                                    "cpu_model": cpu_model(),
                                    "sample": "%d steps of fp64 scan + 4096 searches + weights "
                                              "(all_cores: chunked scan, draws split over threads)" % k}))


def run_config3(args):
    """Decision-Transformer windows: 100 000 variable-length trajectories, 1024 x 20 steps + mask."""
    import numpy as np
    import torch
    from gear_amd import ops
    tab = GenericTable([68, 24, 4, 4, 4], 1000, args.trajectories3)
    log("building %.1f GB table in HBM" % (tab.nbytes / 1e9))
    table = fill_device_table(torch, tab.nbytes, 1003)
    B, span = 1024, 20
    rng = np.random.default_rng(1003)
    lengths = torch.from_numpy(rng.integers(200, 1001, size=tab.capacity).astype(np.int64)).cuda()
    g = torch.Generator(device="cuda")
    g.manual_seed(1003)
    total = args.warmup + args.steps
    u1 = torch.rand((total, B), dtype=torch.float64, device="cuda", generator=g)
    u2 = torch.rand((total, B), dtype=torch.float64, device="cuda", generator=g)
    prefix = torch.empty(tab.capacity, dtype=torch.int64, device="cuda")
    dsts = [torch.empty((B, span * sb), dtype=torch.uint8, device="cuda") for sb in tab.step_bytes]
    mask = torch.empty((B, span), dtype=torch.uint8, device="cuda")
    cols = [dict(dst=dsts[c], ofst=0, span=span, step_bytes=tab.step_bytes[c],
                 col_base=tab.col_base(c), pad_head=False, mask_out=mask if c == 0 else None)
            for c in range(5)]
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(args.steps)]

    # length-weighted draw, sort, length look-up and window starts in one launch, and the gather
    # through a plan made once (same batch tensors every step)
    traj = torch.empty(B, dtype=torch.int64, device="cuda")
    loc = torch.empty(B, dtype=torch.int64, device="cuda")
    lens = torch.empty(B, dtype=torch.int64, device="cuda")
    start = torch.empty(B, dtype=torch.int64, device="cuda")
    plan = ops.GatherPlan(table, tab.traj_stride, cols, B)

    def select(ua, ub):
        # length-weighted trajectories, sorted, their lengths and the window starts
        # floor(ub * (len - span + 1)): one launch after the prefix sum
        ops.prefix_sum_i64(lengths, out=prefix)
        ops.sample_lookup(prefix, ua, lengths_table=lengths, sampled_out=traj, local_out=loc,
                          lens_out=lens, start_uniforms=ub, window=span, starts_out=start)

    def step(i, slot):
        select(u1[i], u2[i])
        if slot is not None:
            ev[slot][0].record()
        plan.run(traj, start, lens)
        if slot is not None:
            ev[slot][1].record()

    ms = _time_steps(torch, step, args.steps, args.warmup)
    gms = sum(a.elapsed_time(b) for a, b in ev) / args.steps
    uc = torch.empty((2, B), dtype=torch.float64, device="cuda")

    def body():
        select(uc[0], uc[1])
        plan.run(traj, start, lens)

    def feed(i):
        uc[0].copy_(u1[i])
        uc[1].copy_(u2[i])

    ms_graph = _time_graph(torch, body, feed, args.steps, args.warmup)
    alg = 2 * B * span * sum(tab.step_bytes) + B * span
    extra = _graph_extra(B, "windows/s", ms_graph)
    if not args.no_cpu_baseline:
        # CPU oracle on a bounded sample: the same sampler over all lengths, the gather on the
        # first trajectories of the table (index taken modulo their number)
        from oracle import oracle as orc
        keep = min(2000, tab.capacity)
        host = table[:keep * tab.traj_stride].cpu().numpy()
        hl = lengths.cpu().numpy()
        hd = [np.zeros((B, span * sb), np.uint8) for sb in tab.step_bytes]
        crng = np.random.default_rng(3003)
        t0 = time.perf_counter()
        nrun = 0
        while nrun < 3 or (time.perf_counter() - t0 < 3.0 and nrun < 2000):
            pre = orc.scan_i64(hl)
            traj = orc.sort_i64(orc.upper_bound_i64(pre, crng.random(B), unit_uniforms=True))
            lens_h = hl[traj]
            start = (crng.random(B) * (lens_h - (span - 1))).astype(np.int64)
            for c in range(5):
                orc.subcopy(host, traj % keep, start, lens_h, False, 0, span, tab.traj_stride,
                            tab.step_bytes[c], tab.col_base(c), dst=hd[c], want_mask=(c == 0))
            nrun += 1
        cpu_ms = (time.perf_counter() - t0) * 1e3 / nrun
        cores = max(1, min(16, os.cpu_count() or 1))
        t0 = time.perf_counter()
        nmt = 0
        while nmt < 3 or (time.perf_counter() - t0 < 2.0 and nmt < 2000):
            pre = orc.scan_i64(hl)
            traj = orc.sort_i64(orc.upper_bound_i64(pre, crng.random(B), unit_uniforms=True))
            lens_h = hl[traj]
            start = (crng.random(B) * (lens_h - (span - 1))).astype(np.int64)
            for c in range(5):
                orc.subcopy(host, traj % keep, start, lens_h, False, 0, span, tab.traj_stride,
                            tab.step_bytes[c], tab.col_base(c), dst=hd[c], want_mask=(c == 0),
                            threads=cores)
            nmt += 1
        mt_ms = (time.perf_counter() - t0) * 1e3 / nmt
        extra["cpu_baseline"] = {
            "value": B / (cpu_ms * 1e-3), "unit": "windows/s", "cores": 1, "kind": "port",
            "ms_per_step": cpu_ms,
            "all_cores": {"value": B / (mt_ms * 1e-3), "unit": "windows/s", "cores": cores,
                          "ms_per_step": mt_ms, "steps": nmt,
                          "what": "windows of the gather split over threads"},
            "cpu_model": cpu_model(),
            "sample": "%d steps of int64 scan + 1024 searches + sort + 5-column gather with mask, "
                      "table cut to its first %d trajectories" % (nrun, keep)}
    return _line(B / (ms * 1e-3), "windows/s", args, ms,
                 "config3: %d variable-length trajectories (T=1000), length-weighted int64 sampler, "
                 "1024 windows x 20 steps x 5 columns + uint8 mask" % tab.capacity,
                 {"bound": "hbm", "kernel": "subcopy_multi_kernel", "achieved": alg / (gms * 1e-3) / 1e9,
                  "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": alg / (gms * 1e-3) / 1e9 / HBM_PEAK_GBPS,
                  "avg_launch_ms": gms, "algorithmic_bytes": alg, "traffic": None},
                 extra)


def run_config5(args):
    """Zero-copy host-resident table + priority maintenance."""
    import ctypes
    import numpy as np
    import torch
    from gear_amd import _cabi, ops
    lib = _cabi.load()
    T, B, span, ofst = 1000, 2048, 30, -29
    cap = args.trajectories5
    tab = AtariTable(T, cap)
    host_ptr, dev_ptr = ctypes.c_void_p(), ctypes.c_void_p()
    while True:
        log("pinning %.1f GB of host memory" % (tab.nbytes / 1e9))
        rc = lib.gear_hip_host_alloc(tab.nbytes, ctypes.byref(host_ptr), ctypes.byref(dev_ptr))
        if rc == 0:
            break
        cap //= 2
        if cap < 16:
            raise RuntimeError("cannot pin a host table")
        tab = AtariTable(T, cap)
    # fill the host table from a 1 GiB random device buffer (byte values do not matter)
    g = torch.Generator(device="cuda")
    g.manual_seed(1005)
    piece = torch.randint(0, 256, (1 << 30,), dtype=torch.uint8, device="cuda", generator=g)
    for o in range(0, tab.nbytes, 1 << 30):
        nb = min(1 << 30, tab.nbytes - o)
        _cabi.call("gear_hip_memcpy", ctypes.c_void_p(host_ptr.value + o),
                   ctypes.c_void_p(piece.data_ptr()), nb)
    del piece
    src = dev_ptr.value
    npri, k, m = 10_000_000, 65_536, 65_536
    rng = np.random.default_rng(1005)
    pri = torch.from_numpy((rng.lognormal(0, 1, size=npri) ** 0.6).astype(np.float32)).cuda()
    total = args.warmup + args.steps
    upd_idx = [torch.from_numpy(rng.permutation(npri)[:m].astype(np.int64)).cuda() for _ in range(4)]
    upd_val = [torch.from_numpy((rng.lognormal(0, 1, size=m) ** 0.6).astype(np.float32)).cuda()
               for _ in range(4)]
    g.manual_seed(2005)
    u01 = torch.rand((total, B), dtype=torch.float32, device="cuda", generator=g)
    prefix = torch.empty(npri, dtype=torch.float64, device="cuda")
    flat = torch.empty(B, dtype=torch.int64, device="cuda")
    idxs, tss, lens = (torch.empty(B, dtype=torch.int64, device="cuda") for _ in range(3))
    dsts = [torch.empty((B, span * sb), dtype=torch.uint8, device="cuda") for sb in tab.step_bytes]
    cols = [dict(dst=dsts[c], ofst=ofst, span=span, step_bytes=tab.step_bytes[c],
                 col_base=tab.col_base(c), pad_head=True) for c in range(4)]
    names = ["scatter", "topk", "scan", "sample", "gather"]
    selection = ops.TopKState()   # steps after the first start from the last step's bound
    ev = [[torch.cuda.Event(enable_timing=True) for _ in range(len(names) + 1)]
          for _ in range(args.steps)]

    def step(i, slot):
        e = ev[slot] if slot is not None else None
        if e: e[0].record()
        ops.scatter(pri, upd_idx[i % 4], upd_val[i % 4], unique_indices=True)
        if e: e[1].record()
        selection.select(pri, k, sorted_by_value=True)
        if e: e[2].record()
        ops.prefix_sum(pri, out=prefix)
        if e: e[3].record()
        ops.sample_sorted(prefix, u01[i], unit_uniforms=True, sorted_out=flat,
                          trajectory_length=T, modulo=T * cap, idxs=idxs, tss=tss, lens=lens)
        if e: e[4].record()
        ops.subcopy_multi(src, idxs, tss, lens, tab.traj_stride, cols)
        if e: e[5].record()

    ms = _time_steps(torch, step, args.steps, args.warmup)
    parts = {n: sum(ev[s][j].elapsed_time(ev[s][j + 1]) for s in range(args.steps)) / args.steps
             for j, n in enumerate(names)}
    payload = B * span * sum(tab.step_bytes)
    # host-link yardstick: pinned -> device copy of the same number of bytes in the same run
    pin = torch.empty(payload, dtype=torch.uint8, pin_memory=True)
    dev = torch.empty(payload, dtype=torch.uint8, device="cuda")
    for _ in range(2):
        dev.copy_(pin, non_blocking=True)
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(5):
        dev.copy_(pin, non_blocking=True)
    b.record()
    torch.cuda.synchronize()
    link_gbps = payload / (a.elapsed_time(b) / 5 * 1e-3) / 1e9
    gather_gbps = payload / (parts["gather"] * 1e-3) / 1e9
    extra5 = {}
    if not args.no_cpu_baseline:
        # CPU oracle, bounded: the maintenance step on the full 1e7 priorities, the gather on the
        # first trajectories of the host table
        from oracle import oracle as orc
        keep = min(64, cap)
        host = np.ctypeslib.as_array(
            ctypes.cast(host_ptr, ctypes.POINTER(ctypes.c_uint8)), shape=(keep * tab.traj_stride,))
        hp = pri.cpu().numpy().copy()
        hidx = [t.cpu().numpy() for t in upd_idx]
        hval = [t.cpu().numpy() for t in upd_val]
        hd = [np.zeros((B, span * sb), np.uint8) for sb in tab.step_bytes]
        crng = np.random.default_rng(3005)
        parts_cpu = {n: 0.0 for n in names}
        t_all = time.perf_counter()
        nrun = 0
        while nrun < 2 or (time.perf_counter() - t_all < 10.0 and nrun < 20):
            t0 = time.perf_counter()
            orc.scatter_f32(hp, hidx[nrun % 4], hval[nrun % 4])
            t1 = time.perf_counter()
            orc.topk_f32(hp, k, True)
            t2 = time.perf_counter()
            pre = orc.scan_f32_f64(hp)
            t3 = time.perf_counter()
            fl = orc.sort_i64(orc.upper_bound_f64(pre, crng.random(B, dtype=np.float32),
                                                  unit_uniforms=True)) % (T * cap)
            t4 = time.perf_counter()
            for c in range(4):
                orc.subcopy(host, (fl // T) % keep, fl % T, fl % T + 1, True, ofst, span,
                            tab.traj_stride, tab.step_bytes[c], tab.col_base(c), dst=hd[c])
            t5 = time.perf_counter()
            for n_, d_ in zip(names, (t1 - t0, t2 - t1, t3 - t2, t4 - t3, t5 - t4)):
                parts_cpu[n_] += d_ * 1e3
            nrun += 1
        cpu_ms = (time.perf_counter() - t_all) * 1e3 / nrun
        # the same step over the host's share of cores: per-chunk top-k selection + merge, two-level
        # chunked scan, draws and windows split over threads (scatter and the 2048-key sort stay
        # sequential)
        cores = max(1, min(16, os.cpu_count() or 1))
        parts_mt = {n: 0.0 for n in names}
        t_mt = time.perf_counter()
        nmt = 0
        while nmt < 2 or (time.perf_counter() - t_mt < 6.0 and nmt < 40):
            t0 = time.perf_counter()
            orc.scatter_f32(hp, hidx[nmt % 4], hval[nmt % 4])
            t1 = time.perf_counter()
            orc.topk_f32(hp, k, True, threads=cores)
            t2 = time.perf_counter()
            pre = orc.scan_f32_f64(hp, threads=cores)
            t3 = time.perf_counter()
            fl = orc.sort_i64(orc.upper_bound_f64(pre, crng.random(B, dtype=np.float32),
                                                  unit_uniforms=True, threads=cores)) % (T * cap)
            t4 = time.perf_counter()
            for c in range(4):
                orc.subcopy(host, (fl // T) % keep, fl % T, fl % T + 1, True, ofst, span,
                            tab.traj_stride, tab.step_bytes[c], tab.col_base(c), dst=hd[c],
                            threads=cores)
            t5 = time.perf_counter()
            for n_, d_ in zip(names, (t1 - t0, t2 - t1, t3 - t2, t4 - t3, t5 - t4)):
                parts_mt[n_] += d_ * 1e3
            nmt += 1
        mt_ms = (time.perf_counter() - t_mt) * 1e3 / nmt
        extra5["cpu_baseline"] = {
            "value": B / (cpu_ms * 1e-3), "unit": "windows/s", "cores": 1, "kind": "port",
            "ms_per_step": cpu_ms, "parts_ms": {n_: v / nrun for n_, v in parts_cpu.items()},
            "all_cores": {"value": B / (mt_ms * 1e-3), "unit": "windows/s", "cores": cores,
                          "ms_per_step": mt_ms, "steps": nmt,
                          "parts_ms": {n_: v / nmt for n_, v in parts_mt.items()}},
            "cpu_model": cpu_model(),
            "sample": "%d steps: scatter 65536, top-65536 of 1e7, fp64 rescan of 1e7, 2048 draws, "
                      "4-column gather from the first %d trajectories of the host table"
                      % (nrun, keep)}
    lib.gear_hip_host_free(host_ptr)
    return _line(B / (ms * 1e-3), "windows/s", args, ms,
                 "config5: %d-step Atari-shape table in pinned host memory (%.1f GB, zero-copy), per "
                 "step scatter 65536 -> top-65536 of 1e7 -> rescan 1e7 -> 2048 draws -> gather"
                 % (T * cap, tab.nbytes / 1e9),
                 {"bound": "host-link", "kernel": "subcopy_multi_kernel (source in host memory)",
                  "achieved": gather_gbps, "peak": link_gbps, "unit": "GB/s",
                  "frac": gather_gbps / link_gbps, "avg_launch_ms": parts["gather"],
                  "algorithmic_bytes": payload,
                  "peak_source": "pinned hipMemcpyAsync H2D of the same bytes in this run",
                  "traffic": None},
                 dict(extra5, parts_ms=parts,
                      maintenance={"topk_GBps_one_read": 4 * npri / (parts["topk"] * 1e-3) / 1e9,
                                   "rescan_GBps": 12 * npri / (parts["scan"] * 1e-3) / 1e9}))


def _calibrate_copy(torch, ops):
    """Three plain 1 GiB copies through the library's slice kernel: the launch of known size that
    the FETCH_SIZE / WRITE_SIZE counters of the other kernels in the same run are scaled by."""
    nb = 1 << 30
    csrc = torch.zeros(nb, dtype=torch.uint8, device="cuda")
    cdst = torch.empty(nb, dtype=torch.uint8, device="cuda")
    zero = torch.zeros(1, dtype=torch.int64, device="cuda")
    for _ in range(3):
        ops.copy(csrc, cdst, zero, zero, nb)
    torch.cuda.synchronize()


def run_scan(args):
    """One kernel chain on its own: fp64 prefix sum of --n fp32 priorities.  The variant follows
    GEAR_HIP_SCAN_SINGLE_PASS (unset or 1: chained single pass, 0: range sums + scan in two
    launches)."""
    import numpy as np
    import torch
    from gear_amd import ops
    n = args.n
    rng = np.random.default_rng(7)
    pri = torch.from_numpy((rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)).cuda()
    prefix = torch.empty(n, dtype=torch.float64, device="cuda")
    if args.calibrate_copy:
        _calibrate_copy(torch, ops)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(args.steps)]

    def step(i, slot):
        if slot is not None:
            ev[slot][0].record()
        ops.prefix_sum(pri, out=prefix)
        if slot is not None:
            ev[slot][1].record()

    ms = _time_steps(torch, step, args.steps, args.warmup)
    sms = sorted(a.elapsed_time(b) for a, b in ev)
    avg = sum(sms) / len(sms)
    alg = 12 * n

    # Yardsticks of the same run, same n, through torch's own kernels: the plain fp32 -> fp64
    # conversion copy (the scan's memory pattern without any arithmetic or dependence between
    # workgroups), an fp64 fill (its writes alone) and torch.cumsum in fp64 (the library scan).
    def timed_us(fn, reps=50):
        for _ in range(5):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps * 1e3

    ybuf = torch.empty(n, dtype=torch.float64, device="cuda")
    yard = {"back_to_back_us": timed_us(lambda: ops.prefix_sum(pri, out=prefix)),
            "torch_f32_to_f64_copy_us": timed_us(lambda: ybuf.copy_(pri)),
            "torch_fill_f64_us": timed_us(lambda: ybuf.fill_(1.0)),
            "torch_cumsum_f64_us": timed_us(lambda: torch.cumsum(pri, 0, dtype=torch.float64, out=ybuf)),
            "what": "HIP events around 50 back-to-back launches each, same n"}
    forced = os.environ.get("GEAR_HIP_SCAN_SINGLE_PASS", "")
    ranges = -(-n // 8192)     # what the library does at this size: see gear_amd/csrc/scan.hip
    by_size = ("three launches (range sums, their prefix, scan)" if ranges > 16384 else
               "two launches" if ranges > 8192 or forced == "0" else "chained single pass")
    variant = by_size + (" (default)" if forced == "" else "")
    return _line(n / (ms * 1e-3), "priorities/s", args, ms,
                 "scan: fp64 prefix sum of %d fp32 priorities, %s" % (n, variant),
                 {"bound": "hbm", "kernel": "prefix sum chain (" + variant + ")",
                  "achieved": alg / (avg * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                  "frac": alg / (avg * 1e-3) / 1e9 / HBM_PEAK_GBPS, "avg_launch_ms": avg,
                  "median_launch_ms": sms[len(sms) // 2], "algorithmic_bytes": alg,
                  "traffic": None}, {"yardsticks": yard})


TOPK_INPUTS = {
    "lognormal": "lognormal ** 0.6 (the priorities of every other workload here)",
    "equal": "all priorities equal",
    "integers": "integers 0..999 (ten thousand ties per value at n = 1e7)",
    "ties": "every 166th priority at one value above all others (60 000 ties at n = 1e7)",
    "ties-neighbours": "the same with a hundred entries a few ulps above the ties",
    "ascending": "sorted ascending (the selection is the array's end)",
    "hot-stretch": "k consecutive entries above everything else",
    "hot-half": "k / 2 consecutive entries above everything else",
    "misleading": "the 2048 sampled positions hold the largest priorities (the sampled bound fails)",
}


def _topk_input(np, n, k, kind):
    """The priorities of --workload topk: lognormal, or one of the shapes that take the selection
    off its usual path (masses of ties, clustered maxima, a sample that misleads)."""
    rng = np.random.default_rng(7)
    w = (rng.lognormal(0, 1, size=n) ** 0.6).astype(np.float32)
    if kind == "equal":
        w[:] = 1.0
    elif kind == "integers":
        w = rng.integers(0, 1000, size=n).astype(np.float32)
    elif kind in ("ties", "ties-neighbours"):
        w[rng.random(n) < 1.0 / 166.0] = 100.0
        if kind == "ties-neighbours":
            at = rng.permutation(n)[:100]
            w[at] = np.float32(100.0) + np.float32(1e-4) * rng.integers(1, 8, size=100).astype(np.float32)
    elif kind == "ascending":
        w.sort()
    elif kind in ("hot-stretch", "hot-half"):
        m = k if kind == "hot-stretch" else k // 2
        a = min(7 * n // 10, n - m)
        w[a:a + m] += np.float32(100.0)
    elif kind == "misleading":
        samples = 2048
        stride = n // samples
        s_ = np.arange(samples, dtype=np.uint64)
        off = (((s_ * np.uint64(2654435761)) & np.uint64(0xffffffff)) * np.uint64(stride)) >> np.uint64(32)
        w[(s_ * np.uint64(stride) + off).astype(np.int64)] = (1000.0 + np.arange(samples)).astype(np.float32)
    return w


def run_topk(args):
    """One kernel chain on its own: top --k of --n fp32 priorities (--topk-order value|index)."""
    import numpy as np
    import torch
    from gear_amd import ops
    n, k = args.n, args.k
    by_value = args.topk_order == "value"
    pri = torch.from_numpy(_topk_input(np, n, k, args.topk_input)).cuda()
    if args.calibrate_copy:
        _calibrate_copy(torch, ops)
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
          for _ in range(args.steps)]

    # --topk-warm: every call after the first starts from the bound the call before it left in the
    # workspace (gear_hip_topk_f32_warm), as a loop over a slowly changing array does
    state = ops.TopKState() if args.topk_warm else None

    def select():
        if state is not None:
            return state.select(pri, k, sorted_by_value=by_value)
        return ops.topk(pri, k, sorted_by_value=by_value)

    def step(i, slot):
        if slot is not None:
            ev[slot][0].record()
        select()
        if slot is not None:
            ev[slot][1].record()

    ms = _time_steps(torch, step, args.steps, args.warmup)
    sms = sorted(a.elapsed_time(b) for a, b in ev)
    avg = sum(sms) / len(sms)
    alg = 4 * n + 12 * k

    def timed_us(fn, reps=50):
        for _ in range(5):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) / reps * 1e3

    yard = {"back_to_back_us": timed_us(select),
            "torch_topk_us": timed_us(lambda: torch.topk(pri, k, sorted=by_value), reps=10),
            "torch_sum_read_only_us": timed_us(lambda: pri.sum()),
            "what": "HIP events around back-to-back launches, same n and k; torch.topk is the "
                    "library selection, pri.sum() one read of the priorities (two launches)"}
    return _line(n / (ms * 1e-3), "priorities/s", args, ms,
                 "topk: top %d of %d fp32 priorities (%s), ordered by %s%s" %
                 (k, n, args.topk_input, args.topk_order, ", warm calls" if args.topk_warm else ""),
                 {"bound": "hbm", "kernel": "top-k chain (prep, level0, member_hist x2, count, "
                                            "write" + (", segment_sort)" if by_value else ")"),
                  "achieved": alg / (avg * 1e-3) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                  "frac": alg / (avg * 1e-3) / 1e9 / HBM_PEAK_GBPS, "avg_launch_ms": avg,
                  "median_launch_ms": sms[len(sms) // 2], "algorithmic_bytes": alg,
                  "traffic": None}, {"yardsticks": yard})


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--trajectories", type=int, default=1000,
                    help="config 4: trajectories of 1000 steps in the table (1000 = full size)")
    ap.add_argument("--workload", default="config4",
                    choices=["config1", "config2", "config3", "config4", "config5", "scan", "topk"],
                    help="benchmark config to run (config4 is the bench line); scan and topk run "
                         "one maintenance kernel chain on its own, for profiles")
    ap.add_argument("--n", type=int, default=10_000_000, help="scan / topk: number of priorities")
    ap.add_argument("--k", type=int, default=65_536, help="topk: entries kept")
    ap.add_argument("--no-hostlink", action="store_true",
                    help="config4: skip the bounded config-5 host-link sub-record")
    ap.add_argument("--hostlink-trajectories", type=int, default=150,
                    help="config4: trajectories (28.2 MB each) of the pinned table of that sub-record")
    ap.add_argument("--topk-order", default="value", choices=["value", "index"])
    ap.add_argument("--topk-input", default="lognormal", choices=sorted(TOPK_INPUTS),
                    help="topk: the shape of the priorities; " +
                         "; ".join("%s = %s" % kv for kv in sorted(TOPK_INPUTS.items())))
    ap.add_argument("--topk-warm", action="store_true",
                    help="topk: calls after the first take up the previous call's bound")
    ap.add_argument("--trajectories3", type=int, default=100_000,
                    help="config 3: number of trajectories (100000 = full size, 10.4 GB)")
    ap.add_argument("--trajectories5", type=int, default=2000,
                    help="config 5: trajectories of 1000 steps in pinned host memory (2000 = 56.5 GB)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-pipelined", action="store_true",
                    help="config 4: skip the pipelined pass over the same steps and the copy yardsticks")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three 1 GiB plain copies (slices kernel) before the steps")
    ap.add_argument("--traffic-bytes", type=float, default=None,
                    help="measured HBM bytes per gather launch (from rocprofv3 --pmc runs)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the hot path on ONE GPU only; --gpus %d is not supported"
              % args.gpus, file=sys.stderr)
        sys.exit(2)
    runner = {"config1": run_config1, "config2": run_config2, "config3": run_config3,
              "config4": run_config4, "config5": run_config5, "scan": run_scan,
              "topk": run_topk}[args.workload]
    result = runner(args)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
