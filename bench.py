#!/usr/bin/env python3
"""Benchmark of the replay-sampling hot path on one MI355X.

    python bench.py --gpus 1 --steps K --warmup W

A step is one pass of the hot path over one batch: prefix sum of the per-step priorities, search
of the batch's seeded uniforms, sort of the drawn indices, split into (trajectory, timestep) and
the gather of all columns of the windows into contiguous batch tensors.  The default workload is
BASELINE config 4 (Atari-shape table resident in HBM, 2048 windows of 30 steps).  Rank 0 prints
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
MEASURED_GATHER_TRAFFIC_BYTES = 3536154859


def log(msg):
    print("[bench] " + msg, file=sys.stderr, flush=True)


class AtariTable:
    """BASELINE config 4 / 5 schema: obs uint8[4,84,84], action int32, reward fp32, done uint8."""
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
    gather_ms = sum(a.elapsed_time(b) for a, b in ev) / args.steps

    payload = B * span * sum(tab.step_bytes)
    alg_bytes = 2 * payload  # every gathered byte is read once and written once
    achieved = alg_bytes / (gather_ms * 1e-3) / 1e9
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
        "step_GBps": alg_bytes / (ms_per_step * 1e-3) / 1e9,
        "step_frac_of_hbm_peak": alg_bytes / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBPS,
        "roofline": {"bound": "hbm", "kernel": "subcopy_multi_kernel", "achieved": achieved,
                     "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBPS,
                     "avg_launch_ms": gather_ms, "algorithmic_bytes": alg_bytes,
                     "traffic": args.traffic_bytes if args.traffic_bytes is not None else
                     (MEASURED_GATHER_TRAFFIC_BYTES if cap == 1000 else None)},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline_config4(np, torch, tab, table, pri, B, span, ofst)
    return result


def cpu_baseline_config4(np, torch, tab, table, pri, B, span, ofst):
    """The CPU oracle (a single-threaded C restatement of the reference's host path) on a bounded
    sample: the same priorities and batch shape, the table restricted to its first trajectories."""
    from oracle import oracle as orc
    keep = min(64, tab.capacity)
    host = table[:keep * tab.traj_stride].cpu().numpy()
    T = tab.T
    rng = np.random.default_rng(3004)
    dsts = [np.zeros((B, span * sb), np.uint8) for sb in tab.step_bytes]
    nrun, t_total = 0, 0.0
    budget = 12.0
    while nrun < 3 or (t_total < budget and nrun < 20):
        u01 = rng.random(B, dtype=np.float32)
        t0 = time.perf_counter()
        prefix = orc.scan_f32_f64(pri)
        flat = orc.upper_bound_f64(prefix, u01, unit_uniforms=True)
        flat = orc.sort_i64(flat)
        idxs = (flat // T) % keep
        tss = flat % T
        lens = tss + 1
        for c in range(4):
            orc.subcopy(host, idxs, tss, lens, True, ofst, span, tab.traj_stride,
                        tab.step_bytes[c], tab.col_base(c), zero_fill=True, dst=dsts[c])
        t_total += time.perf_counter() - t0
        nrun += 1
    return {"value": B * nrun / t_total, "unit": "windows/s", "cores": 1, "kind": "port",
            "ms_per_step": t_total / nrun * 1e3,
            "sample": "%d steps of the same pipeline (fp64 scan of 1e6 priorities, 2048 searches, "
                      "sort, 4-column gather with memset+memcpy per window) on the first %d of %d "
                      "trajectories (%.1f GB of the table, trajectory index taken modulo %d); "
                      "host has %d logical cores, 1 used"
                      % (nrun, keep, tab.capacity, keep * tab.traj_stride / 1e9, keep,
                         os.cpu_count() or 0)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--trajectories", type=int, default=1000,
                    help="config 4: trajectories of 1000 steps in the table (1000 = full size)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three 1 GiB plain copies (slices kernel) before the steps")
    ap.add_argument("--traffic-bytes", type=float, default=None,
                    help="measured HBM bytes per gather launch (from rocprofv3 --pmc runs)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the hot path on ONE GPU only; --gpus %d is not supported"
              % args.gpus, file=sys.stderr)
        sys.exit(2)
    result = run_config4(args)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
