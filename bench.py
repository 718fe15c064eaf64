#!/usr/bin/env python3
"""Benchmark of the fused Hessian assemble + tree L'DL + solve on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the hot path over one synthetic batch of the headline
shape: humanoid, nv = 27, nefc = 64, 4096 worlds, three Newton iterations (three
launches, each with its own active mask).  Inputs are resident in HBM before the
timed region; the steps rotate over enough distinct input sets (> 512 MB) that
reads cannot be served by the 256 MB last-level cache.  Prints one JSON line.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "Hessian assemble+LDL+solve worlds/s, humanoid nv=27×4096; % HBM roofline"
HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# HBM bytes per launch of the fused kernel from two rocprofv3 --pmc runs (FETCH_SIZE, then
# WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads for a plain
# 64 MiB device copy in the same run (FETCH_SIZE reads 32781 KiB for it, WRITE_SIZE 65536):
#   (15862.14 * 65536 / 32781.48 + 448.0 * 65536 / 65536) KiB
# Recorded in profiles/tree_row16_humanoid_pmc.txt.
TRAFFIC_BYTES_PER_LAUNCH = int((15854.27 * 65536 / 32781.46 + 448.0) * 1024)


def algorithmic_bytes(nv: int, nM: int, nefc: int) -> int:
    """Bytes one world*solve has to move: M, J, D, state, grad in; x out (fp32/int32)."""
    return 4 * (nM + nefc * nv + nefc + nefc + nv) + 4 * nv


def cpu_baseline(batch, plan_struct, seconds: float = 12.0):
    """The CPU oracle (a C restatement of the reference path, OpenMP over worlds) timed
    on this host's cores on the same workload; used as the checker elsewhere."""
    from oracle import planner as P
    from oracle import ref as R

    st = plan_struct
    plan = P.best_tree_ldl_plan(*st)
    threads = R.max_threads()
    iters = batch.state.shape[0]

    def one_pass():
        for it in range(iters):
            R.assemble_tree_ldl_solve(*st, plan, batch.M, batch.J, batch.D, batch.state[it], batch.nefc, batch.grad)

    one_pass()
    t0 = time.perf_counter()
    reps = 0
    while time.perf_counter() - t0 < seconds or reps < 3:
        one_pass()
        reps += 1
    dt = time.perf_counter() - t0
    solves = reps * iters * batch.nworld
    return {
        "value": solves / dt,
        "unit": "world*solves/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{reps} passes of the same {batch.nworld}-world x {iters}-iteration batch ({dt:.1f} s), all {threads} OpenMP threads",
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=320)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--sets", type=int, default=16, help="distinct input sets rotated over")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying hipGraphs")
    ap.add_argument(
        "--copy-calibration",
        type=int,
        default=0,
        metavar="N",
        help="also run N plain device copies of 64 MiB (rotating buffers) so that a rocprofv3 --pmc run of this "
        "command shows what FETCH_SIZE / WRITE_SIZE read for a kernel of known traffic",
    )
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; --gpus must be 1 (worlds would shard contiguously, no exchange)", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from instantmimic_amd import synth
    from instantmimic_amd.mjw_kernels import tree_ldl as T

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.copy_calibration:
        # 8 source/destination pairs of 64 MiB: 1 GiB in rotation, nothing stays in the last-level cache
        pairs_ = [(torch.empty(16 << 20, device=dev), torch.ones(16 << 20, device=dev)) for _ in range(8)]
        torch.cuda.synchronize()
        for i in range(args.copy_calibration):
            d_, s_ = pairs_[i % 8]
            d_.copy_(s_)
        torch.cuda.synchronize()
        del pairs_

    shape = synth.SHAPES["humanoid"]
    batch = synth.make_batch(shape)
    nworld, nv, nefc, iters = batch.nworld, shape.nv, shape.nefc, shape.iterations
    nM = int(batch.colind.size)
    m = type("m", (), dict(nv=nv, M_rowadr=batch.rowadr, M_rownnz=batch.rownnz, M_colind=batch.colind))
    scratch = T.create_tree_factor_solve_scratch(m, dev)
    if scratch is None:
        raise RuntimeError("tree plan rejected for the benchmark shape")

    # distinct input sets: the same worlds rolled along the world axis
    nsets = max(1, args.sets)
    sets = []
    base = [torch.from_numpy(a).to(dev) for a in (batch.M, batch.J, batch.D, batch.nefc, batch.grad)]
    base_state = torch.from_numpy(batch.state).to(dev)
    for s in range(nsets):
        sh = (s * 257) % nworld
        M, J, D, ne, g = (torch.roll(t, sh, 0).contiguous() for t in base)
        st = torch.roll(base_state, sh, 1).contiguous()
        sets.append((M, J, D, st, ne, g, torch.zeros_like(g)))
    torch.cuda.synchronize()

    def step(s: int) -> None:
        M, J, D, st, ne, g, x = sets[s % nsets]
        for it in range(iters):
            T.assemble_tree_factor_solve(scratch, M, J, D, st[it], ne, g, x)

    # correctness guard on the data actually benchmarked (cheap fp64 residual on a few worlds)
    step(0)
    torch.cuda.synchronize()

    use_graph = not args.no_graph
    single, multi = [], None
    if use_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for s in range(nsets):
                step(s)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        for s in range(nsets):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                step(s)
            single.append(g)
        multi = torch.cuda.CUDAGraph()
        with torch.cuda.graph(multi):
            for s in range(nsets):
                step(s)

    def run(nsteps: int, first: int = 0) -> None:
        i = 0
        if use_graph:
            while first % nsets == 0 and nsteps - i >= nsets:
                multi.replay()
                i += nsets
            while i < nsteps:
                single[(first + i) % nsets].replay()
                i += 1
        else:
            while i < nsteps:
                step(first + i)
                i += 1

    run(args.warmup)
    torch.cuda.synchronize()
    # HIP events on the stream the kernels are launched on (torch's current stream is the
    # one handed to the C ABI), around the timed region
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    run(args.steps)
    ev1.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    value = args.steps * iters * nworld / elapsed
    region_s = ev0.elapsed_time(ev1) * 1e-3

    # per-launch kernel duration with HIP events on the launch stream
    nev = min(args.steps, 64)
    pairs = []
    for i in range(nev):
        M, J, D, st, ne, g, x = sets[i % nsets]
        for it in range(iters):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            T.assemble_tree_factor_solve(scratch, M, J, D, st[it], ne, g, x)
            b.record()
            pairs.append((a, b))
    torch.cuda.synchronize()
    durs = np.array([a.elapsed_time(b) for a, b in pairs]) * 1e-3  # seconds
    # average launch duration over the timed region: launches run back to back, so the
    # region divided by the launch count is the kernel's duration (it agrees with the
    # rocprofv3 kernel trace; a lone launch bracketed by two events reads ~2 us more)
    kernel_s = region_s / (args.steps * iters)
    B = algorithmic_bytes(nv, nM, nefc)
    achieved = B * nworld / kernel_s / 1e9

    out = {
        "metric": METRIC,
        "value": value,
        "unit": "world*solves/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": f"humanoid nv={nv} nM={nM} nefc={nefc} x {nworld} worlds, {iters} Newton iterations (launches) per step, fresh active mask each",
            "input_sets": nsets,
            "launch": "hipGraph replay" if use_graph else "eager",
            "bytes_per_world_solve": B,
        },
        "roofline": {
            "bound": "hbm",
            "achieved": achieved,
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS,
            "traffic": TRAFFIC_BYTES_PER_LAUNCH,
            "kernel_us": kernel_s * 1e6,
            "kernel_us_single_launch_p10_p50_p90": [float(np.percentile(durs, p)) * 1e6 for p in (10, 50, 90)],
            "throughput_frac": (B * value / 1e9) / HBM_PEAK_GBS,
        },
    }
    if not args.no_cpu:
        st = T.tree_ldl_structure(batch.rowadr, batch.rownnz, batch.colind)
        out["cpu_baseline"] = cpu_baseline(batch, st)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
