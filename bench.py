#!/usr/bin/env python3
"""Benchmark of the fused Hessian assemble + tree L'DL + solve on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the hot path over one synthetic batch of the headline shape: humanoid,
nv = 27, nefc = 64, 4096 worlds, three Newton iterations with a fresh active mask each -- three
calls of im_assemble_tree_ldl_solve, one launch per solve, which is the form a Newton loop can
issue (an iteration's states come out of the one before).  Inputs are resident in HBM before the
timed region; every launch takes the next of 16 distinct input sets (> 560 MB in rotation), so no
launch finds its M or J in the 256 MB memory-side cache.  `value` and `roofline` are this form's.
Beside it, `iterations_launch`: the three solves of a step as one launch of
im_assemble_tree_ldl_solve_iters (a grid over worlds x iterations, for callers that know every
iteration's states in advance; the solves are then independent of one another), and `newton_solve`:
whole constraint solves of the same batch shape with dependent iterations (init_context, the resident
Newton kernel, force recovery) with the fused tree stage, and `newton_solve_dense_stage`: the same with
the single-tile dense stage of the reference's own loop; both informative.  Prints one JSON line.
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
# HBM bytes per launch of the iterations kernel (3 solves x 4096 worlds) from two rocprofv3 --pmc
# runs (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads
# for a plain 64 MiB device copy in the same run; recorded in
# profiles/tree_row16_humanoid_pmc.txt:  (18296.13 * 65536 / 32781.84 + 1344.0) KiB
TRAFFIC_BYTES_PER_LAUNCH = int((18296.13 * 65536 / 32781.84 + 1344.0) * 1024)
# the same for one launch of the single-solve kernel (4096 worlds):  (15566.21 * 65536 / 32781.84 + 448.0) KiB
TRAFFIC_BYTES_PER_SINGLE_LAUNCH = int((15566.21 * 65536 / 32781.84 + 448.0) * 1024)
MIN_TIMED_LAUNCHES = 256  # the kernel duration is averaged over at least this many launches


def algorithmic_bytes(nv: int, nM: int, nefc: int) -> int:
    """Bytes one world*solve has to move: M, J, D, state, grad in; x out (fp32/int32)."""
    return 4 * (nM + nefc * nv + nefc + nefc + nv) + 4 * nv


def algorithmic_bytes_fused(nv: int, nM: int, nefc: int, iters: int) -> int:
    """Bytes of one world over `iters` fused solves when M and J are counted once per launch."""
    return 4 * (nM + nefc * nv) + iters * 4 * (2 * nefc + 2 * nv)


def cpu_baseline(batch, plan_struct, gpu_x, seconds: float = 10.0):
    """The CPU oracle (a C restatement of the reference path, OpenMP over worlds) timed on this
    host's cores on the same workload: all threads, then one thread.  As the checker it also
    compares what the GPU computed for the first input set of the benchmarked batch (`gpu_x`,
    (iterations, worlds, nv), every world) with its own result, bit for bit."""
    import numpy as np

    from oracle import planner as P
    from oracle import ref as R

    st = plan_struct
    plan = P.best_tree_ldl_plan(*st)
    threads = R.max_threads()
    iters = batch.state.shape[0]
    n = gpu_x.shape[1]
    for it in range(iters):  # every world of the first input set
        want = R.assemble_tree_ldl_solve(*st, plan, batch.M[:n], batch.J[:n], batch.D[:n], batch.state[it][:n], batch.nefc[:n], batch.grad[:n])
        if not np.array_equal(gpu_x[it], want):
            raise RuntimeError(f"the benchmarked kernel disagrees with the CPU restatement in iteration {it}")

    def timed(nworld: int, budget: float):
        M, J, D, ne, g = batch.M[:nworld], batch.J[:nworld], batch.D[:nworld], batch.nefc[:nworld], batch.grad[:nworld]

        def one_pass():
            for it in range(iters):
                R.assemble_tree_ldl_solve(*st, plan, M, J, D, batch.state[it][:nworld], ne, g)

        one_pass()
        t0 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t0 < budget or reps < 2:
            one_pass()
            reps += 1
        dt = time.perf_counter() - t0
        return reps * iters * nworld / dt, reps, dt

    rate_all, reps_all, dt_all = timed(batch.nworld, seconds)
    R.set_threads(1)
    try:
        rate_one, reps_one, dt_one = timed(min(batch.nworld, 512), seconds / 2)
    finally:
        R.set_threads(threads)
    return {
        "value": rate_all,
        "unit": "world*solves/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{reps_all} passes of the same {batch.nworld}-world x {iters}-iteration batch ({dt_all:.1f} s), all {threads} OpenMP threads",
        "single_core_value": rate_one,
        "single_core_sample": f"{reps_one} passes over the first {min(batch.nworld, 512)} worlds ({dt_one:.1f} s), 1 thread",
    }


def newton_solve_leg(torch, use_graph: bool, stage: str = "tree", nsets: int = 8, replays: int = 5, solves_per_replay: int = 8):
    """Beside the headline: whole constraint solves of the same batch shape with dependent iterations
    (newton_fusion.solve: init_context, the resident Newton kernel with the fused tree stage -- or,
    ``stage="dense"``, with the single-tile dense stage that the reference's own loop runs at this
    size -- and the force recovery; tolerance 1e-7, at most 10 iterations), on rotating input sets.
    Informative: the headline's metric is the factor-and-solve launch."""
    from instantmimic_amd.mjw_kernels import newton_fusion as NF
    from instantmimic_amd.rowbench import newton_case

    cases = [newton_case("humanoid", stage, seed=21 + k) for k in range(nsets)]
    for c in cases[:2]:
        NF.solve(*c)
    torch.cuda.synchronize()
    its = cases[0][1].solver_niter.cpu().numpy()
    unfinished = int((cases[0][2].done.cpu().numpy() == 0).sum())
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    times = []
    if use_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        g = torch.cuda.CUDAGraph()
        with torch.cuda.stream(side):
            with torch.cuda.graph(g, stream=side):
                for k in range(solves_per_replay):
                    NF.solve(*cases[k % nsets])
        torch.cuda.current_stream().wait_stream(side)
        g.replay()
        torch.cuda.synchronize()
    for _ in range(replays):
        a.record()
        if use_graph:
            g.replay()
        else:
            for k in range(solves_per_replay):
                NF.solve(*cases[k % nsets])
        b.record()
        torch.cuda.synchronize()
        times.append(a.elapsed_time(b) * 1e-3 / solves_per_replay)
    sec = min(times)
    m, d = cases[0][0], cases[0][1]
    return {
        "entry": ("newton_fusion.solve: im_newton_init_context, im_newton_tree_stage, im_newton_solve_tree (one resident kernel for the dependent iterations), im_qfrc_constraint_from_grad"
                  if stage == "tree" else
                  "newton_fusion.solve: im_newton_init_context, im_dense_init_factor, im_newton_solve_dense_tile (one resident kernel for the dependent iterations), im_qfrc_constraint_from_grad"),
        "workload": f"humanoid nv={int(m.nv)} nefc={int(d.njmax)} x {int(d.nworld)} worlds, tolerance 1e-7, at most {int(m.opt.iterations)} iterations",
        "us_per_solve": sec * 1e6,
        "iterations_mean": float(its.mean()),
        "iterations_max": int(its.max()),
        "worlds_unfinished": unfinished,
        "world_iterations_per_s": float(its.sum()) / sec,
        "input_sets": nsets,
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=320)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--sets", type=int, default=16, help="distinct input sets rotated over")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-solve", action="store_true", help="skip the whole-solve figure (newton_solve)")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying hipGraphs")
    ap.add_argument("--single-only", action="store_true", help="time the one-launch-per-solve form only (for profiles of that kernel)")
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
        sets.append((M, J, D, st, ne, g, torch.zeros((iters, nworld, nv), device=dev)))
    torch.cuda.synchronize()

    def step(s: int) -> None:
        M, J, D, st, ne, g, x = sets[s % nsets]
        T.assemble_tree_factor_solve_iters(scratch, M, J, D, st, ne, g, x)

    def step_single(s: int) -> None:
        # the same work as one launch per iteration, every launch on another input set
        for it in range(iters):
            M, J, D, st, ne, g, x = sets[(s * iters + it) % nsets]
            T.assemble_tree_factor_solve(scratch, M, J, D, st[it], ne, g, x[it])

    # both forms once on set 0 (the batch as generated), checked against the CPU restatement in the CPU leg:
    # every world of every iteration
    step(0)
    torch.cuda.synchronize()
    x_first = sets[0][6].cpu().numpy().copy()
    sets[0][6].zero_()
    for it in range(iters):
        M, J, D, st, ne, g, x = sets[0]
        T.assemble_tree_factor_solve(scratch, M, J, D, st[it], ne, g, x[it])
    torch.cuda.synchronize()
    if not np.array_equal(sets[0][6].cpu().numpy(), x_first):
        raise RuntimeError("one launch per solve and the iterations launch disagree")

    use_graph = not args.no_graph

    MAX_GRAPH_STEPS = 1024  # steps recorded in one graph; longer runs replay it several times

    def runner(fn):
        """`run(n)`: n steps over the rotation of input sets.  With graphs, the steps of a run are
        one graph (recorded and replayed once when `prepare(n)` is called, outside any timed
        region), so that a timed region is one graph launch whatever its length."""
        graphs = {}
        if use_graph:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                for s in range(nsets):
                    fn(s)
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()

        def prepare(nsteps: int) -> None:
            n = min(nsteps, MAX_GRAPH_STEPS)
            if not use_graph or n <= 0 or n in graphs:
                return
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g):
                for s in range(n):
                    fn(s)
            g.replay()  # the first replay of a graph also uploads it
            torch.cuda.synchronize()
            graphs[n] = g

        def run(nsteps: int) -> None:
            if not use_graph:
                for i in range(nsteps):
                    fn(i)
                return
            left = nsteps
            while left > 0:
                n = min(left, MAX_GRAPH_STEPS)
                prepare(n)
                graphs[n].replay()
                left -= n

        run.prepare = prepare
        return run

    def region(run, nsteps: int):
        """Wall time and HIP-event time (on the stream the kernels are launched on: torch's
        current stream is the one handed to the C ABI) of `nsteps` steps."""
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record()
        run(nsteps)
        ev1.record()
        torch.cuda.synchronize()
        return time.perf_counter() - t0, ev0.elapsed_time(ev1) * 1e-3

    def spread(run, launches_per_step: int, regions: int = 32, steps_per_region: int = 8):
        """Median, 10th and 90th percentile of the per-launch duration over `regions` timed regions of
        `steps_per_region` steps each (HIP events around every region)."""
        run.prepare(steps_per_region)
        per = []
        for _ in range(regions):
            _, ev = region(run, steps_per_region)
            per.append(ev / (steps_per_region * launches_per_step) * 1e6)
        per.sort()
        return {"median": per[len(per) // 2], "p10": per[len(per) // 10], "p90": per[(9 * len(per)) // 10], "regions": regions,
                "launches_per_region": steps_per_region * launches_per_step}

    B = algorithmic_bytes(nv, nM, nefc)
    B3 = algorithmic_bytes_fused(nv, nM, nefc, iters)

    # ---- the headline: one launch per solve, three launches per step
    run_single = runner(step_single)
    n_kernel = max(args.steps, -(-MIN_TIMED_LAUNCHES // iters))
    for n in (args.warmup, args.steps, n_kernel):
        run_single.prepare(n)
    run_single(max(args.warmup, 1))
    elapsed, _ = region(run_single, args.steps)
    value = args.steps * iters * nworld / elapsed
    _, ev_kernel = region(run_single, n_kernel)  # the kernel's duration from a region whose length does not depend on --steps
    kernel_s = ev_kernel / (n_kernel * iters)  # one launch = one solve of every world
    achieved = B * nworld / kernel_s / 1e9
    if args.single_only:
        print(json.dumps({"single_launch": {"kernel_us": kernel_s * 1e6, "frac": achieved / HBM_PEAK_GBS}}))
        return 0

    # ---- beside it: the step's three solves as one launch over (worlds x iterations)
    run_iters = runner(step)
    n_iters = max(args.steps, MIN_TIMED_LAUNCHES)
    run_iters.prepare(n_iters)
    run_iters(max(args.warmup, 1))
    _, ev_iters = region(run_iters, n_iters)
    iters_s = ev_iters / n_iters
    iterations_launch = {
        "entry": "im_assemble_tree_ldl_solve_iters: three independent solves per launch (every iteration's states known before the launch)",
        "kernel_us": iters_s * 1e6,
        "us_per_solve": iters_s * 1e6 / iters,
        "launches_timed": n_iters,
        "kernel_us_spread": spread(run_iters, 1),
        "world_solves_per_s": iters * nworld / iters_s,
        "frac_per_solve_bytes": B * iters * nworld / iters_s / 1e9 / HBM_PEAK_GBS,
        "frac_per_solve_bytes_definition": f"{B} bytes x {iters} solves x {nworld} worlds per launch: every solve counted as if it read M and J itself, which the launch does not do",
        "frac_fused_bytes": B3 * nworld / iters_s / 1e9 / HBM_PEAK_GBS,
        "frac_fused_bytes_definition": f"B3 = {B3} bytes per world and launch: M and J once, state / D / gradient / x per iteration",
        "traffic": TRAFFIC_BYTES_PER_LAUNCH,
    }

    newton = None if args.no_solve else newton_solve_leg(torch, use_graph)
    newton_dense = None if args.no_solve else newton_solve_leg(torch, use_graph, stage="dense")

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
            "workload": f"humanoid nv={nv} nM={nM} nefc={nefc} x {nworld} worlds, {iters} Newton iterations per step with a fresh active mask each, one launch per solve (im_assemble_tree_ldl_solve), every launch on an input set of its own",
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
            "traffic": TRAFFIC_BYTES_PER_SINGLE_LAUNCH,
            "kernel_us": kernel_s * 1e6,
            "kernel_us_spread": spread(run_single, iters),
            "launches_timed": n_kernel * iters,
            "solves_per_launch": 1,
            "bytes_definition": f"B = {B} bytes per world*solve (M, J, D, state, gradient in; x out) x {nworld} worlds per launch",
            "throughput_frac": (B * value / 1e9) / HBM_PEAK_GBS,
        },
        "iterations_launch": iterations_launch,
    }
    if newton is not None:
        out["newton_solve"] = newton
        out["newton_solve_dense_stage"] = newton_dense
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(batch, T.tree_ldl_structure(batch.rowadr, batch.rownnz, batch.colind), x_first)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
