#!/usr/bin/env python3
"""Benchmark of the batched plan evaluator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--no-cpu] [--no-sa]
    python bench.py --config 5 [--chains 64] [--sa-steps 2000]      (batched simulated annealing)

A step is one pass of the hot path (signature kernel, class grouping, evaluation kernel) over the
whole seeded candidate set of the configuration (config 2: 65,536 GRPO plans), with the plan
tensors already resident in HBM and the results left in HBM.  Prints one JSON line.
"""

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E, published
FP64_PEAK_TFLOPS = 78.6     # MI355X vector FP64, published
ISSUE_PEAK = 256 * 4 * 2.4e9   # wave-instructions per second: 256 CUs x 4 SIMDs x 2.4 GHz, one instruction per clock
# algorithmic bytes per plan: int16 plan fields (10 per vertex) + 4 header bytes in, 3 doubles + 1 mask byte out
ALG_BYTES = {1: 149, 2: 109, 3: 149, 4: 89, 5: 149}
# fp64 operations per plan (additions, multiplications, divisions, comparisons incl. max/min, 2 per fused
# multiply-add), counted by oracle/flop_count.cpp (the kernels' arithmetic compiled with a counting number
# type) and averaged over the seeded set of the configuration (config 5: over 4,096 seeded plans);
# tests/test_cpu_port.py holds these constants to a fresh count
ALG_FLOPS = {1: 3697.0, 2: 2165.3, 3: 6502.9, 4: 1245.8, 5: 4155.6}
# Counter figures of one step.  A run cannot read hardware counters of itself: these come from the rocprofv3 --pmc
# summaries under profiles/ and are printed only when the run's kernel layout (`layout`: wave tasks, LDS bytes, plans
# per wavefront with LDS state, single-plan tasks, four-lanes-per-plan tasks of rpeg_engine_stats) is the profiled
# one to within 5 % in every task count; any other run prints null.  HBM bytes of the evaluation kernels
# (FETCH_SIZE / WRITE_SIZE scaled by a 256 MiB copy) and instructions issued per plan (SQ_INSTS_VALU + SALU + LDS +
# VMEM_RD + VMEM_WR of the evaluation kernels / plans).
MEASURED = {
    2: dict(layout=(6330, 17648, 0, 4815, 574), traffic=209.8e6, instructions_per_plan=3157.5),
    3: dict(layout=(24672, 29984, 0, 20364, 0), traffic=4639.9e6, instructions_per_plan=None),
    4: dict(layout=(16396, 14640, 0, 6, 0), traffic=1547.6e6, instructions_per_plan=None),
}


def cpu_baseline(cfg, batch, seconds=12.0):
    """The Python oracle (restatement of the reference's pure-Python path) on one core, on the first
    plans of the same candidate set, for about `seconds`."""
    from oracle import rpeg_oracle as oracle
    p = cfg.problem
    t0 = time.perf_counter()
    done = 0
    while done < batch.n and time.perf_counter() - t0 < seconds:
        rpeg, plan, wl = batch.configuration(p, done)
        oracle.evaluate_plan(rpeg, plan, p.device_space, p.suite, wl, p.hw, p.K_eval, p.memory_policy)
        done += 1
    dt = time.perf_counter() - t0
    return dict(value=done / dt, unit="plan evals/s", cores=1, kind="port",
                sample=f"first {done} plans of the same seeded set, Python oracle, 1 process, {dt:.1f} s")


def _pool_worker(i):
    from oracle import rpeg_oracle as oracle
    cfg, batch = _POOL_STATE
    p = cfg.problem
    rpeg, plan, wl = batch.configuration(p, i)
    return oracle.evaluate_plan(rpeg, plan, p.device_space, p.suite, wl, p.hw, p.K_eval, p.memory_policy)["score"]


_POOL_STATE = None


def cpu_pool_baseline(cfg, batch, seconds=10.0, workers=None):
    """The same Python oracle behind multiprocessing.Pool(min(6, cores)) with a blocking map over the
    candidates of a step, as the reference dispatches them (RPEG/search/optimizer.py:414-417, 793-798).
    Must run before the process touches the GPU (the workers are forked)."""
    import multiprocessing as mp
    global _POOL_STATE
    workers = workers or min(6, os.cpu_count() or 1)
    _POOL_STATE = (cfg, batch)
    done, chunk = 0, 6 * workers
    with mp.get_context("fork").Pool(workers) as pool:
        pool.map(_pool_worker, range(chunk))          # start-up and imports are not timed
        t0 = time.perf_counter()
        while done + chunk <= batch.n and time.perf_counter() - t0 < seconds:
            pool.map(_pool_worker, range(done, done + chunk))
            done += chunk
        dt = time.perf_counter() - t0
    return dict(value=done / dt, unit="plan evals/s", cores=workers, kind="port",
                sample=f"first {done} plans, Python oracle behind multiprocessing.Pool({workers}), blocking map of "
                       f"{chunk} plans at a time, {dt:.1f} s")


def cxx_port(cfg, batch, threads):
    """Host build of the kernels' arithmetic on all host cores; returns the figure and the results."""
    from oracle.cpu_port import CpuPort
    from rpeg_amd.engine import abi
    port = CpuPort(cfg.problem)
    port.eval(batch.slice(0, 256), threads=threads)
    t0 = time.perf_counter()
    ref = port.eval(batch, flags=abi.GATE_STALE, threads=threads)
    dt = time.perf_counter() - t0
    return dict(value=batch.n / dt, unit="plan evals/s", cores=threads,
                sample=f"all {batch.n} plans, host build of the kernels' arithmetic (OpenMP), lowering included"), ref


def parity_block(out, ref):
    """The timed GPU results against the host build's on the same plans: masks, every score, ranking, best plan."""
    import numpy as np
    ok = np.isfinite(ref["score"]) & np.isfinite(out["score"])
    rel = np.abs(out["score"][ok] - ref["score"][ok]) / np.maximum(np.abs(ref["score"][ok]), 1e-300)
    rel_m = np.abs(out["makespan"][ok] - ref["makespan"][ok]) / np.maximum(np.abs(ref["makespan"][ok]), 1e-300)
    return dict(
        against="host build of the same arithmetic (oracle/cpu_port.cpp), which the CPU tests tie to the reference's vectors",
        plans=int(len(ref["score"])),
        mask_equal=bool(np.array_equal(out["mask"], ref["mask"])),
        scores_bit_equal=bool(np.array_equal(out["score"].view(np.uint64), ref["score"].view(np.uint64))),
        ranking_equal=bool(np.array_equal(np.argsort(-out["score"], kind="stable"), np.argsort(-ref["score"], kind="stable"))),
        argmax_equal=bool(int(np.nanargmax(out["score"])) == int(np.nanargmax(ref["score"]))),
        max_rel_err=float(max(rel.max() if rel.size else 0.0, rel_m.max() if rel_m.size else 0.0)))


def sa_measure(args, deadlines=True):
    """Config 5: `args.chains` chains x `args.sa_steps` steps of batched simulated annealing on the GPU evaluator, the
    first steps of the same chains over the host build of the evaluator, and (deadlines=True) the serial optimize()
    loop under wall-clock deadlines.  Returns the fields of the config-5 line."""
    import zlib
    import numpy as np
    import torch
    from rpeg_amd import configs
    from rpeg_amd.engine.runtime import Engine
    from rpeg_amd.search.moves import build_candidate_directory, directory_arrays
    from rpeg_amd.search.optimizer import OptimizerConfig, optimize_chains, sa_params

    cfg = configs.config(5)
    p = cfg.problem
    opt = OptimizerConfig(K_x=6, T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=10)
    variants = [(0, 0), (1, 0)]          # actor staleness {0, 1}, critic {0}; chains alternate
    eng = Engine(p, "cuda:0")
    rpeg0 = p.template(0, ())
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    table, _ = build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, eng)
    arrays = directory_arrays(rpeg0, table)
    dir_s = time.perf_counter() - t0
    runs = []
    for rep in range(3):   # the first run lowers every class it meets
        res = optimize_chains(p, opt, args.chains, args.sa_steps, variants, seed=42, engine=eng, directory=arrays)
        runs.append(res)
    cold, warm = runs[0], runs[-1]
    c = cold.argbest()
    assert all((r.best_plan == cold.best_plan).all() and (r.best_score == cold.best_score).all() for r in runs)
    line = {
        "metric": "SA wall-clock, 64 chains x 2000 steps, to best plan", "value": cold.wall_s, "unit": "s",
        "n_gpus": 1, "steps": args.sa_steps, "warmup": 0, "ms_per_step": cold.wall_s / max(1, args.sa_steps) * 1e3,
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f64", "data": "synthetic",
        "config": {"workload": cfg.name, "chains": args.chains, "steps_per_chain": args.sa_steps, "K_x": opt.K_x,
                   "T_init": opt.T_init, "T_min": opt.T_min, "T_warm": opt.T_warm, "stag_window": opt.stag_window,
                   "seed": 42, "staleness_variants": variants, "memory_per_gpu": p.hw.memory_per_gpu},
        "time_to_best_s": float(cold.best_time[c]), "best_chain": c, "best_step": int(cold.best_step[c]),
        "best_score": float(cold.best_score[c]), "best_feasible": bool(cold.best_feasible[c]),
        "best_plan_crc": zlib.crc32(cold.best_plan[c].tobytes()),
        "plans_evaluated": int(cold.n_plans), "launches": int(cold.n_launch),
        "evals_per_s": cold.n_plans / cold.wall_s, "eval_share_of_wall": cold.eval_s / cold.wall_s,
        "wall_s_of_runs": [r.wall_s for r in runs], "warm_wall_s": warm.wall_s,
        "warm_time_to_best_s": float(warm.best_time[c]),
        "directory_s": dir_s, "directory_sizes": [int(a.shape[0]) for a in arrays],
        "accept_rate": float((((cold.log >> 4) & 3) == 2).sum() / max(1, (((cold.log >> 4) & 3) != 0).sum())),
        "restarts": int(cold.restarts.sum()), "dead_chains": int(cold.dead.sum()),
        "feasible_chains": int(cold.best_feasible.sum()),
    }
    split = 1 if p.workload.gen_quantiles else 0
    if deadlines:
        # optimize() as the reference runs it (one chain at a time, cache, restarts), under a wall-clock deadline as
        # `pipeline.py --time` sets it: the best score reached within t seconds, on the GPU evaluator and -- the same
        # loop, the same generator -- on the host build of the evaluator
        from rpeg_amd.engine import abi
        from rpeg_amd.search import candidates
        seeds = candidates.generate(p, 64, cfg.tau_choices, seed=42, tag=5)
        verdict = eng.eval(seeds)["mask"]
        start = next(i for i in range(seeds.n) if verdict[i] & abi.MASK_VALID and verdict[i] & abi.MASK_MEM_OK)
        row = np.ascontiguousarray(seeds.vert[:, start])

        def timed(seconds):
            prm = sa_params(opt, 1, 1, [(0, 0)], 0, split, 42)
            prm.timed, prm.deadline_s = 1, seconds
            return prm
        line["within_deadline"] = []
        for seconds in (0.1, 0.3, 1.0):
            r = eng.sa_optimize(timed(seconds), arrays, row, 10 ** 9, 10 ** 9, stream_key=(5, 0, 0))
            line["within_deadline"].append(dict(seconds=seconds, best_score=r["best_score"], best_feasible=r["best_feasible"],
                                                evaluations=r["E"], timed_out=r["timed_out"]))
    if not args.no_cpu:
        # the same host logic over the CPU build of the evaluator, all host cores, on a bounded number of steps
        from oracle.cpu_port import CpuPort
        threads = min(16, os.cpu_count() or 1)
        if deadlines:
            for rec in line["within_deadline"]:
                r = CpuPort(p).sa_optimize(timed(rec["seconds"]), arrays, row, 10 ** 9, 10 ** 9, stream_key=(5, 0, 0),
                                           threads=threads)
                rec.update(cpu_port_best_score=r["best_score"], cpu_port_evaluations=r["E"])
        steps = max(1, min(args.sa_steps, 40))
        t0 = time.perf_counter()
        ref = CpuPort(p).sa_run(sa_params(opt, args.chains, steps, variants, 0, split, 42), arrays, threads=threads)
        dt = time.perf_counter() - t0
        same = bool((ref["log"] == cold.log[:, :steps]).all())
        n_ev = int(ref["n_eval"].sum())
        line["cpu_baseline"] = dict(value=dt / steps * args.sa_steps, unit="s", cores=threads, kind="port",
                                    sample=f"first {steps} steps of the same {args.chains} chains over the host build "
                                           f"of the evaluator ({dt:.1f} s, {n_ev} evaluations), scaled to "
                                           f"{args.sa_steps} steps; same decisions as the GPU run: {same}")
        line["host_cores"] = os.cpu_count()
    else:
        line["cpu_baseline"] = None
    eng.close()
    return line


def bench_sa(args):
    """Prints the config-5 line: value = wall-clock of the whole run (directory build excluded, reported beside it)."""
    print(json.dumps(sa_measure(args)))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline legs")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MiB",
                    help="also run one device-to-device copy of this size (reference dispatch for scaling "
                         "FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--no-sa", action="store_true", help="leave the annealing run of config 5 out of the line")
    ap.add_argument("--chains", type=int, default=64)
    ap.add_argument("--sa-steps", type=int, default=2000)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path needs no second one (plans are independent: with more GPUs the "
                 "candidate tensor or the annealing chains would be split evenly across them). Use --gpus 1.")

    if args.config == 5:
        return bench_sa(args)

    from rpeg_amd import configs
    from rpeg_amd.search import candidates

    c = args.config
    cfg = configs.config(c)
    n = cfg.n_plans
    batch = candidates.generate(cfg.problem, n, cfg.tau_choices, seed=42, tag=c)
    # the CPU legs first: the pool forks its workers, which must happen before this process touches the GPU
    cpu = None
    if not args.no_cpu:
        cpu = dict(pool=cpu_pool_baseline(cfg, batch), one=cpu_baseline(cfg, batch))
        cpu["cxx"], cpu["ref"] = cxx_port(cfg, batch, threads=min(16, os.cpu_count() or 1))

    import torch
    from rpeg_amd.engine import abi
    from rpeg_amd.engine.runtime import DeviceBatch, Engine
    eng = Engine(cfg.problem, "cuda:0")
    db = DeviceBatch(batch, "cuda:0")
    out = eng.alloc_outputs(n)

    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eng.eval_device(db, out)
    torch.cuda.synchronize()
    first_call_ms = (time.perf_counter() - t0) * 1e3
    for _ in range(args.warmup):
        eng.eval_device(db, out)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    host_s = 0.0
    for _ in range(args.steps):
        h0 = time.perf_counter()
        eng.eval_device(db, out)
        host_s += time.perf_counter() - h0
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    value = n * args.steps / dt
    # run-to-run spread: the same number of steps again, each one bracketed by a synchronisation of its own
    each = []
    for _ in range(args.steps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.eval_device(db, out)
        torch.cuda.synchronize()
        each.append((time.perf_counter() - t0) * 1e3)
    host_us = eng.host_us()   # of the last of those calls
    each.sort()
    spread = {"min": each[0], "median": each[len(each) // 2], "max": each[-1],
              "note": "ms per step over the same number of steps run again, each synchronised on its own"}

    # duration of the evaluation launches (k_eval, k_plan, or the three side by side from fork to join): HIP events
    # on the launch stream, recorded by the library -- in the same steady state as the timed region above
    eng.set_timing(True)
    k_ms = []
    for _ in range(args.steps):
        eng.eval_device(db, out)
        k_ms.append(eng.last_kernel_ms())
    eng.set_timing(False)
    kernel_ms = sum(k_ms) / len(k_ms)
    stats = eng.stats()

    # cold steps: every class of the batch is lowered again inside the step
    cold_steps = max(1, min(args.steps, 5))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(cold_steps):
        eng.reset_classes()
        eng.eval_device(db, out)
    torch.cuda.synchronize()
    cold_ms = (time.perf_counter() - t0) / cold_steps * 1e3

    for _ in range(max(args.warmup, 8)):   # (the cold steps forgot what the engine had learned about its classes)
        eng.eval_device(db, out)

    if args.copy_probe:
        src = torch.ones(args.copy_probe << 20, dtype=torch.uint8, device="cuda:0")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()

    # two independent batches in flight: a second engine on a second stream, steps alternating between them,
    # so that the tail of one launch (its slowest wavefronts) overlaps the head of the next
    eng2 = Engine(cfg.problem, "cuda:0")
    out2 = eng2.alloc_outputs(n)
    s2 = torch.cuda.Stream()
    with torch.cuda.stream(s2):
        for _ in range(4):
            eng2.eval_device(db, out2)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for k in range(args.steps):
        if k & 1:
            with torch.cuda.stream(s2):
                eng2.eval_device(db, out2)
        else:
            eng.eval_device(db, out)
    torch.cuda.synchronize()
    two_stream = n * args.steps / (time.perf_counter() - t0)
    assert torch.equal(out2["score"].view(torch.int64), out["score"].view(torch.int64))
    eng2.close()

    # the same step when the caller hands over host buffers: H2D of the plan tensors, D2H of the results
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(3):
        eng.eval(batch)
    pcie_ms = (time.perf_counter() - t0) / 3 * 1e3

    eng.eval_device(db, out)
    torch.cuda.synchronize()
    res = {k: v.cpu().numpy() for k, v in out.items()}
    mask, score = res["mask"], res["score"]
    valid = (mask & abi.MASK_VALID) != 0
    alg_bytes = ALG_BYTES[c] * n
    # what the timed launch consists of: one plan per wavefront for a batch that would not fill the chip
    # otherwise; else the throughput kernel, for mid-size batches with the largest graphs on a second stream
    if stats["state_lanes"] == 1:
        kernel_name = "k_plan"
    elif stats["single_plan_tasks"] and stats.get("quad_tasks"):
        kernel_name = (f"k_eval<0> beside k_quad ({stats['quad_tasks']} wavefronts of 16 plans) and k_plan "
                       f"({stats['single_plan_tasks']} plans), one launch each, timed from fork to join")
    elif stats["single_plan_tasks"]:
        kernel_name = f"k_eval<0> beside k_plan ({stats['single_plan_tasks']} plans), one launch each, timed from fork to join"
    else:
        kernel_name = f"k_eval<{stats['state_lanes']}>"
    achieved_gbs = alg_bytes / (kernel_ms * 1e-3) / 1e9
    achieved_tflops = ALG_FLOPS[c] * n / (kernel_ms * 1e-3) / 1e12
    hbm = {"bound": "hbm", "achieved": achieved_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
           "frac": achieved_gbs / HBM_PEAK_GBS, "algorithmic_bytes_per_plan": ALG_BYTES[c]}
    fp64 = {"bound": "fp64_valu", "achieved": achieved_tflops, "peak": FP64_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": achieved_tflops / FP64_PEAK_TFLOPS, "algorithmic_flops_per_plan": ALG_FLOPS[c]}
    # the roofline of the line is the one with the larger fraction: achieved = max(bytes fraction, flops fraction)
    roofline = dict(fp64 if fp64["frac"] >= hbm["frac"] else hbm)
    layout = (stats["wave_tasks"], stats["lds_bytes"], stats["state_lanes"], stats["single_plan_tasks"], stats.get("quad_tasks", 0))
    measured = MEASURED.get(c)
    # (which classes run where is decided from times the kernels measure on themselves: the task counts of two runs
    # differ by up to a fifth, the number of k_quad's tasks by up to a third)
    same_layout = measured is not None and tuple(measured["layout"][1:3]) == layout[1:3] and all(
        abs(a - b) <= 0.05 * max(a, b) + 8 for a, b in zip((measured["layout"][0],) + tuple(measured["layout"][3:]),
                                                           (layout[0],) + layout[3:]))
    roofline.update(traffic=measured["traffic"] if same_layout else None, kernel=kernel_name, kernel_ms=kernel_ms,
                    layout=list(layout))
    ipp = measured["instructions_per_plan"] if same_layout else None
    issue = {"instructions_per_plan": ipp, "peak": ISSUE_PEAK, "unit": "wave-instructions/s",
             "achieved": None if ipp is None else ipp * n / (kernel_ms * 1e-3),
             "frac": None if ipp is None else ipp * n / (kernel_ms * 1e-3) / ISSUE_PEAK,
             "note": "instructions issued per plan from the rocprofv3 counter summary under profiles/; "
                     "null when the kernel layout of this run is not the profiled one"}
    line = {
        "metric": "cost-model plan evals/sec on 1 MI355X",
        "value": value, "unit": "plan evals/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "ms_per_step_spread": spread, "host_ms_in_calls_per_step": host_s / args.steps * 1e3,
        "host_us_of_a_call": host_us,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64", "data": "synthetic",
        "config": {"workload": cfg.name, "n_plans": n, "seed": 42, "K_eval": cfg.problem.K_eval,
                   "device_mesh": [cfg.problem.device_space.R, cfg.problem.device_space.N, cfg.problem.device_space.G],
                   "classes": stats["classes"], "inputs": "resident in HBM", "outputs": "left in HBM"},
        "roofline": roofline, "hbm": hbm, "fp64_valu": fp64, "issue": issue,
        "kernel_only_evals_per_s": n / (kernel_ms * 1e-3),
        "two_stream_evals_per_s": two_stream,
        "pcie_inclusive_ms_per_step": pcie_ms, "pcie_inclusive_evals_per_s": n / (pcie_ms * 1e-3),
        "first_call_ms": first_call_ms, "cold_ms_per_step": cold_ms, "cold_evals_per_s": n / (cold_ms * 1e-3),
        "feasible_fraction": float(((mask & abi.MASK_MEM_OK) != 0)[valid].mean()),
        "best_plan": int(score.argmax()), "best_score": float(score.max()),
    }
    if cpu is not None:
        line["cpu_baseline"] = cpu["one"]
        line["cpu_baseline_pool"] = cpu["pool"]
        line["cpu_port_cxx"] = cpu["cxx"]
        line["parity"] = parity_block(res, cpu["ref"])
        line["host_cores"] = os.cpu_count()
    else:
        line["cpu_baseline"] = None
        line["parity"] = None
    if not args.no_sa:
        # the second half of the metric: the annealing run of config 5, timed in the same process
        eng.close()
        sa = sa_measure(args, deadlines=False)
        line["sa"] = {k: sa[k] for k in ("metric", "value", "unit", "config", "time_to_best_s", "best_step", "best_score",
                                         "best_feasible", "best_plan_crc", "plans_evaluated", "launches", "evals_per_s",
                                         "eval_share_of_wall", "wall_s_of_runs", "directory_s", "cpu_baseline")}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
