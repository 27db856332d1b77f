#!/usr/bin/env python3
"""Benchmark of the batched plan evaluator on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2] [--no-cpu]
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
# algorithmic bytes per plan: int16 plan fields (10 per vertex) + 4 header bytes in, 3 doubles + 1 mask byte out
ALG_BYTES = {1: 149, 2: 109, 3: 149, 4: 89, 5: 149}
# HBM bytes per step of the evaluation kernels measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by
# a 256 MiB copy (the counter summary of this workload is committed under profiles/); None where no counter
# run exists
MEASURED_TRAFFIC = {2: 243.5e6}
# algorithmic fp64 operations per plan (cost model + scheduler + memory model of the fully split DAG)
ALG_FLOPS = {1: 3.7e3, 2: 2.5e3, 3: 6.0e3, 4: 0.83e3, 5: 3.7e3}


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


def cxx_port(cfg, batch, threads):
    from oracle.cpu_port import CpuPort
    port = CpuPort(cfg.problem)
    n = min(batch.n, 65536)
    sub = batch.slice(0, n)
    port.eval(sub.slice(0, 256), threads=threads)
    t0 = time.perf_counter()
    port.eval(sub, threads=threads)
    dt = time.perf_counter() - t0
    return dict(value=n / dt, unit="plan evals/s", cores=threads,
                sample=f"first {n} plans, host build of the kernels' arithmetic (OpenMP), lowering included")


def bench_sa(args):
    """Config 5: 64 chains x 2000 steps of batched simulated annealing.  Prints one JSON line whose value
    is the wall-clock of the whole run (directory build excluded and reported beside it)."""
    import zlib
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
    for rep in range(max(1, args.steps if args.steps < 20 else 2)):   # first run lowers every class it meets
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
        "warm_wall_s": warm.wall_s, "warm_time_to_best_s": float(warm.best_time[c]),
        "directory_s": dir_s, "directory_sizes": [int(a.shape[0]) for a in arrays],
        "accept_rate": float((((cold.log >> 4) & 3) == 2).sum() / max(1, (((cold.log >> 4) & 3) != 0).sum())),
        "restarts": int(cold.restarts.sum()), "dead_chains": int(cold.dead.sum()),
        "feasible_chains": int(cold.best_feasible.sum()),
    }
    if not args.no_cpu:
        # the same host logic over the CPU build of the evaluator, all host cores, on a bounded number of steps
        from oracle.cpu_port import CpuPort
        threads = min(16, os.cpu_count() or 1)
        steps = max(1, min(args.sa_steps, 40))
        split = 1 if p.workload.gen_quantiles else 0
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
    print(json.dumps(line))


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
    ap.add_argument("--chains", type=int, default=64)
    ap.add_argument("--sa-steps", type=int, default=2000)
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the path needs no second one (plans are independent: with more GPUs the "
                 "candidate tensor or the annealing chains would be split evenly across them). Use --gpus 1.")

    if args.config == 5:
        return bench_sa(args)

    import torch
    from rpeg_amd import configs
    from rpeg_amd.engine import abi
    from rpeg_amd.engine.runtime import DeviceBatch, Engine
    from rpeg_amd.search import candidates

    c = args.config
    cfg = configs.config(c)
    n = cfg.n_plans
    batch = candidates.generate(cfg.problem, n, cfg.tau_choices, seed=42, tag=c)
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
    for _ in range(args.steps):
        eng.eval_device(db, out)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    ms_per_step = dt / args.steps * 1e3
    value = n * args.steps / dt

    # cold steps: every class of the batch is lowered again inside the step
    cold_steps = max(1, min(args.steps, 5))
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(cold_steps):
        eng.reset_classes()
        eng.eval_device(db, out)
    torch.cuda.synchronize()
    cold_ms = (time.perf_counter() - t0) / cold_steps * 1e3

    # duration of the evaluation launch (k_eval, k_plan, or both side by side from fork to join): HIP events on
    # the launch stream, recorded by the library
    eng.set_timing(True)
    k_ms = []
    for _ in range(args.steps):
        eng.eval_device(db, out)
        k_ms.append(eng.last_kernel_ms())
    eng.set_timing(False)
    kernel_ms = sum(k_ms) / len(k_ms)
    stats = eng.stats()

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

    mask = out["mask"].cpu().numpy()
    score = out["score"].cpu().numpy()
    valid = (mask & abi.MASK_VALID) != 0
    alg_bytes = ALG_BYTES[c] * n
    # what the timed launch consists of: one plan per wavefront for a batch that would not fill the chip
    # otherwise; else the throughput kernel, for mid-size batches with the largest graphs on a second stream
    if stats["state_lanes"] == 1:
        kernel_name = "k_plan"
    elif stats["single_plan_tasks"]:
        kernel_name = f"k_eval<0> beside k_plan ({stats['single_plan_tasks']} plans), one launch each, timed from fork to join"
    else:
        kernel_name = f"k_eval<{stats['state_lanes']}>"
    achieved_gbs = alg_bytes / (kernel_ms * 1e-3) / 1e9
    achieved_tflops = ALG_FLOPS[c] * n / (kernel_ms * 1e-3) / 1e12
    line = {
        "metric": "cost-model plan evals/sec on 1 MI355X",
        "value": value, "unit": "plan evals/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f64", "data": "synthetic",
        "config": {"workload": cfg.name, "n_plans": n, "seed": 42, "K_eval": cfg.problem.K_eval,
                   "device_mesh": [cfg.problem.device_space.R, cfg.problem.device_space.N, cfg.problem.device_space.G],
                   "classes": stats["classes"], "inputs": "resident in HBM", "outputs": "left in HBM"},
        "roofline": {"bound": "hbm", "achieved": achieved_gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved_gbs / HBM_PEAK_GBS, "traffic": MEASURED_TRAFFIC.get(c),
                     "kernel": kernel_name, "kernel_ms": kernel_ms, "algorithmic_bytes_per_plan": ALG_BYTES[c]},
        "fp64_valu": {"achieved": achieved_tflops, "peak": FP64_PEAK_TFLOPS, "unit": "TFLOP/s",
                      "frac": achieved_tflops / FP64_PEAK_TFLOPS, "algorithmic_flops_per_plan": ALG_FLOPS[c]},
        "kernel_only_evals_per_s": n / (kernel_ms * 1e-3),
        "two_stream_evals_per_s": two_stream,
        "pcie_inclusive_ms_per_step": pcie_ms, "pcie_inclusive_evals_per_s": n / (pcie_ms * 1e-3),
        "first_call_ms": first_call_ms, "cold_ms_per_step": cold_ms, "cold_evals_per_s": n / (cold_ms * 1e-3),
        "feasible_fraction": float(((mask & abi.MASK_MEM_OK) != 0)[valid].mean()),
        "best_plan": int(score.argmax()), "best_score": float(score.max()),
    }
    if not args.no_cpu:
        line["cpu_baseline"] = cpu_baseline(cfg, batch)
        line["cpu_port_cxx"] = cxx_port(cfg, batch, threads=min(16, os.cpu_count() or 1))
        line["host_cores"] = os.cpu_count()
    else:
        line["cpu_baseline"] = None
    print(json.dumps(line))


if __name__ == "__main__":
    main()
