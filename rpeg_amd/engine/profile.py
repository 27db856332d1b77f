"""Per-wavefront clocks of the evaluation kernels on one of the benchmark configurations.

    python -m rpeg_amd.engine.profile --config 3 [--plans N] [--sections]

Runs the seeded candidate set of the configuration through rpeg_eval_batch with the per-wavefront stamps switched
on (rpeg_engine_profile) and prints, for the main kernel (k_eval) and for the one-plan-per-wavefront kernel
(k_plan) and the four-lanes-per-plan kernel (k_quad) beside it: when their tasks start and end, how many run at a time, the longest tasks, and the durations
by node count.  A kernel ends with its slowest wavefront, so the table of the longest tasks is the critical
path of the step.

--sections loads the measurement build (python -m rpeg_amd.build --profile), in which k_eval sums the shader
clocks of the four sections of its scheduling loop -- the heap's pops up to the next dispatch, the removal of
the dispatched entry, the successors (their state comes from the HBM workspace), the ordered insertion of the
entries that became ready -- and prints them per dispatch, for all tasks and for the forty slowest.
"""

from __future__ import annotations

import argparse
import ctypes as C

import numpy as np


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--config", type=int, default=2)
    ap.add_argument("--plans", type=int, default=0, help="plans of the seeded set (default: the configuration's own size)")
    ap.add_argument("--sections", action="store_true", help="section clocks of the scheduling loop (measurement build)")
    ap.add_argument("--quad-share", type=int, default=-1, help="percent of the batch for the four-lanes-per-plan kernel (default: the engine's)")
    args = ap.parse_args()
    import torch
    from .. import build as B, configs
    from ..search import candidates
    from . import runtime as R
    if args.sections:
        import os
        if not os.path.exists(B.PROFILE_LIB):
            raise SystemExit("build the measurement library first: python -m rpeg_amd.build --profile")
        R._lib = R.load_library(B.PROFILE_LIB)
    cfg = configs.config(args.config)
    n = args.plans or cfg.n_plans
    batch = candidates.generate(cfg.problem, n, cfg.tau_choices, seed=42, tag=args.config)
    eng = R.Engine(cfg.problem)
    if args.quad_share >= 0:
        eng.set_quad_share(args.quad_share)
    lib = eng.lib
    lib.rpeg_engine_profile.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_uint64]
    db = R.DeviceBatch(batch)
    out = eng.alloc_outputs(batch.n)
    for _ in range(2):            # classes lowered, ready-list capacity learned
        eng.eval_device(db, out)
        torch.cuda.synchronize()
    lib.rpeg_engine_profile(eng._h, 1, None, 0)
    eng.set_timing(True)
    eng.eval_device(db, out)
    torch.cuda.synchronize()
    s = eng.stats()
    print(f"config {args.config}: {n} plans, kernels {eng.last_kernel_ms():.3f} ms (fork to join), layout {s}")
    rows = s["wave_tasks"]
    buf = np.zeros((rows, 8), np.uint64)
    got = lib.rpeg_engine_profile(eng._h, 1, buf.ctypes.data, rows)
    buf = buf[:got]
    n_eval = s["wave_tasks"] - s["single_plan_tasks"] - s["quad_tasks"]
    n_lane = n_eval + s["quad_tasks"]
    b = buf.astype(np.float64)
    nodes = (buf[:, 7] >> np.uint64(32)).astype(np.int64)
    t0 = b[:, 0][b[:, 0] > 0].min()
    start, end = (b[:, 0] - t0) / 100.0, (b[:, 6] - t0) / 100.0          # the stamps tick at 100 MHz: microseconds
    for name, sl in (("k_eval", slice(0, n_eval)), ("k_quad", slice(n_eval, n_lane)), ("k_plan", slice(n_lane, got))):
        S, E, N = start[sl], end[sl], nodes[sl]
        ok = E > 0
        S, E, N = S[ok], E[ok], N[ok]
        if len(S) == 0:
            continue
        d = E - S
        print(f"{name}: {len(S)} tasks, first start {S.min():.1f} us, last end {E.max():.1f} us, sum of durations "
              f"{d.sum() / 1000:.1f} ms, mean {d.mean():.1f} us, longest {d.max():.1f} us")
        T = E.max()
        print("   tasks running at t =", ", ".join(f"{q:.0f} us: {int(((S <= q) & (E > q)).sum())}" for q in np.linspace(T / 20, T * 19 / 20, 10)))
        o = np.argsort(-d)[:6]
        print("   longest tasks (nodes, start us, duration us):", [(int(N[k]), round(float(S[k]), 1), round(float(d[k]), 1)) for k in o])
        o = np.argsort(-E)[:6]
        print("   last to end   (nodes, start us, duration us):", [(int(N[k]), round(float(S[k]), 1), round(float(d[k]), 1)) for k in o])
        if not args.sections:   # (the measurement build keeps the section clocks where the phase stamps are, in every kernel)
            ph = np.diff(b[sl][ok][:, :7], axis=1) / 100.0
            names = ("plan fields", "durations", "memory model", "ranks", "scheduling", "outputs") if name == "k_eval" else \
                    ("plan fields", "durations", "memory model", "ranks and positions", "scheduling", "outputs") if name == "k_quad" else \
                    ("plan fields", "durations", "memory model and ranks", "positions in the order", "scheduling", "outputs")
            print("   phases, mean us per task: " + ", ".join(f"{nm} {x:.1f}" for nm, x in zip(names, ph.mean(0))))
            slow = np.argsort(-d)[:40]
            print("   phases of the 40 longest: " + ", ".join(f"{nm} {x:.1f}" for nm, x in zip(names, ph[slow].mean(0))))
        for lo, hi in ((0, 50), (50, 100), (100, 150), (150, 200), (200, 300), (300, 4096)):
            m = (N >= lo) & (N < hi)
            if m.sum():
                print(f"   nodes [{lo},{hi}): {int(m.sum()):6d} tasks, mean {d[m].mean():8.1f} us, longest {d[m].max():8.1f} us, "
                      f"sum {d[m].sum() / 1000:8.1f} ms")
    if args.sections and n_eval:
        pops = (buf[:n_eval, 7] & np.uint64(0xFFFFFFFF)).astype(np.float64)
        nn = nodes[:n_eval].astype(np.float64)
        clk = b[:n_eval, 1:5]
        dur = end[:n_eval] - start[:n_eval]
        ok = (nn > 0) & (dur > 0)
        slow = np.argsort(-np.where(ok, dur, 0))[:40]

        def line(sel, what):
            per = clk[sel] / nn[sel, None]
            print(f"   {what}: clocks per dispatch: pops {per[:, 0].mean():.0f}, removal {per[:, 1].mean():.0f}, successors "
                  f"{per[:, 2].mean():.0f}, insertion {per[:, 3].mean():.0f}, total {per.sum(1).mean():.0f}; pops per dispatch "
                  f"{(pops[sel] / nn[sel]).mean():.2f}; clocks per pop {(clk[sel, 0] / pops[sel]).mean():.0f}")
        print("k_eval scheduling loop (shader clocks):")
        line(np.flatnonzero(ok), "all tasks")
        line(slow, f"the 40 slowest tasks ({int(nn[slow].min())}-{int(nn[slow].max())} nodes, {dur[slow].mean():.0f} us)")


if __name__ == "__main__":
    main()
