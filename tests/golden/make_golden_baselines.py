"""Writes tests/golden/ref_baselines.json: the start plans the REFERENCE's pipeline builds before it calls
optimize() (pipeline.py:389-435 greedy per-vertex plan, :437-1048 topology-aware concurrent plan, :1051-1108
fully colocated plan, :1111-1201 the hand-partitioned concurrent plan), for the templates of the benchmark configurations.

Run in the development container only (it needs the read-only reference tree):

    python tests/golden/make_golden_baselines.py [--ref /root/reference]

pipeline.py is imported unmodified.  Its import chain reaches `search/evaluate.py` (does not parse; served by
the record and function names make_golden_sa.py / make_golden_optimize.py register, none of which the three
constructors call), `search/optimizer.py` (three names it uses in annotations are made visible) and
`scripts/visualize.py` (plotting helpers, served by an empty module).  The constructors use the reference's
candidate directory, `packing_geometry`, the plan records and, for the concurrent plan, its lowering and
memory check.
"""

from __future__ import annotations

import argparse
import builtins
import contextlib
import importlib.util
import io
import json
import os
import sys
import types
import typing

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

import make_golden_sa as SA   # noqa: E402

CONFIGS = (1, 2, 3, 4, 5)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    args = ap.parse_args()
    mods, moves, Configuration, ct = SA.load_moves(args.ref)
    import ir.rpeg
    import schedule.trace
    stub = sys.modules["search.evaluate"]
    for name in ("evaluation_cache_key", "evaluate_cached", "_eval_worker", "is_valid"):
        setattr(stub, name, None)          # imported by name, never called by the constructors
    builtins.TemplateVertex, builtins.List, builtins.Trace = ir.rpeg.TemplateVertex, typing.List, schedule.trace.Trace
    vis = types.ModuleType("scripts.visualize")
    for name in ("dot_to_img", "exec_to_dot", "rpeg_to_dot", "unrolled_to_dot", "safe_unlink", "trace_to_gantt"):
        setattr(vis, name, None)
    pkg = types.ModuleType("scripts")
    pkg.__path__ = []
    sys.modules["scripts"], sys.modules["scripts.visualize"] = pkg, vis
    spec = importlib.util.spec_from_file_location("ref_pipeline", os.path.join(args.ref, "pipeline.py"))
    pipe = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(pipe)

    from rpeg_amd import configs
    doc = {"configs": {}}
    for c in CONFIGS:
        problem = configs.config(c).problem
        trainable = [m.value for m in problem.structures[0].tau_models]
        rpeg, suite, wl, hw, space, cost, mm = SA.ref_world(mods, problem, {m: 0 for m in trainable})
        rec = {}
        for name in ("build_valid_baseline_plan", "build_fullycolocated_baseline_plan", "build_naive_concurrent_plan"):
            try:
                plan = getattr(pipe, name)(rpeg, space, suite, wl, cost, mm)
                rec[name] = dict(rows=SA.plan_rows(rpeg, plan))
            except (RuntimeError, KeyError) as ex:
                rec[name] = dict(error=type(ex).__name__, message=str(ex))
        # the topology-aware plan (pipeline.py:908-1048): every plan it lowers for its memory check, with the
        # verdict of that check, and what it returns.  The two names it calls are wrapped to listen in.
        tried = []
        real_lower, real_check = pipe.lower, pipe.mem_worst_violation

        def lower(rpeg_, unrolled, plan, *a, **k):
            tried.append(dict(rows=SA.plan_rows(rpeg_, plan)))
            return real_lower(rpeg_, unrolled, plan, *a, **k)

        def check(executable, mem_model):
            v = real_check(executable, mem_model)
            tried[-1]["peak_over_cap"] = None if v is None else float(v[1]).hex()
            return v

        pipe.lower, pipe.mem_worst_violation = lower, check
        try:
            with contextlib.redirect_stdout(io.StringIO()):
                plan, found = pipe.build_concurrent_baseline_plan(rpeg, space, suite, wl, cost, mm)
        finally:
            pipe.lower, pipe.mem_worst_violation = real_lower, real_check
        rec["build_concurrent_baseline_plan"] = dict(rows=SA.plan_rows(rpeg, plan), found=bool(found), tried=tried)
        doc["configs"][str(c)] = rec
        print(c, {k: ("error " + v["error"]) if "error" in v else "ok" for k, v in rec.items()},
              "concurrent: found", found, "after", len(tried), "plans")
    path = os.path.join(HERE, "ref_baselines.json")
    with open(path, "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
