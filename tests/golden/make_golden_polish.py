"""Writes tests/golden/ref_polish.json: what the REFERENCE's polish() (RPEG/search/optimizer.py:949-1188)
returns for seeded start plans of config 1, and the derived fields of its OptimizerConfig.

Run in the development container only (it needs the read-only reference tree):

    python tests/golden/make_golden_polish.py [--ref /root/reference]

The snapshot's `search/optimizer.py` does not import as shipped: its polish() signature annotates with
`TemplateVertex`, `List` and `Trace`, which the module never imports, and it imports the unparsable
`search/evaluate.py`.  The three names are made visible as builtins (they occur in annotations only),
and `search.evaluate` is served by a module holding the `Configuration` record plus the four functions
optimizer.py imports, written here on the reference's own passes (unroll, lower, schedule, memory)
exactly as make_golden.py scores a plan: evaluate.py's score arithmetic (:288, 396-401), its stale-layout
rule (:115-140) and its cache key (:301-326).  polish() itself runs unmodified, with K_x = 1 so that it
evaluates in-process instead of through a worker pool.
"""

from __future__ import annotations

import argparse
import builtins
import json
import math
import os
import sys
import typing

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

import make_golden as MG      # noqa: E402
import make_golden_sa as SA   # noqa: E402


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    args = ap.parse_args()
    mods, moves, Configuration, ct = SA.load_moves(args.ref)
    import ir.rpeg
    import search.cache as rcache
    stub = sys.modules["search.evaluate"]
    state = {}

    def _eval(config, gate):
        p = state["problem"]
        rpeg, plan = config.rpeg, config.plan
        unrolled = mods["passes.unroll"].unroll(rpeg, p.K_eval)
        lowered = mods["passes.lower"].lower(rpeg, unrolled, plan, state["suite"], p.K_eval, workload=state["wl"])
        trace = mods["schedule.scheduler"].schedule(lowered, state["cost"], state["space"])
        wl = state["wl"]
        raw = trace.throughput(W_step=wl.B * wl.K * (wl.S + wl.T), K=p.K_eval)
        if gate:
            for e in rpeg.pub_edges:
                if int(rpeg.tau.get(e.src.kind.model, 0)) > 0:
                    a, b = plan.sigma[e.src], plan.sigma[e.dst]
                    if all(a.origin[i] < b.origin[i] + b.extent[i] and b.origin[i] < a.origin[i] + a.extent[i] for i in range(3)):
                        return 0.0, trace, False
        violation = mods["model.memory"].mem_worst_violation(lowered, state["mm"])
        if violation is None:
            return raw, trace, True
        _, req, cap = violation
        return raw * max(math.exp(-40.0 * max(0.0, req / cap - 1.0)), 1e-12), trace, False

    def evaluation_cache_key(config, memory_policy=None):
        return rcache.config_hash(config.rpeg, config.plan) + ":mem:fusion=0:transfer=destination_only,destination_only:2:1:0:0:activation_cache=0:groups=0"

    def evaluate_cached(config, cache, suite, workload, hw, K_eval, memory_policy=None):
        h = evaluation_cache_key(config)
        if h in cache:
            s, t, f = cache.get(h)
            return s, t, f, False
        s, t, f = _eval(config, gate=True)
        cache.put(h, s, t, f)
        return s, t, f, True

    def _eval_worker(args):
        state["n_worker"] += 1
        return _eval(args[0], gate=False)

    stub.evaluation_cache_key, stub.evaluate_cached, stub._eval_worker = evaluation_cache_key, evaluate_cached, _eval_worker
    stub.is_valid = lambda *a, **k: True
    import schedule.trace
    builtins.TemplateVertex, builtins.List, builtins.Trace = ir.rpeg.TemplateVertex, typing.List, schedule.trace.Trace
    import search.optimizer as ropt

    from rpeg_amd import configs
    from rpeg_amd.search import candidates
    cfg = configs.config(1)
    p = cfg.problem
    rpeg0, suite, wl, hw, space, cost, mm = SA.ref_world(mods, p, {"Pi": 0, "V": 0})
    state.update(problem=p, suite=suite, wl=wl, space=space, cost=cost, mm=mm, n_worker=0)
    table, index = moves.build_candidate_directory(rpeg0, suite, space, wl, cost, mm)
    batch = candidates.generate(p, 64, cfg.tau_choices, seed=42, tag=1)
    oc = ropt.OptimizerConfig(K_x=1, T_init=0.30, T_min=0.03)
    doc = {"optimizer_config": {"default": [ropt.OptimizerConfig().I_max, ropt.OptimizerConfig().T_cool.hex()],
                                "cfg5": [ropt.OptimizerConfig(K_x=6, T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=10).I_max,
                                         ropt.OptimizerConfig(K_x=6, T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=10).T_cool.hex()],
                                "e800": [ropt.OptimizerConfig(E_struct=800, K_x=4).I_max, ropt.OptimizerConfig(E_struct=800, K_x=4).T_cool.hex()]},
           "T_init": 0.30, "T_min": 0.03, "cases": [], "utilisation_cases": []}
    done = 0
    for i in range(64):
        if done >= 4:
            break
        plan = SA.ref_plan(mods, rpeg0, batch, p, i)
        start = Configuration(rpeg0, plan, space)
        s0, _, f0 = _eval(start, gate=True)
        if not f0:
            continue
        state["n_worker"] = 0
        out = ropt.polish(start, suite, wl, hw, p.K_eval, oc, rcache.EvalCache(), table, index)
        s1, _, f1 = _eval(out, gate=True)
        doc["cases"].append(dict(i=i, start_score=s0.hex(), final_score=s1.hex(), final_feasible=f1,
                                 evaluations=state["n_worker"], plan=SA.plan_rows(rpeg0, out.plan)))
        # the same start under the utilisation objective (optimizer.py:1021-1044)
        oc_u = ropt.OptimizerConfig(K_x=1, T_init=0.30, T_min=0.03, max_throughput_loss=0.10)
        state["n_worker"] = 0
        out = ropt.polish(start, suite, wl, hw, p.K_eval, oc_u, rcache.EvalCache(), table, index)
        s1, tr1, f1 = _eval(out, gate=True)
        doc["utilisation_cases"].append(dict(i=i, max_throughput_loss=0.10, final_score=s1.hex(), final_feasible=f1,
                                             final_utilization=float(tr1.utilization()).hex(),
                                             evaluations=state["n_worker"], plan=SA.plan_rows(rpeg0, out.plan)))
        done += 1
    path = os.path.join(HERE, "ref_polish.json")
    with open(path, "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    print(path, os.path.getsize(path), "bytes;", [(c["i"], float.fromhex(c["start_score"]), float.fromhex(c["final_score"]), c["evaluations"]) for c in doc["cases"]])


if __name__ == "__main__":
    main()
