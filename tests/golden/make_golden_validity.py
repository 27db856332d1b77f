"""Writes tests/golden/ref_validity.json: verdicts of the REFERENCE's own gate functions.

Run in the development container only (it needs the read-only reference tree):

    python tests/golden/make_golden_validity.py [--ref /root/reference]

`search/evaluate.py` of the reference snapshot does not parse as a whole: the annotation of `_eval_worker`
(line 407) lacks a bracket.  Everything before that function does parse.  This script reads the file where it
lies, compiles the text up to the line `def _eval_worker(` as the module `search.evaluate` (nothing is copied
into this repository, nothing else is altered) and records what the reference's own

    is_compatible, allocations_overlap, stale_publication_layout_valid, is_valid,
    evaluation_cache_key, evaluate_cached (score, feasibility: the penalty arithmetic of :388-401, and the score
    under ABLATION_HARD_OOM for the plans that do not fit)

return for seeded plans of all five configurations (every template: PPO, GRPO, DPO and AC-share) and for the
same plans broken one rule at a time.  Inputs are regenerated from the seed by the tests through
`validity_cases()` of this file, which needs no reference; outputs are stored as booleans, hex floats and
CRCs of the key strings.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import types
import zlib

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

N_PLANS = 48
N_BROKEN_RULES = 9
SEED = 42


def broken(problem, rpeg, plan, v, rule):
    """`plan` with one rule of the gate broken at vertex v (this repository's records)."""
    from rpeg_amd.core.types import Allocation
    from rpeg_amd.ir.plan import ExecutionPlan
    sigma, pi, mb = dict(plan.sigma), dict(plan.pi), dict(plan.mb)
    dp, pp, tp = pi[v]
    a = sigma[v]
    sp = problem.device_space
    if rule == 0:
        mb[v] = mb[v] + 1                                          # micro-batch rule
    elif rule == 1:
        pi[v] = (dp, pp, 3)                                        # tp does not divide G
    elif rule == 2:
        sigma[v] = Allocation(origin=(a.origin[0], a.origin[1] + sp.N, a.origin[2]), extent=a.extent)   # out of bounds
    elif rule == 3:
        sigma[v] = Allocation(origin=a.origin, extent=(a.extent[0], a.extent[1], a.extent[2] + 1))      # g_ext mismatch
    elif rule == 4:
        pi[v] = (dp * 3 + 1, pp, tp)                               # dp does not divide B
    elif rule == 5:
        pi[v] = (dp, 7, tp)                                        # pp does not divide L
    elif rule == 6:
        sigma[v] = Allocation(origin=a.origin, extent=(a.extent[0] + 1, a.extent[1], a.extent[2]))      # not a layout of the node count
    elif rule == 7:
        pi[v] = (dp, pp, tp * 8)                                   # tp above G
    elif rule == 8:                                                # every vertex onto the allocation of v: publication
        for u in rpeg.vertices:                                    # endpoints intersect (matters with staleness > 0)
            if pi[u] == pi[v] and mb[u] == mb[v]:
                sigma[u] = a
    return ExecutionPlan(sigma, pi, mb)


def validity_cases(c):
    """[(plan index, rule or None, rpeg, plan, workload)] of configuration c, this repository's records."""
    from tests.helpers import seeded_batch
    cfg, batch = seeded_batch(c, N_PLANS)
    p = cfg.problem
    cases = []
    for i in range(batch.n):
        rpeg, plan, wl = batch.configuration(p, i)
        cases.append((i, None, rpeg, plan, wl))
        v = rpeg.vertices[i % len(rpeg.vertices)]
        cases.append((i, i % N_BROKEN_RULES, rpeg, broken(p, rpeg, plan, v, i % N_BROKEN_RULES), wl))
    return cfg, batch, cases


def load_reference_evaluate(ref_root, mods):
    """The part of RPEG/search/evaluate.py that parses, compiled in place as module `search.evaluate`."""
    import search.cache  # noqa: F401  (reference module; parses)
    import schedule.trace  # noqa: F401
    path = os.path.join(ref_root, "RPEG", "search", "evaluate.py")
    with open(path) as f:
        lines = f.readlines()
    end = next(k for k, ln in enumerate(lines) if ln.startswith("def _eval_worker("))
    mod = types.ModuleType("search.evaluate")
    mod.__file__ = path
    sys.modules["search.evaluate"] = mod
    exec(compile("".join(lines[:end]), path, "exec"), mod.__dict__)
    return mod


def reference_plan(mods, ref_rpeg, plan_m):
    ct = mods["core.types"]
    by_id = {v.id: v for v in ref_rpeg.vertices}
    return mods["ir.plan"].ExecutionPlan(
        sigma={by_id[v.id]: ct.Allocation(origin=a.origin, extent=a.extent) for v, a in plan_m.sigma.items()},
        pi={by_id[v.id]: x for v, x in plan_m.pi.items()},
        mb={by_id[v.id]: x for v, x in plan_m.mb.items()})


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    args = ap.parse_args()
    sys.path.insert(0, HERE)
    import make_golden as mg
    mods = mg.load_reference(args.ref)
    ev = load_reference_evaluate(args.ref, mods)
    MemoryPolicy = mods["model.memory"].MemoryPolicy
    NodeMemoryModel = mods["model.memory"].NodeMemoryModel
    EvalCache = sys.modules["search.cache"].EvalCache
    out = {"n_plans": N_PLANS, "seed": SEED, "configs": {}}
    for c in (1, 2, 3, 4, 5):
        cfg, batch, cases = validity_cases(c)
        p = cfg.problem
        pol_m = p.memory_policy
        pol = MemoryPolicy(**{k: getattr(pol_m, k) for k in pol_m.__dataclass_fields__})
        rows = []
        for i, rule, rpeg_m, plan_m, wl_m in cases:
            ref_rpeg, _, wl, suite, hw, space = mg.to_reference(mods, p, batch, i)
            plan = reference_plan(mods, ref_rpeg, plan_m)
            config = ev.Configuration(ref_rpeg, plan, space)
            verts = list(ref_rpeg.vertices)
            compat = [bool(ev.is_compatible(plan.sigma[v], plan.pi[v], space)) for v in verts]
            overlap = 0
            for x, u in enumerate(verts):
                for y, w in enumerate(verts):
                    if ev.allocations_overlap(plan.sigma[u], plan.sigma[w]):
                        overlap |= 1 << (8 * x + y)
            stale_ok = bool(ev.stale_publication_layout_valid(config))
            mem_model = NodeMemoryModel.from_policy(hw, suite, wl, pol, trainable=frozenset(ref_rpeg.trainable))
            try:
                valid = bool(ev.is_valid(config, suite, wl, mem_model))
            except ZeroDivisionError:
                valid = "ZeroDivisionError"
            row = {"plan": i, "rule": rule, "compatible": compat, "overlap": overlap, "stale_ok": stale_ok,
                   "is_valid": valid,
                   "key_crc": zlib.crc32(ev.evaluation_cache_key(config, pol).encode())}
            if rule is None or all(compat):   # evaluate_cached presumes a plan the gate's integer rules admit
                try:
                    score, _, feasible, miss = ev.evaluate_cached(config, EvalCache(), suite, wl, hw, p.K_eval, pol)
                    row.update(score=float(score).hex(), feasible=bool(feasible), miss=bool(miss))
                    if not feasible:   # the hard-OOM switch (evaluate.py:297-298, 392) on the reference's own function
                        ev.ABLATION_HARD_OOM = True
                        try:
                            hard = ev.evaluate_cached(config, EvalCache(), suite, wl, hw, p.K_eval, pol)
                        finally:
                            ev.ABLATION_HARD_OOM = False
                        row.update(score_hard_oom=float(hard[0]).hex(), feasible_hard_oom=bool(hard[2]))
                except (ZeroDivisionError, KeyError, ValueError) as e:
                    row.update(raises=type(e).__name__)
            rows.append(row)
        out["configs"][str(c)] = rows
        n_valid = sum(1 for r in rows if r["is_valid"] is True)
        print(f"config {c}: {len(rows)} cases, is_valid true on {n_valid}, stale rule false on "
              f"{sum(1 for r in rows if not r['stale_ok'])}, scored {sum(1 for r in rows if 'score' in r)}", flush=True)
    with open(os.path.join(HERE, "ref_validity.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))


if __name__ == "__main__":
    main()
