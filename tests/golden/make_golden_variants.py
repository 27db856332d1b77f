"""Writes tests/golden/ref_variants.json: evaluations by the REFERENCE on problems away from the five shipped
configurations -- PPO and GRPO without generation quantiles, one and six quantiles, K > 1 for PPO, device
meshes with 2 and 8 devices per node, model records with 4-byte elements, another head size and a stated
parameter count.

Run in the development container only (it needs the read-only reference tree):

    python tests/golden/make_golden_variants.py [--ref /root/reference]

For the first plans of a seeded candidate set of every problem below the reference evaluates each plan;
stored per plan: makespan, worst device peak and penalised score as hex floats, feasibility, lowered graph
size and a checksum of the dispatch order.  Inputs are regenerated from the seed by the tests through
`variant_problems()` of this file, which needs no reference.
"""

from __future__ import annotations

import argparse
import dataclasses
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
N_PLANS = 64
SEED = 42


def variant_problems():
    """[(name, problem, tau_choices, tag)] -- built from this repository's own records only."""
    from rpeg_amd import configs
    from rpeg_amd.core.types import DeviceSpace, Model
    from rpeg_amd.model.models import ModelSpec, ModelSuite
    from rpeg_amd.model.workload import Workload
    c1, c2 = configs.config(1), configs.config(2)
    small = ModelSpec(L=24, d=2048, d_ff=5632, V=50304, dtype_bytes=4, d_head=64)
    counted = ModelSpec(L=32, d=4096, d_ff=11008, V=32000, parameter_count=6_738_415_616)
    out = []
    p = dataclasses.replace(
        c1.problem, workload=Workload(B=96, K=1, S=256, T=768, gen_quantiles=None), device_space=DeviceSpace(1, 4, 8),
        suite=ModelSuite({Model.ACTOR: counted, Model.REFERENCE: counted, Model.REWARD: small, Model.CRITIC: small,
                          Model.AC_SHARE: counted}))
    out.append(("ppo_unsplit_1x4x8", p, c1.tau_choices, 11))
    p = dataclasses.replace(
        c2.problem, device_space=DeviceSpace(2, 2, 8), K_eval=4,
        workload=Workload(B=64, K=4, S=256, T=2048, gen_quantiles=((0.2, 256), (0.4, 512), (0.6, 768), (0.8, 1024),
                                                                   (0.95, 1536), (1.0, 2048))))
    out.append(("grpo_six_quantiles_2x2x8", p, c2.tau_choices, 12))
    p = dataclasses.replace(
        c1.problem, device_space=DeviceSpace(2, 4, 2), K_eval=3,
        workload=Workload(B=32, K=2, S=128, T=1024, gen_quantiles=((1.0, 1024),)))
    out.append(("ppo_one_quantile_k2_2x4x2", p, c1.tau_choices, 13))
    p = dataclasses.replace(
        c2.problem, device_space=DeviceSpace(1, 8, 4), K_eval=6,
        workload=Workload(B=128, K=2, S=512, T=512, gen_quantiles=None),
        suite=ModelSuite({Model.ACTOR: small, Model.REFERENCE: small, Model.REWARD: counted}))
    out.append(("grpo_unsplit_small_1x8x4", p, c2.tau_choices, 14))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    args = ap.parse_args()
    sys.path.insert(0, HERE)
    import make_golden as mg
    mods = mg.load_reference(args.ref)
    from rpeg_amd.search import candidates
    real_to_reference = mg.to_reference

    def to_reference(mods_, problem, batch, i):   # make_golden's, with the stated parameter counts carried over
        rpeg, plan, wl, suite, hw, space = real_to_reference(mods_, problem, batch, i)
        ct = mods_["core.types"]
        specs = {ct.Model(m.value): dataclasses.replace(suite.specs[ct.Model(m.value)], parameter_count=s.parameter_count)
                 for m, s in problem.suite.specs.items()}
        suite = mods_["model.models"].ModelSuite(specs)
        name = problem.structures[int(batch.head[0, i])].name
        build = {"ppo": mods_["ir.ppo"].build_PPO_RPEG, "grpo": mods_["ir.grpo"].build_GRPO_RPEG}[name]
        rpeg2 = build(suite, wl, tau=dict(rpeg.tau))
        by_id = {v.id: v for v in rpeg2.vertices}
        plan2 = mods_["ir.plan"].ExecutionPlan(sigma={by_id[v.id]: a for v, a in plan.sigma.items()},
                                               pi={by_id[v.id]: x for v, x in plan.pi.items()},
                                               mb={by_id[v.id]: x for v, x in plan.mb.items()})
        return rpeg2, plan2, wl, suite, hw, space

    mg.to_reference = to_reference
    out = {"n_plans": N_PLANS, "seed": SEED, "problems": {}}
    for name, problem, tau_choices, tag in variant_problems():
        batch = candidates.generate(problem, N_PLANS, tau_choices, seed=SEED, tag=tag)
        rows, n_infeasible = [], 0
        for i in range(N_PLANS):
            rec, _, _, _ = mg.reference_eval(mods, problem, batch, i)
            rows.append({k: rec[k] for k in ("makespan", "peak", "score", "feasible", "n_nodes", "n_edges", "order_crc")})
            n_infeasible += not rec["feasible"]
        out["problems"][name] = rows
        print(f"{name}: {N_PLANS} plans, {n_infeasible} infeasible, nodes {min(r['n_nodes'] for r in rows)}-"
              f"{max(r['n_nodes'] for r in rows)}", flush=True)
    with open(os.path.join(HERE, "ref_variants.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))


if __name__ == "__main__":
    main()
