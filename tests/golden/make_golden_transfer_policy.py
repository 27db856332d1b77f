"""Writes tests/golden/ref_transfer_policy.json: schedules of the REFERENCE scheduler under the three
non-default transfer resource policies (core/types.py:128-200, passes/transfer_resources.py:73-148).

Run in the development container only (it needs the read-only reference tree):

    python tests/golden/make_golden_transfer_policy.py [--ref /root/reference]

For the first plans of this repository's seeded candidate sets of all five configurations the
reference lowers each plan and schedules it with `transfer_resource_policy` set to both endpoints
for weights, for activations, and for both.  Stored per plan: makespan, sum of finish times and
utilisation as hex floats, and a checksum of the dispatch order.  Only data is written; the inputs
are regenerated from the seed by the tests.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import zlib

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import make_golden as mg  # noqa: E402

N_PLANS = {1: 96, 2: 96, 3: 64, 4: 96, 5: 64}
POLICIES = (("both_endpoints", "destination_only"), ("destination_only", "both_endpoints"),
            ("both_endpoints", "both_endpoints"))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    args = ap.parse_args()
    mods = mg.load_reference(args.ref)
    ct = mods["core.types"]
    from rpeg_amd import configs
    from rpeg_amd.search import candidates
    out = {"policies": [list(p) for p in POLICIES], "configs": {}}
    for c in (1, 2, 3, 4, 5):
        cfg = configs.config(c)
        problem, n = cfg.problem, N_PLANS[c]
        batch = candidates.generate(problem, n, cfg.tau_choices, seed=42, tag=c)
        pol = problem.memory_policy
        rows = []
        n_differ = 0
        for i in range(n):
            rpeg, plan, wl, suite, hw, space = mg.to_reference(mods, problem, batch, i)
            unrolled = mods["passes.unroll"].unroll(rpeg, problem.K_eval)
            lowered = mods["passes.lower"].lower(rpeg, unrolled, plan, suite, problem.K_eval, workload=wl)
            cost = mods["model.cost"].NodeCostModel(hw, suite, wl, optimizer_stage=pol.optimizer_stage,
                                                    activation_checkpointing=pol.activation_checkpointing)
            base = mods["schedule.scheduler"].schedule(lowered, cost, space).makespan()
            per = []
            for w, a in POLICIES:
                trace = mods["schedule.scheduler"].schedule(
                    lowered, cost, space,
                    transfer_resource_policy=ct.TransferResourcePolicy(weight=w, activation=a))
                order = ",".join(nd.id for nd in trace.start)
                per.append(dict(makespan=trace.makespan().hex(), order_crc=zlib.crc32(order.encode()),
                                finish_sum=math.fsum(trace.finish.values()).hex(),
                                utilization=float(trace.utilization()).hex()))
                n_differ += trace.makespan() != base
            rows.append(per)
        out["configs"][str(c)] = dict(n_plans=n, seed=42, rows=rows, n_differ_from_default=n_differ)
        print(f"config {c}: {n} plans, {n_differ} of {3 * n} schedules differ from the default policy's", flush=True)
    with open(os.path.join(HERE, "ref_transfer_policy.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))


if __name__ == "__main__":
    main()
