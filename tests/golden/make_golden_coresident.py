"""Writes tests/golden/ref_coresident.json: the REFERENCE's co-resident memory model.

Run in the development container only (it needs the read-only reference tree):

    python tests/golden/make_golden_coresident.py [--ref /root/reference]

A NodeMemoryModel built without a set of trainable models (`NodeMemoryModel.from_policy(hw, suite, workload, policy)`,
the default of its `trainable` argument) makes `_device_peaks` take its fallback branch (model/memory.py:706-742): per
device the static footprint of every model present -- weights, and for a model with a training vertex there also
optimizer state and gradients at that vertex's dp -- summed over the models, plus the largest transient of the nodes
on the device, plus the per-worker-group overhead.  None of the shipped call sites builds such a model; `is_valid`
takes whatever model its caller hands it.

For the first plans of the seeded candidate sets of all five configurations, under the default policy and under two
others (optimizer stages 0 and 1, overhead bytes, a worker-group limit), the reference computes: the largest device
peak of the K_eval = 1 lowering and of the K_eval lowering (`_device_peaks`), `mem_feasible` of both, and `is_valid`
(the reference's own function, from the part of search/evaluate.py that parses: make_golden_validity.py) with that
memory model.  Inputs are regenerated from the seed by the tests.
"""

from __future__ import annotations

import argparse
import dataclasses
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
import make_golden as mg  # noqa: E402
import make_golden_validity as mv  # noqa: E402

N_PLANS = {1: 48, 2: 48, 3: 48, 4: 48, 5: 32}
POLICIES = [
    dict(),
    dict(optimizer_stage=0, activation_checkpointing=False, worker_overhead_bytes=1.5e9, semantic_activation_cache_bytes=0.5e9),
    dict(optimizer_stage=1, runtime_overhead_fraction=0.05, max_worker_groups_per_gpu=2),
]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    args = ap.parse_args()
    mods = mg.load_reference(args.ref)
    ev = mv.load_reference_evaluate(args.ref, mods)
    mem_mod = mods["model.memory"]
    from rpeg_amd import configs
    from rpeg_amd.search import candidates
    out = {"policies": POLICIES, "configs": {}}
    for c in sorted(N_PLANS):
        cfg = configs.config(c)
        p = cfg.problem
        n = N_PLANS[c]
        batch = candidates.generate(p, n, cfg.tau_choices, seed=42, tag=c)
        rows, n_fit, n_valid = [], 0, 0
        for i in range(n):
            rpeg, plan, wl, suite, hw, space = mg.to_reference(mods, p, batch, i)
            per = []
            for pol in POLICIES:
                mm = mem_mod.NodeMemoryModel.from_policy(hw, suite, wl, mem_mod.MemoryPolicy(**pol))
                assert len(mm.trainable) == 0
                rec = {}
                for name, K in (("k1", 1), ("k", p.K_eval)):
                    lowered = mods["passes.lower"].lower(rpeg, mods["passes.unroll"].unroll(rpeg, K), plan, suite, K, workload=wl)
                    peaks = mem_mod._device_peaks(lowered, mm)
                    rec[name] = dict(peak=float(max(peaks.values())).hex() if max(peaks.values()) != float("inf") else "inf",
                                     feasible=bool(mem_mod.mem_feasible(lowered, mm)))
                rec["is_valid"] = bool(ev.is_valid(ev.Configuration(rpeg, plan, space), suite, wl, mm))
                n_fit += rec["k1"]["feasible"]
                n_valid += rec["is_valid"]
                per.append(rec)
            rows.append(per)
        out["configs"][str(c)] = dict(n_plans=n, seed=42, rows=rows)
        print(f"config {c}: {n} plans x {len(POLICIES)} policies, {n_fit} fit at K_eval = 1, is_valid true on {n_valid}", flush=True)
    with open(os.path.join(HERE, "ref_coresident.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))


if __name__ == "__main__":
    main()
