"""Writes tests/golden/ref_*.json: input/output vectors produced by the REFERENCE implementation.

Run in the development container only (it needs the read-only reference tree):

    python tests/golden/make_golden.py [--ref /root/reference]

It imports the reference's own hot-path modules (passes.unroll, passes.lower, model.cost,
model.memory, schedule.scheduler) and evaluates the first plans of this repository's seeded
candidate sets with them.  These vectors pin the parts of the path that no closed form pins:
the generation roofline, scheduler dispatch order under key ties and the insertion-ordered
float sums of the per-device memory peaks.  Only data is written: inputs are regenerated from
the seed by tests, outputs are stored as hex floats.

The reference snapshot misspells one imported name in ir/rpeg.py (`Edgekind`, while the module
body uses `EdgeKind`); the two aliases below let the module import and run, nothing else is
altered.  `search/evaluate.py` does not parse
in the snapshot, so its few lines of score/penalty arithmetic (evaluate.py:288, 396-401) are
applied here to the reference's makespan and peak.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import zlib

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

N_PLANS = {1: 384, 2: 384, 3: 512, 4: 256, 5: 256}
N_NODE_VECTORS = 48


def load_reference(ref_root):
    sys.dont_write_bytecode = True
    sys.path.insert(0, os.path.join(ref_root, "RPEG"))
    import core.types as ct
    ct.Edgekind = ct.EdgeKind
    import ir.rpeg
    ir.rpeg.EdgeKind = ct.EdgeKind
    import ir.ppo, ir.grpo, ir.dpo, ir.ac_share, ir.plan  # noqa: E401
    import model.cost, model.memory, model.hardware, model.models, model.workload  # noqa: E401
    import passes.unroll, passes.lower  # noqa: E401
    import schedule.scheduler  # noqa: E401
    return sys.modules


def to_reference(mods, problem, batch, i):
    """Reference-side (rpeg, plan, workload, suite, hw, space) of candidate i."""
    ct = mods["core.types"]
    rpeg_m, plan_m, wl_m = batch.configuration(problem, i)
    suite = mods["model.models"].ModelSuite({
        ct.Model(m.value): mods["model.models"].ModelSpec(L=s.L, d=s.d, d_ff=s.d_ff, V=s.V,
                                                          dtype_bytes=s.dtype_bytes, d_head=s.d_head)
        for m, s in problem.suite.specs.items()})
    wl = mods["model.workload"].Workload(B=wl_m.B, K=wl_m.K, S=wl_m.S, T=wl_m.T,
                                         gen_quantiles=wl_m.gen_quantiles)
    hw = mods["model.hardware"].Hardware(**{k: getattr(problem.hw, k)
                                            for k in problem.hw.__dataclass_fields__})
    sp = problem.device_space
    space = ct.DeviceSpace(R=sp.R, N=sp.N, G=sp.G)
    name = problem.structures[int(batch.head[0, i])].name
    build = {"ppo": mods["ir.ppo"].build_PPO_RPEG, "grpo": mods["ir.grpo"].build_GRPO_RPEG,
             "dpo": mods["ir.dpo"].build_DPO_RPEG, "ac_share": mods["ir.ac_share"].build_AC_share_RPEG}[name]
    tau = {ct.Model(m.value): t for m, t in rpeg_m.tau.items()}
    rpeg = build(suite, wl, tau=tau)
    by_id = {v.id: v for v in rpeg.vertices}
    sigma = {by_id[v.id]: ct.Allocation(origin=a.origin, extent=a.extent) for v, a in plan_m.sigma.items()}
    pi = {by_id[v.id]: p for v, p in plan_m.pi.items()}
    mb = {by_id[v.id]: m for v, m in plan_m.mb.items()}
    plan = mods["ir.plan"].ExecutionPlan(sigma=sigma, pi=pi, mb=mb)
    return rpeg, plan, wl, suite, hw, space


def reference_eval(mods, problem, batch, i):
    rpeg, plan, wl, suite, hw, space = to_reference(mods, problem, batch, i)
    pol = problem.memory_policy
    unrolled = mods["passes.unroll"].unroll(rpeg, problem.K_eval)
    lowered = mods["passes.lower"].lower(rpeg, unrolled, plan, suite, problem.K_eval, workload=wl)
    cost = mods["model.cost"].NodeCostModel(hw, suite, wl, optimizer_stage=pol.optimizer_stage,
                                            activation_checkpointing=pol.activation_checkpointing)
    trace = mods["schedule.scheduler"].schedule(lowered, cost, space)
    makespan = trace.makespan()
    raw = trace.throughput(W_step=wl.B * wl.K * (wl.S + wl.T), K=problem.K_eval)
    mem_mod = mods["model.memory"]
    mm = mem_mod.NodeMemoryModel.from_policy(
        hw, suite, wl, mem_mod.MemoryPolicy(
            optimizer_stage=pol.optimizer_stage, activation_checkpointing=pol.activation_checkpointing,
            runtime_overhead_fraction=pol.runtime_overhead_fraction,
            worker_overhead_bytes=pol.worker_overhead_bytes,
            semantic_activation_cache_bytes=pol.semantic_activation_cache_bytes,
            max_worker_groups_per_gpu=pol.max_worker_groups_per_gpu),
        trainable=frozenset(rpeg.trainable),
        shadow_models=frozenset(m for m in rpeg.trainable if rpeg.tau.get(m, 0) > 0))
    peaks = mem_mod._device_peaks(lowered, mm)
    violation = mem_mod.mem_worst_violation(lowered, mm)
    max_peak = max(peaks.values())
    if violation is None:
        score, feasible = raw, True
    else:
        _, req, cap = violation
        assert req == max_peak
        score = raw * max(math.exp(-40.0 * max(0.0, req / cap - 1.0)), 1e-12)
        feasible = False
    order = ",".join(n.id for n in trace.start)
    return dict(makespan=makespan.hex(), raw=raw.hex(), peak=float(max_peak).hex(), score=score.hex(),
                feasible=feasible, n_nodes=len(lowered.nodes), n_edges=len(lowered.edges),
                order_crc=zlib.crc32(order.encode()),
                finish_sum=math.fsum(trace.finish.values()).hex(),
                utilization=float(trace.utilization()).hex(), n_active=trace.n_active()), lowered, cost, mm


def node_vectors(lowered, cost, mm, limit):
    """time() of every distinct node of step 0 and peak_bytes() of its operator nodes."""
    out = []
    for n in lowered.nodes:
        if len(out) >= limit:
            break
        if n.kind.value == "op" and n.op.k != 0:
            continue
        rec = {"id": n.id, "time": cost.time(n).hex()}
        if n.kind.value == "op":
            rec["peak_bytes"] = float(mm.peak_bytes(n)).hex()
            rec["breakdown"] = [x.hex() for x in cost.time_breakdown(n)]
        out.append(rec)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    ap.add_argument("--configs", default="1,2,3,4,5")
    args = ap.parse_args()
    mods = load_reference(args.ref)
    from rpeg_amd import configs
    from rpeg_amd.search import candidates
    for c in (int(x) for x in args.configs.split(",")):
        cfg = configs.config(c)
        n = N_PLANS[c]
        batch = candidates.generate(cfg.problem, n, cfg.tau_choices, seed=42, tag=c)
        plans, nodes = [], []
        for i in range(n):
            rec, lowered, cost, mm = reference_eval(mods, cfg.problem, batch, i)
            plans.append(rec)
            if i < N_NODE_VECTORS:
                nodes.append(node_vectors(lowered, cost, mm, 40))
        doc = dict(config=c, name=cfg.name, seed=42, tag=c, n=n,
                   memory_per_gpu=cfg.problem.hw.memory_per_gpu.hex(),
                   vert_crc=zlib.crc32(batch.vert.tobytes()), head_crc=zlib.crc32(batch.head.tobytes()),
                   plans=plans, nodes=nodes)
        path = os.path.join(HERE, f"ref_cfg{c}.json")
        with open(path, "w") as f:
            json.dump(doc, f, separators=(",", ":"))
        feas = sum(p["feasible"] for p in plans)
        print(f"cfg{c}: {n} plans, {feas} feasible -> {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
