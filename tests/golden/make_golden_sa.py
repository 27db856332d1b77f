"""Writes tests/golden/ref_sa.json: vectors of the simulated-annealing neighbourhood produced by
the REFERENCE implementation (RPEG/search/moves.py).

Run in the development container only (it needs the read-only reference tree):

    python tests/golden/make_golden_sa.py [--ref /root/reference]

`search/moves.py` imports `Configuration` from `search/evaluate.py`, which does not parse in the
snapshot.  `Configuration` is a plain record of five fields (evaluate.py:37-47); a record with the
same fields is registered under that module name so that moves.py imports.  No function of the
reference is replaced.

The reference draws from Python's global `random` module.  To obtain vectors that do not depend on
MT19937, the module attribute `random` of moves.py is pointed at a counter-based generator object
(oracle.sa_oracle.CounterRng) that offers the four methods moves.py calls.  The reference's own
code then decides which draws are made, in which order and how they are used; the restatement
must make the same decisions to reproduce the outputs.
"""

from __future__ import annotations

import argparse
import dataclasses
import json
import os
import sys
import types
import zlib

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

import make_golden as MG  # noqa: E402

CASES = {5: 40, 1: 24}          # configuration -> number of plans used


def load_moves(ref_root):
    mods = MG.load_reference(ref_root)
    ct = mods["core.types"]
    import search  # noqa: F401  (namespace package of the reference)

    @dataclasses.dataclass
    class Configuration:
        rpeg: object
        plan: object
        device_space: object
        intra_stage_fusion: bool = False
        transfer_resource_policy: object = None

    stub = types.ModuleType("search.evaluate")
    stub.Configuration = Configuration
    sys.modules["search.evaluate"] = stub
    import schedule.trace  # noqa: F401
    import search.moves as moves
    return mods, moves, Configuration, ct


def ref_world(mods, problem, tau_by_model):
    ct = mods["core.types"]
    suite = mods["model.models"].ModelSuite({
        ct.Model(m.value): mods["model.models"].ModelSpec(L=s.L, d=s.d, d_ff=s.d_ff, V=s.V,
                                                          dtype_bytes=s.dtype_bytes, d_head=s.d_head)
        for m, s in problem.suite.specs.items()})
    w = problem.workload
    wl = mods["model.workload"].Workload(B=w.B, K=w.K, S=w.S, T=w.T, gen_quantiles=w.gen_quantiles)
    hw = mods["model.hardware"].Hardware(**{k: getattr(problem.hw, k) for k in problem.hw.__dataclass_fields__})
    sp = problem.device_space
    space = ct.DeviceSpace(R=sp.R, N=sp.N, G=sp.G)
    name = problem.structures[0].name
    build = {"ppo": mods["ir.ppo"].build_PPO_RPEG, "grpo": mods["ir.grpo"].build_GRPO_RPEG,
             "dpo": mods["ir.dpo"].build_DPO_RPEG}[name]
    rpeg = build(suite, wl, tau={ct.Model(m): t for m, t in tau_by_model.items()})
    pol = problem.memory_policy
    cost = mods["model.cost"].NodeCostModel(hw, suite, wl, optimizer_stage=pol.optimizer_stage,
                                            activation_checkpointing=pol.activation_checkpointing)
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
    return rpeg, suite, wl, hw, space, cost, mm


def ref_plan(mods, rpeg, batch, problem, i):
    ct = mods["core.types"]
    _, plan_m, _ = batch.configuration(problem, i)
    by_id = {v.id: v for v in rpeg.vertices}
    sigma = {by_id[v.id]: ct.Allocation(origin=a.origin, extent=a.extent) for v, a in plan_m.sigma.items()}
    pi = {by_id[v.id]: p for v, p in plan_m.pi.items()}
    mb = {by_id[v.id]: m for v, m in plan_m.mb.items()}
    return mods["ir.plan"].ExecutionPlan(sigma=sigma, pi=pi, mb=mb)


def plan_rows(rpeg, plan):
    return [[*plan.pi[v], plan.mb[v], *plan.sigma[v].origin, *plan.sigma[v].extent] for v in rpeg.vertices]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    args = ap.parse_args()
    mods, moves, Configuration, ct = load_moves(args.ref)
    from oracle.sa_oracle import CounterRng
    from rpeg_amd import configs
    from rpeg_amd.search import candidates

    doc = {"seed": 42, "configs": {}}
    for c, n_plans in CASES.items():
        cfg = configs.config(c)
        problem = cfg.problem
        trainable = [m.value for m in problem.structures[0].tau_models]
        zero_tau = {m: 0 for m in trainable}
        rpeg0, suite, wl, hw, space, cost, mm = ref_world(mods, problem, zero_tau)
        table, index = moves.build_candidate_directory(rpeg0, suite, space, wl, cost, mm)
        dir_doc = {}
        for v in rpeg0.vertices:
            keys = ",".join(str(x) for e in table[v] for x in e[:6])
            times = ",".join(e[6].hex() for e in table[v])
            dir_doc[v.id] = dict(n=len(table[v]), n_enumerated=len(moves._enumerate_strategies(v, suite, space, wl)),
                                 key_crc=zlib.crc32(keys.encode()), time_crc=zlib.crc32(times.encode()),
                                 head=[list(e[:6]) + [e[6].hex()] for e in table[v][:6]])
        batch = candidates.generate(problem, n_plans, cfg.tau_choices, seed=42, tag=c)
        cases = []
        for i in range(n_plans):
            tau = dict(zero_tau)
            tau[trainable[0]] = i % 2
            rpeg, *_ = ref_world(mods, problem, tau)
            # the directory is keyed by the vertices of rpeg0; templates of equal structure share vertex ids
            tbl = {v: table[v0] for v, v0 in zip(rpeg.vertices, rpeg0.vertices)}
            idx = {v: index[v0] for v, v0 in zip(rpeg.vertices, rpeg0.vertices)}
            plan = ref_plan(mods, rpeg, batch, problem, i)
            config = Configuration(rpeg, plan, space)
            unrolled = mods["passes.unroll"].unroll(rpeg, problem.K_eval)
            lowered = mods["passes.lower"].lower(rpeg, unrolled, plan, suite, problem.K_eval, workload=wl)
            trace = mods["schedule.scheduler"].schedule(lowered, cost, space)
            chain = moves._critical_chain(lowered, trace)
            mass = moves._critical_mass(chain, rpeg, trace)
            rec = dict(i=i, tau=i % 2, n_chain=len(chain),
                       chain_crc=zlib.crc32(",".join(sorted(n.id for n in chain)).encode()),
                       mass=[mass[v].hex() for v in rpeg.vertices])
            T = (0.05, 0.02, 0.3, 0.004)[i % 4]
            T_init = (0.05, 0.05, 0.3, 0.3)[i % 4]
            moves.random = CounterRng(42, c, i, 1)
            stats = moves.MoveStats()
            out = moves.move_gen(config, lowered, trace, tbl, idx, 6, 50, T, T_init, stats)
            rec["move_gen"] = dict(T=T, T_init=T_init, n_draws=moves.random.k, fallback=stats.n_fallback,
                                   plans=[plan_rows(rpeg, x.plan) for x in out])
            moves.random = CounterRng(42, c, i, 2)
            nb = moves.multi_move_pair(config, suite, wl)
            rec["pair"] = dict(n_draws=moves.random.k, plan=None if nb is None else plan_rows(rpeg, nb.plan))
            moves.random = CounterRng(42, c, i, 3)
            samples = []
            for v in rpeg.vertices:
                lo = i % space.R
                hi = min(space.R, lo + 1 + (i // 3) % space.R)
                s = moves.sample_expl_in_region(v, suite, space, wl, r_lo=lo, r_hi=hi)
                samples.append(None if s is None else [*s[1], s[2], *s[0].origin, *s[0].extent])
            rec["sample"] = dict(n_draws=moves.random.k, rows=samples)
            cases.append(rec)
        doc["configs"][str(c)] = dict(directory=dir_doc, cases=cases)
        print(f"cfg{c}: directory sizes {[d['n'] for d in dir_doc.values()]}, {len(cases)} cases, "
              f"{sum(r['pair']['plan'] is not None for r in cases)} pair proposals")
    path = os.path.join(HERE, "ref_sa.json")
    with open(path, "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
