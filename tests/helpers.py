"""Shared helpers for the test-suite: golden fixtures, oracle evaluation of seeded candidates."""

import json
import os
import zlib

from oracle import rpeg_oracle as oracle
from rpeg_amd import configs
from rpeg_amd.search import candidates

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_golden(c):
    with open(os.path.join(GOLDEN, f"ref_cfg{c}.json")) as f:
        return json.load(f)


def seeded_batch(c, n=None, start=0):
    cfg = configs.config(c)
    return cfg, candidates.generate(cfg.problem, n or cfg.n_plans, cfg.tau_choices, seed=42, tag=c, start=start)


def oracle_eval(problem, batch, i, **kw):
    rpeg, plan, wl = batch.configuration(problem, i)
    return oracle.evaluate_plan(rpeg, plan, problem.device_space, problem.suite, wl, problem.hw,
                                problem.K_eval, problem.memory_policy, check_stale=False, **kw)


def order_crc(order):
    return zlib.crc32(",".join(order).encode())


def rows6(rows, nv):
    return [[int(x) for x in rows[v * 10:(v + 1) * 10]] for v in range(nv)]


# ---- structural families of optimize(): the family cases of golden/ref_optimize.json
def family_problem(case=None, c=1):
    """Config `c` (with the memory per device a golden case may set) with the AC-share template and its view
    under the PPO memory model as structures 1, 2."""
    import dataclasses
    from rpeg_amd.engine.problem import STRUCTURES, as_seen_from
    p = configs.config(c).problem
    if case and "memory_per_gpu" in case:
        p = dataclasses.replace(p, hw=dataclasses.replace(p.hw, memory_per_gpu=case["memory_per_gpu"]))
    if case and "transfer" in case:
        p = with_transfer_policy(p, *case["transfer"])
    ppo, ac = STRUCTURES["ppo"], STRUCTURES["ac_share"]
    return dataclasses.replace(p, structures=(ppo, ac, as_seen_from(ac, ppo)))


def family_case_setup(p, case, directory_of, **more):
    """(families, base row, OptimizerConfig) of one family case of tests/golden/ref_optimize.json."""
    from rpeg_amd.core.types import Model
    from rpeg_amd.ir.plan import ExecutionPlan
    from rpeg_amd.search.optimizer import OptimizerConfig, optimize_families, plan_row
    _, batch = seeded_batch(1, 8)
    rpeg0 = p.template(0, ())
    _, plan_m, _ = batch.configuration(p, case["plan"])
    row = plan_row(rpeg0, ExecutionPlan(sigma={v: plan_m.sigma[u] for v, u in zip(rpeg0.vertices, plan_m.sigma)},
                                        pi={v: plan_m.pi[u] for v, u in zip(rpeg0.vertices, plan_m.pi)},
                                        mb={v: plan_m.mb[u] for v, u in zip(rpeg0.vertices, plan_m.mb)}))
    a, c_, s_ = case["T_cand"]
    opt = OptimizerConfig(K_x=6, T_max=50, E_max=case["E_max"], E_struct=case["E_struct"], T_init=case["T_init"],
                          T_warm=case["T_warm"], T_min=case["T_min"], stag_window=case["stag_window"],
                          T_cand={Model.ACTOR: set(a), Model.CRITIC: set(c_), Model.AC_SHARE: set(s_)},
                          structural_candidates=frozenset({"separate", "ac_share"}), lambda_ac=case["lambda_ac"],
                          max_throughput_loss=case.get("max_throughput_loss", 0.0), **more)
    assert opt.T_cool.hex() == case["T_cool"]
    families = optimize_families(p, opt, directory_of)
    families[0][0].seed = case["stream"][0]
    return families, row, opt


def check_family_case(p, case, families, res):
    """The evaluation log of a run over families against the reference's: template, staleness and plan of
    every evaluation in order, the number of draws, the returned configuration."""
    log = []
    for rowv, var in zip(res["eval_log"], res["eval_log_variant"]):
        f, k = (0, None) if var == 255 else (int(var) // 8, int(var) % 8)
        prm = families[f][0]
        st = p.structures[prm.structure]
        taus = list(case["base_tau"]) if k is None else [int(prm.tau[k][i]) for i in range(len(st.tau_models))]
        nv = len(p.template(prm.structure, ()).vertices)
        log.append([p.template(prm.structure, ()).vertices[0].id, taus, rows6(rowv, nv)])
    assert log[:8] == case["first"]
    assert res["n_eval_log"] == case["n_eval"] == len(log)
    assert zlib.crc32(json.dumps(log, separators=(",", ":")).encode()) == case["eval_crc"]
    assert res["n_draws"] == case["n_draws"]
    prm = families[res["best_family"]][0]
    st = p.structures[prm.structure]
    rpeg = p.template(prm.structure, ())
    assert rpeg.vertices[0].id == case["final_first_vertex"]
    k = res["best_variant"]
    taus = list(case["base_tau"]) if k >= prm.n_variants else [int(prm.tau[k][i]) for i in range(len(st.tau_models))]
    assert taus == case["final_tau"]
    assert rows6(res["best_plan"], len(rpeg.vertices)) == case["final"]


# ---- non-default transfer resource policies: golden/ref_transfer_policy.json
def load_transfer_policy_golden():
    with open(os.path.join(GOLDEN, "ref_transfer_policy.json")) as f:
        return json.load(f)


def with_transfer_policy(problem, weight, activation):
    from dataclasses import replace
    from rpeg_amd.core.types import TransferResourcePolicy
    return replace(problem, transfer_resource_policy=TransferResourcePolicy(weight=weight, activation=activation))


# ---- non-default memory policies: golden/ref_memory_policy.json
def load_memory_policy_golden():
    with open(os.path.join(GOLDEN, "ref_memory_policy.json")) as f:
        return json.load(f)


def with_memory_policy(problem, fields):
    from dataclasses import replace
    from rpeg_amd.model.memory import MemoryPolicy
    return replace(problem, memory_policy=MemoryPolicy(**fields))


# ---- calibrated hardware records: golden/ref_hardware.json
def load_hardware_golden():
    with open(os.path.join(GOLDEN, "ref_hardware.json")) as f:
        return json.load(f)


def with_hardware(problem, fields):
    from dataclasses import replace
    return replace(problem, hw=replace(problem.hw, **fields))


# ---- problems away from the shipped configurations: golden/ref_variants.json
def variant_cases():
    """[(name, problem, seeded batch, reference rows)]"""
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_golden_variants", os.path.join(GOLDEN, "make_golden_variants.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    with open(os.path.join(GOLDEN, "ref_variants.json")) as f:
        gold = json.load(f)
    out = []
    for name, problem, tau_choices, tag in mod.variant_problems():
        batch = candidates.generate(problem, gold["n_plans"], tau_choices, seed=gold["seed"], tag=tag)
        out.append((name, problem, batch, gold["problems"][name]))
    return out
