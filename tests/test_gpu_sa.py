"""GPU tests of the annealing path through the C ABI: critical-chain masses, the candidate directory,
and whole populations of chains (rpeg_sa_run) against the same host logic over the CPU build of the
evaluator, which the CPU suite ties to the Python restatement and the reference's vectors."""

import json
import os
import zlib

import numpy as np
import pytest

from oracle.cpu_port import CpuPort
from rpeg_amd import configs
from rpeg_amd.engine import abi
from rpeg_amd.search.moves import build_candidate_directory, directory_arrays
from rpeg_amd.search.optimizer import OptimizerConfig, optimize_chains, sa_params
from tests.helpers import GOLDEN, check_family_case, family_case_setup, family_problem, seeded_batch

pytestmark = pytest.mark.gpu

_engines = {}


def engine(c):
    from rpeg_amd.engine.runtime import Engine
    if c not in _engines:
        _engines[c] = Engine(configs.config(c).problem)
    return _engines[c]


def same_bits(a, b):
    return np.array_equal(np.asarray(a, np.float64).view(np.uint64), np.asarray(b, np.float64).view(np.uint64))


@pytest.mark.parametrize("c,n", [(1, 4096), (2, 16384), (3, 16384), (4, 16384), (5, 4096)])
def test_critical_mass_bit_exact(c, n):
    cfg, batch = seeded_batch(c, n)
    got = engine(c).eval_mass(batch)
    ref = CpuPort(cfg.problem).eval(batch, threads=16, want_mass=True)
    assert np.array_equal(got["mask"], ref["mask"])
    assert same_bits(got["score"], ref["score"])
    assert same_bits(got["mass"], ref["mass"])
    # the mass output must not disturb the plain outputs
    plain = engine(c).eval(batch, gate_stale=False)
    assert same_bits(plain["score"], got["score"]) and same_bits(plain["makespan"], got["makespan"])


@pytest.mark.parametrize("c", [1, 5])
def test_candidate_directory_matches_reference(c):
    with open(os.path.join(GOLDEN, "ref_sa.json")) as f:
        g = json.load(f)["configs"][str(c)]["directory"]
    p = configs.config(c).problem
    rpeg0 = p.template(0, ())
    table, index = build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, engine(c))
    for v in rpeg0.vertices:
        want = g[v.id]
        assert len(table[v]) == want["n"]
        keys = ",".join(str(x) for e in table[v] for x in e[:6])
        times = ",".join(e[6].hex() for e in table[v])
        assert zlib.crc32(keys.encode()) == want["key_crc"], v.id
        assert zlib.crc32(times.encode()) == want["time_crc"], v.id
        assert all(index[v][e[:6]] == j for j, e in enumerate(table[v]))


def _variants(p):
    n_tau = len(p.structures[0].tau_models)
    return [(0,) * n_tau, (1,) + (0,) * (n_tau - 1)]


@pytest.mark.parametrize("c,n_chains,n_steps,kw", [
    (1, 64, 200, dict(T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=10)),
    (2, 32, 100, dict(T_init=0.30, T_min=0.01, T_warm=0.05, stag_window=5, geometric_cooling=True)),
    (5, 64, 2000, dict(T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=10)),   # the whole run of config 5
])
def test_chains_equal_host_replay(c, n_chains, n_steps, kw):
    """Same counter-based draws, GPU evaluator against CPU evaluator: every decision of every chain,
    the final plans, the best plans and their scores are identical."""
    p = configs.config(c).problem
    eng = engine(c)
    opt = OptimizerConfig(**kw)
    rpeg0 = p.template(0, ())
    table, _ = build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, eng)
    arrays = directory_arrays(rpeg0, table)
    got = optimize_chains(p, opt, n_chains, n_steps, _variants(p), seed=42, engine=eng, directory=arrays)
    split = 1 if p.workload.gen_quantiles else 0
    ref = CpuPort(p).sa_run(sa_params(opt, n_chains, n_steps, _variants(p), 0, split, 42), arrays, threads=16)
    assert np.array_equal(got.log, ref["log"])
    assert np.array_equal(got.cur_plan, ref["cur_plan"]) and same_bits(got.cur_score, ref["cur_score"])
    assert np.array_equal(got.best_plan, ref["best_plan"]) and same_bits(got.best_score, ref["best_score"])
    assert np.array_equal(got.best_step, ref["best_step"]) and np.array_equal(got.best_feasible, ref["best_feasible"])
    assert np.array_equal(got.restarts, ref["restarts"]) and np.array_equal(got.n_eval, ref["n_eval"])
    assert np.array_equal(got.dead, ref["dead"])
    live = ~got.dead.astype(bool)
    assert live.any()
    assert ((got.log >> 4) & 3 == 2).sum() > 0, "no accepted move in the whole population"
    assert got.n_launch >= n_steps


def test_groups_of_chains_overlap_without_changing_the_run():
    """rpeg_engine_set_sa_groups: 1, 2 and 3 groups (streams, staging buffers, polled completion flags of their own)
    give the same decisions, plans and scores bit for bit, and as many launches as groups per step."""
    p = configs.config(5).problem
    eng = engine(5)
    opt = OptimizerConfig(T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=10)
    rpeg0 = p.template(0, ())
    table, _ = build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, eng)
    arrays = directory_arrays(rpeg0, table)
    runs = {}
    try:
        for groups in (1, 2, 3, 8):
            eng.set_sa_groups(groups)
            runs[groups] = optimize_chains(p, opt, 32, 150, _variants(p), seed=7, engine=eng, directory=arrays)
    finally:
        eng.set_sa_groups(3)
    one = runs[1]
    assert ((one.log >> 4) & 3 == 2).sum() > 0
    for groups, got in runs.items():
        assert np.array_equal(got.log, one.log), groups
        assert np.array_equal(got.cur_plan, one.cur_plan) and same_bits(got.cur_score, one.cur_score), groups
        assert np.array_equal(got.best_plan, one.best_plan) and same_bits(got.best_score, one.best_score), groups
        assert np.array_equal(got.restarts, one.restarts) and np.array_equal(got.n_eval, one.n_eval), groups
        assert got.n_launch >= min(groups, 4) * 150, groups     # (at least 8 chains to a group: 32 chains make 4)
    with pytest.raises(Exception):
        eng.set_sa_groups(0)


def test_base_plan_start_and_gate():
    p = configs.config(1).problem
    eng = engine(1)
    cfg, batch = seeded_batch(1, 64)
    out = eng.eval(batch, gate_stale=True)
    ok = np.flatnonzero((out["mask"] & 7) == 7)
    assert ok.size
    rpeg, plan, _ = batch.configuration(p, int(ok[0]))
    opt = OptimizerConfig(T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=10)
    res = optimize_chains(p, opt, 8, 50, [(0, 0)], seed=7, base_plan=plan, engine=eng, gate_candidates=True)
    assert not res.dead.any() and res.best_feasible.all()
    # a chain never reports a best feasible score below that of its valid start
    assert (res.best_score >= out["score"][ok[0]]).all()
    c = res.argbest()
    assert res.best_score[c] == res.best_score.max()


def test_polish_equals_reference():
    """The drop-in polish() on the GPU evaluator against what the reference's own polish() returned for the
    same start plans (tests/golden/make_golden_polish.py): same final plan, same score."""
    from rpeg_amd.ir.plan import ExecutionPlan
    from rpeg_amd.search.cache import EvalCache
    from rpeg_amd.search.evaluate import Configuration, evaluate_cached
    from rpeg_amd.search.optimizer import plan_row, polish
    with open(os.path.join(GOLDEN, "ref_polish.json")) as f:
        g = json.load(f)
    cfg, batch = seeded_batch(1, 64)
    p = cfg.problem
    rpeg0 = p.template(0, ())
    table, index = build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, engine(1))
    opt = OptimizerConfig(K_x=1, T_init=g["T_init"], T_min=g["T_min"])
    nv = len(rpeg0.vertices)
    for case in g["cases"]:
        _, plan_m, _ = batch.configuration(p, case["i"])
        by_id = {v.id: v for v in rpeg0.vertices}
        plan = ExecutionPlan(sigma={by_id[v.id]: a for v, a in plan_m.sigma.items()},
                             pi={by_id[v.id]: x for v, x in plan_m.pi.items()},
                             mb={by_id[v.id]: x for v, x in plan_m.mb.items()})
        start = Configuration(rpeg0, plan, p.device_space)
        cache = EvalCache()
        out = polish(start, p.suite, p.workload, p.hw, p.K_eval, opt, cache, table, index)
        rows = plan_row(rpeg0, out.plan)
        assert [[int(x) for x in rows[v * 10:(v + 1) * 10]] for v in range(nv)] == case["plan"], case["i"]
        score, _, feasible, _ = evaluate_cached(out, EvalCache(), p.suite, p.workload, p.hw, p.K_eval, p.memory_policy)
        assert float(score).hex() == case["final_score"] and feasible == case["final_feasible"]
        assert cache.misses - 1 == case["evaluations"]
    # the same starts under the utilisation objective (max_throughput_loss > 0, optimizer.py:1021-1044): other
    # final plans, again the reference's
    for case in g["utilisation_cases"]:
        _, plan_m, _ = batch.configuration(p, case["i"])
        by_id = {v.id: v for v in rpeg0.vertices}
        plan = ExecutionPlan(sigma={by_id[v.id]: a for v, a in plan_m.sigma.items()},
                             pi={by_id[v.id]: x for v, x in plan_m.pi.items()},
                             mb={by_id[v.id]: x for v, x in plan_m.mb.items()})
        opt_u = OptimizerConfig(K_x=1, T_init=g["T_init"], T_min=g["T_min"], max_throughput_loss=case["max_throughput_loss"])
        cache = EvalCache()
        out = polish(Configuration(rpeg0, plan, p.device_space), p.suite, p.workload, p.hw, p.K_eval, opt_u, cache, table, index)
        rows = plan_row(rpeg0, out.plan)
        assert [[int(x) for x in rows[v * 10:(v + 1) * 10]] for v in range(nv)] == case["plan"], case["i"]
        score, trace, feasible, _ = evaluate_cached(out, EvalCache(), p.suite, p.workload, p.hw, p.K_eval, p.memory_policy)
        assert float(score).hex() == case["final_score"] and feasible == case["final_feasible"]
        assert float(trace.utilization()).hex() == case["final_utilization"]
        assert cache.misses - 1 == case["evaluations"]


def test_optimize_equals_reference_trajectory():
    """rpeg_sa_optimize on the GPU evaluator against the trajectory of the reference's own optimize() on the
    same generator: same plans evaluated in the same order, same draws, same returned plan; and the
    drop-in optimize() built on it."""
    from rpeg_amd.ir.plan import ExecutionPlan
    from rpeg_amd.search.cache import EvalCache
    from rpeg_amd.search.evaluate import Configuration, evaluate_cached
    from rpeg_amd.search.optimizer import optimize, plan_row
    with open(os.path.join(GOLDEN, "ref_optimize.json")) as f:
        g = json.load(f)
    cfg, batch = seeded_batch(1, 8)
    p = cfg.problem
    eng = engine(1)
    rpeg0 = p.template(0, ())
    nv = len(rpeg0.vertices)
    table, _ = build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, eng)
    arrays = directory_arrays(rpeg0, table)

    def rows(r):
        return [[int(x) for x in r[v * 10:(v + 1) * 10]] for v in range(nv)]
    from rpeg_amd.core.types import TransferResourcePolicy
    from rpeg_amd.engine.runtime import Engine
    from tests.helpers import with_transfer_policy
    for case in [c for c in g["cases"] if not c.get("families")]:
        # a case may ask for both-endpoints transfer reservations: another problem, hence another engine
        tp = TransferResourcePolicy(*case["transfer"]) if "transfer" in case else None
        eng = Engine(with_transfer_policy(p, *case["transfer"])) if tp else engine(1)
        _, plan_m, _ = batch.configuration(p, case["plan"])
        by_id = {v.id: v for v in rpeg0.vertices}
        plan = ExecutionPlan(sigma={by_id[v.id]: a for v, a in plan_m.sigma.items()},
                             pi={by_id[v.id]: x for v, x in plan_m.pi.items()},
                             mb={by_id[v.id]: x for v, x in plan_m.mb.items()})
        opt = OptimizerConfig(K_x=6, T_max=50, E_max=case["E_max"], E_struct=case["E_struct"], T_init=case["T_init"],
                              T_warm=case["T_warm"], T_min=case["T_min"], stag_window=case["stag_window"],
                              T_cand={m: {0} for m in rpeg0.tau}, structural_candidates=frozenset({"separate"}))
        res = eng.sa_optimize(sa_params(opt, 1, 1, [(0, 0)], 0, 1, case["stream"][0]), arrays, plan_row(rpeg0, plan),
                              case["E_max"], case["E_struct"], stream_key=case["stream"][1:], log_cap=4096)
        log = [rows(r) for r in res["eval_log"]]
        assert log[:8] == case["first"] and res["n_eval_log"] == case["n_eval"]
        assert zlib.crc32(json.dumps(log, separators=(",", ":")).encode()) == case["eval_crc"]
        assert res["n_draws"] == case["n_draws"] and rows(res["best_plan"]) == case["final"]
        base = Configuration(rpeg0, plan, p.device_space, transfer_resource_policy=tp)
        out = optimize(base, p.suite, p.workload, p.hw, p.K_eval, opt, EvalCache(), seed=case["stream"][0],
                       stream_key=case["stream"][1:])
        assert rows(plan_row(out.rpeg, out.plan)) == case["final"] and out.transfer_resource_policy == tp
        s1, _, f1, _ = evaluate_cached(out, EvalCache(), p.suite, p.workload, p.hw, p.K_eval, p.memory_policy)
        s0, _, _, _ = evaluate_cached(base, EvalCache(), p.suite, p.workload, p.hw, p.K_eval, p.memory_policy)
        assert f1 and s1 >= s0


def test_annealing_argument_errors_and_edges():
    from rpeg_amd.engine.runtime import EngineError
    p = configs.config(1).problem
    eng = engine(1)
    rpeg0 = p.template(0, ())
    table, _ = build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, eng)
    arrays = directory_arrays(rpeg0, table)
    opt = OptimizerConfig(T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=10)
    res = optimize_chains(p, opt, 4, 0, [(0, 0)], engine=eng, directory=arrays)          # no steps: only the starts
    assert res.log.shape == (4, 0) and not res.dead.any() and (res.best_step == -1).all()
    for bad in (dict(K_x=17), dict(K_x=0)):
        with pytest.raises(EngineError, match="bad annealing parameters"):
            optimize_chains(p, OptimizerConfig(T_init=0.05, T_min=0.05, **bad), 2, 1, [(0, 0)], engine=eng, directory=arrays)
    big = [np.full((3, 6), 2000, np.int16)] * 6
    with pytest.raises(EngineError, match="outside 0..1023"):
        optimize_chains(p, opt, 2, 1, [(0, 0)], engine=eng, directory=big)
    empty = [np.zeros((0, 6), np.int16)] * 6                                              # empty directory: placement and pair moves only
    res = optimize_chains(p, opt, 4, 20, [(0, 0)], engine=eng, directory=empty)
    assert not res.dead.any() and ((res.log >> 1) & 7).max() <= 1


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_start_plans_equal_the_reference_pipelines(c):
    """The greedy, fully colocated and hand-partitioned start plans (RPEG/pipeline.py:389-435, 1051-1201)
    from the engine's directory: same rows as the reference built on the same template, and where the
    reference finds no plan, the same error with the same text."""
    from rpeg_amd.search import baselines
    with open(os.path.join(GOLDEN, "ref_baselines.json")) as f:
        g = json.load(f)["configs"][str(c)]
    p = configs.config(c).problem
    rpeg0 = p.template(0, ())
    table, _ = build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, engine(c))
    for name in ("build_valid_baseline_plan", "build_fullycolocated_baseline_plan", "build_naive_concurrent_plan"):
        want, build = g[name], getattr(baselines, name)
        if "error" in want:
            with pytest.raises(RuntimeError) as ex:
                build(rpeg0, p.device_space, p.suite, p.workload, engine(c), table=table)
            assert str(ex.value) == want["message"]
            continue
        plan = build(rpeg0, p.device_space, p.suite, p.workload, engine(c), table=table)
        rows = [[*plan.pi[v], plan.mb[v], *plan.sigma[v].origin, *plan.sigma[v].extent] for v in rpeg0.vertices]
        assert rows == want["rows"], name
    # without a directory handed in the constructor builds its own
    plan = baselines.build_valid_baseline_plan(rpeg0, p.device_space, p.suite, p.workload, engine(c))
    assert [[*plan.pi[v], plan.mb[v]] for v in rpeg0.vertices] == [r[:4] for r in g["build_valid_baseline_plan"]["rows"]]


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_concurrent_start_plan_takes_the_reference_cascade(c):
    """build_concurrent_baseline_plan (RPEG/pipeline.py:908-1048): the plans it would try are the plans the
    reference lowered for its memory check, in the same order (1 to 473 of them; on config 3 all 345 fail and
    the greedy plan is returned); the engine's peak of each failing one equals the peak the reference's K = 1
    check reported, bit for bit; the returned plan and flag are the reference's."""
    from rpeg_amd.engine.problem import PlanBatch
    from rpeg_amd.search import baselines
    with open(os.path.join(GOLDEN, "ref_baselines.json")) as f:
        g = json.load(f)["configs"][str(c)]["build_concurrent_baseline_plan"]
    p = configs.config(c).problem
    rpeg0 = p.template(0, ())
    eng = engine(c)
    table, _ = build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, eng)

    def rows(plan):
        return [[*plan.pi[v], plan.mb[v], *plan.sigma[v].origin, *plan.sigma[v].extent] for v in rpeg0.vertices]

    cascade = baselines.concurrent_plan_cascade(rpeg0, p.device_space, table)
    tried = g["tried"]
    assert len(cascade) >= len(tried)
    assert [rows(pl) for pl, _, _ in cascade[:len(tried)]] == [t["rows"] for t in tried]
    if not g["found"]:
        assert len(cascade) == len(tried)

    batch = PlanBatch.empty(len(tried))
    taus = [int(rpeg0.tau[m]) for m in p.structures[0].tau_models]
    for i, (pl, _, _) in enumerate(cascade[:len(tried)]):
        batch.set_plan(i, 0, 1 if p.workload.gen_quantiles else 0, taus, rpeg0, pl)
    out = eng.eval(batch, gate_stale=False)
    for i, t in enumerate(tried):
        fits = bool(out["mask"][i] & abi.MASK_MEM_OK)
        assert fits == (t["peak_over_cap"] is None), i
        if not fits:
            assert float(out["peak"][i]).hex() == t["peak_over_cap"], i

    plan, found = baselines.build_concurrent_baseline_plan(rpeg0, p.device_space, p.suite, p.workload, eng, table=table)
    assert found == g["found"] and rows(plan) == g["rows"]


def test_optimize_over_structural_families_equals_reference():
    """rpeg_sa_optimize_families on the GPU evaluator against the reference's optimize() with
    structural_candidates {"separate", "ac_share"} (RPEG/search/optimizer.py:541-946): the separate
    template's staleness variants, then the AC-share template's, started from random plans that is_valid
    checks with the base configuration's memory model (structure 2 of the problem).  Every evaluated
    (template, staleness, plan) in order, the number of draws, the returned configuration -- an AC-share one
    in two of the four cases; the third runs with 12.5 GB per device, where the two memory models disagree; the
    fourth ranks by throughput x utilisation (max_throughput_loss = 0.1, optimizer.py:461-486), every evaluated
    plan traced for Trace.utilization().  The drop-in optimize() returns the same configurations."""
    from rpeg_amd.engine.runtime import Engine
    from rpeg_amd.search.cache import EvalCache
    from rpeg_amd.search.evaluate import Configuration
    from rpeg_amd.search.optimizer import optimize, plan_row, row_plan
    with open(os.path.join(GOLDEN, "ref_optimize.json")) as f:
        g = json.load(f)
    cases = [c for c in g["cases"] if c.get("families")]
    assert len(cases) == 5 and cases[3]["max_throughput_loss"] > 0 and cases[4]["transfer"][1] == "both_endpoints"
    for case in cases:
        p = family_problem(case)
        eng = Engine(p)

        def directory_of(structure):
            rpeg = p.template(structure, ())
            return directory_arrays(rpeg, build_candidate_directory(rpeg, p.suite, p.device_space, p.workload, eng,
                                                                    structure)[0])

        families, row, opt = family_case_setup(p, case, directory_of)
        res = eng.sa_optimize_families(families, case["base_tau"], row, case["E_max"], case["E_struct"],
                                       stream_key=case["stream"][1:], log_cap=4096)
        check_family_case(p, case, families, res)

        base_rpeg = p.template(0, case["base_tau"])
        base = Configuration(base_rpeg, row_plan(base_rpeg, row), p.device_space,
                             transfer_resource_policy=p.transfer_resource_policy if "transfer" in case else None)
        out = optimize(base, p.suite, p.workload, p.hw, p.K_eval, opt, EvalCache(), seed=case["stream"][0],
                       stream_key=case["stream"][1:])
        assert out.rpeg.vertices[0].id == case["final_first_vertex"]
        assert [out.rpeg.tau[m] for m in sorted(out.rpeg.tau, key=lambda m: m.value)] == case["final_tau"]
        nv = len(out.rpeg.vertices)
        got = plan_row(out.rpeg, out.plan)
        assert [[int(x) for x in got[v * 10:(v + 1) * 10]] for v in range(nv)] == case["final"]
        eng.close()


def test_search_pipeline_equals_reference_pipeline():
    """search_plan on config 1 against the same steps of the reference's pipeline (RPEG/pipeline.py:1412-1560,
    tests/golden/make_golden_optimize.py): the concurrent and the greedy start plan, the configuration optimize()
    returns over both structural families when seeded with the concurrent plan, what polish() makes of it on
    the shared cache, their scores, and the number of evaluations that end up in the cache."""
    from rpeg_amd.search.optimizer import plan_row
    from rpeg_amd.search.pipeline import search_plan
    with open(os.path.join(GOLDEN, "ref_optimize.json")) as f:
        g = json.load(f)["pipeline"]
    p = configs.config(1).problem
    opt = OptimizerConfig(K_x=6, T_max=50, E_max=g["E_max"], E_struct=g["E_struct"], T_init=g["T_init"],
                          T_warm=g["T_warm"], T_min=g["T_min"], stag_window=g["stag_window"], lambda_ac=g["lambda_ac"],
                          structural_candidates=frozenset({"separate", "ac_share"}))
    res = search_plan(p.suite, p.workload, p.hw, p.device_space, p.K_eval, opt, algorithm="ppo", seed=g["stream"][0],
                      stream_key=g["stream"][1:])

    def rows(config):
        r = plan_row(config.rpeg, config.plan)
        return [[int(x) for x in r[v * 10:(v + 1) * 10]] for v in range(len(config.rpeg.vertices))]

    def setting(config):
        return dict(first_vertex=config.rpeg.vertices[0].id, rows=rows(config),
                    tau=[config.rpeg.tau[m] for m in sorted(config.rpeg.tau, key=lambda m: m.value)])

    assert res.concurrent_found == g["concurrent_found"]
    assert rows(res.start) == g["start"] and rows(res.greedy) == g["greedy"]
    assert setting(res.optimized) == g["optimized"] and float(res.scores["optimized"]).hex() == g["optimized_score"]
    assert setting(res.polished) == g["polished"] and float(res.scores["polished"]).hex() == g["polished_score"]
    n_before = len({json.dumps(g["start"]), json.dumps(g["greedy"])})
    assert res.cache.misses == n_before + g["n_optimize"] + g["n_polish"]


def test_search_from_config_file_writes_loadable_plans(tmp_path):
    """search_from_config on the YAML of config 1 (the reference's schema) with small budgets: the plan files named
    in its output section are written in the reference's plan schema and load back to the plans returned; the
    polished plan is feasible and no worse than the start."""
    import yaml
    from rpeg_amd import config_io
    from rpeg_amd.ir.serialize import load_plan
    from rpeg_amd.search.cache import EvalCache
    from rpeg_amd.search.evaluate import evaluate_cached
    from rpeg_amd.search.optimizer import plan_row
    from rpeg_amd.search.pipeline import search_from_config
    here = os.path.dirname(os.path.abspath(config_io.__file__))
    cfg = config_io.load_config(os.path.join(here, "config_files", "cfg1.yaml"))
    cfg["optimizer"].update(e_max=200, e_struct=60, stag_window=4)
    cfg["output"] = {"base_plan": str(tmp_path / "base.yaml"), "opt_plan": str(tmp_path / "opt.yaml"), "seed": 7}
    hw = tmp_path / "hw.yaml"
    hw.write_text(f"memory_per_gpu: {cfg['hardware']['memory_per_gpu']}  # unchanged\n")
    res = search_from_config(cfg, hw_overlay=str(hw))
    assert res.scores["polished"] >= res.scores["optimized"] >= res.scores["start"] > 0
    for config, name in ((res.start, "base.yaml"), (res.polished, "opt.yaml")):
        back = load_plan(str(tmp_path / name), config.rpeg)
        assert list(plan_row(config.rpeg, back)) == list(plan_row(config.rpeg, config.plan))
    p = config_io.problem_from_config(cfg)
    _, _, feasible, _ = evaluate_cached(res.polished, EvalCache(), p.suite, p.workload, p.hw, p.K_eval, p.memory_policy)
    assert feasible
    # the run is a function of the seed
    again = search_from_config(cfg, hw_overlay=str(hw))
    assert list(plan_row(again.polished.rpeg, again.polished.plan)) == list(plan_row(res.polished.rpeg, res.polished.plan))


def test_planner_sequence_of_the_runtime_under_a_transfer_policy():
    """The calls of the reference's second caller in its order (runtime/job_plan.py:85-213): a base configuration
    that carries a both-endpoints policy, is_valid, optimize(), then the result lowered and scheduled at another
    horizon and serialised.  The optimised plan is no worse than the base under that policy, and the schedule at
    the new horizon equals the oracle's under the same policy (times, dispatch order)."""
    from rpeg_amd.core.types import CONSERVATIVE_TRANSFER_RESOURCE_POLICY as tp
    from rpeg_amd.ir import serialize as ser
    from rpeg_amd.model.memory import NodeMemoryModel
    from rpeg_amd.search.baselines import build_valid_baseline_plan
    from rpeg_amd.search.cache import EvalCache
    from rpeg_amd.search.evaluate import Configuration, _engine_for, evaluate, evaluate_cached, is_valid
    from rpeg_amd.search.optimizer import optimize
    from oracle import rpeg_oracle as oracle
    p = configs.config(1).problem
    rpeg = p.template(0, ())
    eng, _ = _engine_for(rpeg, p.suite, p.workload, p.hw, p.device_space, p.K_eval, p.memory_policy, transfer_policy=tp)
    plan = build_valid_baseline_plan(rpeg, p.device_space, p.suite, p.workload, eng)
    base = Configuration(rpeg, plan, p.device_space, transfer_resource_policy=tp)
    mm = NodeMemoryModel.from_policy(p.hw, p.suite, p.workload, p.memory_policy, trainable=frozenset(rpeg.trainable))
    assert is_valid(base, p.suite, p.workload, mm)
    opt = OptimizerConfig(K_x=6, T_max=50, E_max=150, E_struct=150, T_cand={m: {0} for m in rpeg.tau},
                          structural_candidates=frozenset({"separate"}))
    cache = EvalCache()
    best = optimize(base, p.suite, p.workload, p.hw, p.K_eval, opt, cache, seed=5)
    assert best.transfer_resource_policy == tp
    s0 = evaluate_cached(base, EvalCache(), p.suite, p.workload, p.hw, p.K_eval, p.memory_policy)[0]
    s1, _, feasible, _ = evaluate_cached(best, EvalCache(), p.suite, p.workload, p.hw, p.K_eval, p.memory_policy)
    assert feasible and s1 >= s0
    for config, score in ((base, s0), (best, s1)):   # the scores are the oracle's under that policy, not the default's
        want = oracle.evaluate_plan(config.rpeg, config.plan, p.device_space, p.suite, p.workload, p.hw, p.K_eval,
                                    p.memory_policy, transfer_policy=(tp.weight, tp.activation))
        assert score == want["score"]
    horizon = 3
    _, trace, lowered = evaluate(best, p.suite, p.workload, p.hw, horizon, p.memory_policy)
    want = oracle.evaluate_plan(best.rpeg, best.plan, p.device_space, p.suite, p.workload, p.hw, horizon,
                                p.memory_policy, want_trace=True, transfer_policy=(tp.weight, tp.activation))
    doc = ser.execution_schedule_to_dict(trace, horizon=horizon)
    assert doc["horizon"] == horizon and doc["predicted_makespan_s"] == want["makespan"]
    assert [n["node_id"] for n in doc["nodes"]] == list(want["order"])
    assert [n["predicted_finish_s"] for n in doc["nodes"]] == [want["finish"][i] for i in want["order"]]


@pytest.mark.parametrize("k", range(8))
def test_optimize_ablations_and_deadlines_equal_reference(k):
    """OptimizerConfig's ablation switches and wall-clock deadline on the GPU evaluator, through
    rpeg_sa_optimize / rpeg_sa_optimize_families and through the drop-in optimize(), against the reference's own
    optimize() run with the same switches, generator and ticking clock (the flag cases of
    tests/golden/make_golden_optimize.py): every evaluated plan and its score in order, the draws, the number
    of clock readings, the returned configuration."""
    import ctypes as C
    from rpeg_amd.engine.runtime import Engine
    from rpeg_amd.search import evaluate as evaluate_mod, moves as moves_mod
    from rpeg_amd.search.cache import EvalCache
    from rpeg_amd.search.evaluate import Configuration
    from rpeg_amd.search.optimizer import optimize, plan_row, row_plan
    with open(os.path.join(GOLDEN, "ref_optimize.json")) as f:
        case = json.load(f)["flag_cases"][k]
    flags = {name: bool(case.get(name)) for name in ("fixed_mb", "uniform_vertex", "hard_oom")}

    class Ticking:
        def __init__(self):
            self.reads = 0
            self.fn = abi.CLOCK_FN(lambda _ctx: self())

        def __call__(self):
            self.reads += 1
            return float(self.reads)

    def timed(params, clock):
        if "deadline" in case:
            params.timed, params.deadline_s, params.clock = 1, case["deadline"], C.cast(clock.fn, C.c_void_p)

    p = family_problem(case) if case.get("families") else configs.config(1).problem
    eng = Engine(p)
    moves_mod.ABLATION_FIXED_MB = flags["fixed_mb"]
    try:
        def directory_of(structure):
            rpeg = p.template(structure, ())
            return directory_arrays(rpeg, build_candidate_directory(rpeg, p.suite, p.device_space, p.workload, eng,
                                                                    structure)[0])
        clock = Ticking()
        if case.get("families"):
            families, row, opt = family_case_setup(p, case, directory_of, **flags)
            timed(families[0][0], clock)
            res = eng.sa_optimize_families(families, case["base_tau"], row, case["E_max"], case["E_struct"],
                                           stream_key=case["stream"][1:], log_cap=4096)
            check_family_case(p, case, families, res)
            base_tau = case["base_tau"]
        else:
            _, batch = seeded_batch(1, 8)
            rpeg0 = p.template(0, ())
            nv = len(rpeg0.vertices)
            _, plan_m, _ = batch.configuration(p, case["plan"])
            by_id = {v.id: v for v in rpeg0.vertices}
            from rpeg_amd.ir.plan import ExecutionPlan
            row = plan_row(rpeg0, ExecutionPlan(sigma={by_id[v.id]: a for v, a in plan_m.sigma.items()},
                                                pi={by_id[v.id]: x for v, x in plan_m.pi.items()},
                                                mb={by_id[v.id]: x for v, x in plan_m.mb.items()}))
            opt = OptimizerConfig(K_x=6, T_max=50, E_max=case["E_max"], E_struct=case["E_struct"], T_init=case["T_init"],
                                  T_warm=case["T_warm"], T_min=case["T_min"], stag_window=case["stag_window"],
                                  T_cand={m: {0} for m in rpeg0.tau}, structural_candidates=frozenset({"separate"}), **flags)
            params = sa_params(opt, 1, 1, [(0, 0)], 0, 1, case["stream"][0])
            timed(params, clock)
            res = eng.sa_optimize(params, directory_of(0), row, case["E_max"], case["E_struct"],
                                  stream_key=case["stream"][1:], log_cap=4096)
            log = [[[int(x) for x in r[v * 10:(v + 1) * 10]] for v in range(nv)] for r in res["eval_log"]]
            assert log[:8] == case["first"] and res["n_eval_log"] == case["n_eval"] == len(log)
            assert zlib.crc32(json.dumps(log, separators=(",", ":")).encode()) == case["eval_crc"]
            assert res["n_draws"] == case["n_draws"]
            base_tau = [0, 0]
        scores = [float(x).hex() for x in res["eval_log_score"]]
        assert zlib.crc32(json.dumps(scores).encode()) == case["eval_scores_crc"]
        assert clock.reads == case["clock_reads"]
        assert res["timed_out"] == ("deadline" in case and case["n_eval"] < case["E_max"])

        # the drop-in: switches and deadline from the OptimizerConfig, the clock in perf_counter's place
        import dataclasses
        clock = Ticking()
        moves_mod.ABLATION_FIXED_MB = False
        base_rpeg = p.template(0, base_tau)
        base = Configuration(base_rpeg, row_plan(base_rpeg, row), p.device_space)
        out = optimize(base, p.suite, p.workload, p.hw, p.K_eval, dataclasses.replace(opt, deadline=case.get("deadline")),
                       EvalCache(), seed=case["stream"][0], stream_key=case["stream"][1:],
                       clock=clock if "deadline" in case else None)
        assert (moves_mod.ABLATION_FIXED_MB, moves_mod.ABLATION_UNIFORM_VERTEX, evaluate_mod.ABLATION_HARD_OOM) == \
            (flags["fixed_mb"], flags["uniform_vertex"], flags["hard_oom"])       # optimizer.py:408-410
        assert out.rpeg.vertices[0].id == case["final_first_vertex"]
        assert [out.rpeg.tau[m] for m in sorted(out.rpeg.tau, key=lambda m: m.value)] == case["final_tau"]
        got = plan_row(out.rpeg, out.plan)
        assert [[int(x) for x in got[v * 10:(v + 1) * 10]] for v in range(len(out.rpeg.vertices))] == case["final"]
        assert clock.reads == case["clock_reads"]
    finally:
        moves_mod.ABLATION_FIXED_MB = moves_mod.ABLATION_UNIFORM_VERTEX = False
        evaluate_mod.ABLATION_HARD_OOM = False
        eng.close()


def test_time_budget_ends_the_search_on_the_wall_clock():
    """--time of the reference's pipeline (RPEG/pipeline.py:1351-1366, 1542-1545) on the real clock: with the
    evaluation budget lifted, a budget of a fraction of a second ends optimize() shortly after it (one batch of
    K_x evaluations may be under way), a budget of zero leaves the start plan, and more time never gives a
    worse plan on the same generator."""
    import time
    from rpeg_amd.search.pipeline import search_plan
    p = configs.config(1).problem
    opt = OptimizerConfig(K_x=6, T_max=50, E_max=100, E_struct=10 ** 6, structural_candidates=frozenset({"separate"}),
                          T_cand={m: {0} for m in p.template(0, ()).tau})
    search_plan(p.suite, p.workload, p.hw, p.device_space, p.K_eval, opt, algorithm="ppo", no_polish=True)   # warm-up
    got = {}
    for budget in (0.0, 0.1, 0.5):
        t0 = time.perf_counter()
        res = search_plan(p.suite, p.workload, p.hw, p.device_space, p.K_eval, opt, algorithm="ppo", no_polish=True,
                          time_budget=budget)
        got[budget] = res
        # (optimize() also enters what the run evaluated into the shared cache afterwards: host work per evaluation)
        assert budget <= res.seconds["optimize"] < budget + 0.1 + 2e-3 * res.cache.misses, (budget, res.seconds)
        assert time.perf_counter() - t0 < budget + 5.0
    assert got[0.0].scores["optimized"] == got[0.0].scores["start"]
    assert got[0.0].scores["optimized"] <= got[0.1].scores["optimized"] <= got[0.5].scores["optimized"]
    counts = {b: (r.cache.misses, r.seconds) for b, r in got.items()}
    assert got[0.5].cache.misses > got[0.1].cache.misses > got[0.0].cache.misses, counts
