"""The Python restatement of the simulated-annealing neighbourhood against vectors written by the
reference's own functions (tests/golden/make_golden_sa.py): candidate directory, critical-chain
masses, single-vertex proposals, donor/receiver proposals and the region sampler, each driven by
the same counter-based draws."""

import json
import os
import zlib

import pytest

from oracle import rpeg_oracle as O
from oracle import sa_oracle as S
from rpeg_amd.ir.plan import ExecutionPlan
from tests.helpers import GOLDEN, seeded_batch


def _gold():
    with open(os.path.join(GOLDEN, "ref_sa.json")) as f:
        return json.load(f)


def _world(c, n):
    cfg, batch = seeded_batch(c, n)
    p = cfg.problem
    rpeg0 = p.template(0, ())
    cost = O.CostModel(p.hw, p.suite, p.workload, p.memory_policy.optimizer_stage,
                       p.memory_policy.activation_checkpointing)
    mem = O.make_mem_model(rpeg0, p.suite, p.workload, p.hw, p.memory_policy)
    return cfg, batch, rpeg0, cost, mem


def _rows(rpeg, plan):
    return [[*plan.pi[v], plan.mb[v], *plan.sigma[v].origin, *plan.sigma[v].extent] for v in rpeg.vertices]


def _case_plan(p, batch, i):
    rpeg = p.template(0, (i % 2,))
    _, plan_m, _ = batch.configuration(p, i)
    by_id = {v.id: v for v in rpeg.vertices}
    plan = ExecutionPlan(sigma={by_id[v.id]: a for v, a in plan_m.sigma.items()},
                         pi={by_id[v.id]: x for v, x in plan_m.pi.items()},
                         mb={by_id[v.id]: x for v, x in plan_m.mb.items()})
    return rpeg, plan


@pytest.fixture(scope="module")
def gold():
    return _gold()


@pytest.mark.parametrize("c", [1, 5])
def test_candidate_directory_matches_reference(gold, c):
    g = gold["configs"][str(c)]["directory"]
    cfg, batch, rpeg0, cost, mem = _world(c, 1)
    p = cfg.problem
    table, index = S.build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, cost, mem)
    for v in rpeg0.vertices:
        want = g[v.id]
        assert len(S.enumerate_strategies(v, p.suite, p.device_space, p.workload)) == want["n_enumerated"]
        assert len(table[v]) == want["n"]
        keys = ",".join(str(x) for e in table[v] for x in e[:6])
        times = ",".join(e[6].hex() for e in table[v])
        assert zlib.crc32(keys.encode()) == want["key_crc"], v.id
        assert zlib.crc32(times.encode()) == want["time_crc"], v.id
        assert [list(e[:6]) + [e[6].hex()] for e in table[v][:6]] == want["head"]
        assert all(index[v][e[:6]] == j for j, e in enumerate(table[v]))


@pytest.mark.parametrize("c", [1, 5])
def test_proposals_match_reference(gold, c):
    cases = gold["configs"][str(c)]["cases"]
    cfg, batch, rpeg0, cost, mem = _world(c, len(cases))
    p = cfg.problem
    sp = p.device_space
    table0, index0 = S.build_candidate_directory(rpeg0, p.suite, sp, p.workload, cost, mem)
    for rec in cases:
        i = rec["i"]
        rpeg, plan = _case_plan(p, batch, i)
        table = {v: table0[v0] for v, v0 in zip(rpeg.vertices, rpeg0.vertices)}
        index = {v: index0[v0] for v, v0 in zip(rpeg.vertices, rpeg0.vertices)}
        r = O.evaluate_plan(rpeg, plan, sp, p.suite, p.workload, p.hw, p.K_eval, p.memory_policy,
                            check_stale=False, want_trace=True)
        chain = S.critical_chain(r["nodes"], r["edges"], r["finish"])
        assert len(chain) == rec["n_chain"], i
        assert zlib.crc32(",".join(sorted(n.id for n in chain)).encode()) == rec["chain_crc"], i
        mass = S.critical_mass(chain, rpeg, r["start"], r["finish"])
        for v, want in zip(rpeg.vertices, rec["mass"]):
            # the reference sums in the iteration order of a set of string-hashed nodes
            assert mass[v] == pytest.approx(float.fromhex(want), rel=1e-13, abs=0.0), (i, v.id)

        mg = rec["move_gen"]
        rng = S.CounterRng(42, c, i, 1)
        stats = {}
        out = S.move_gen(rng, rpeg, plan, sp, mass, table, index, 6, 50, mg["T"], mg["T_init"], stats)
        assert [_rows(rpeg, x) for x in out] == mg["plans"], i
        assert rng.k == mg["n_draws"], i
        assert stats.get("n_fallback", 0) == mg["fallback"], i

        rng = S.CounterRng(42, c, i, 2)
        nb = S.multi_move_pair(rng, rpeg, plan, sp, p.suite, p.workload)
        assert (None if nb is None else _rows(rpeg, nb)) == rec["pair"]["plan"], i
        assert rng.k == rec["pair"]["n_draws"], i

        rng = S.CounterRng(42, c, i, 3)
        rows = []
        for v in rpeg.vertices:
            lo = i % sp.R
            hi = min(sp.R, lo + 1 + (i // 3) % sp.R)
            s = S.sample_expl_in_region(rng, v, p.suite, sp, p.workload, lo, hi)
            rows.append(None if s is None else [*s[2], s[3], *s[0], *s[1]])
        assert rows == rec["sample"]["rows"], i
        assert rng.k == rec["sample"]["n_draws"], i


def test_counter_rng_choices_is_cpython_bisect():
    import random
    from bisect import bisect
    from itertools import accumulate
    rng, ref = S.CounterRng(7, 1, 2, 3), S.CounterRng(7, 1, 2, 3)
    pop, w = list("abcdef"), [0.5, 0.0, 2.0, 1e-6, 3.0, 0.25]
    cum = list(accumulate(w))
    for _ in range(200):
        got = rng.choices(pop, weights=w, k=1)[0]
        assert got == pop[bisect(cum, ref.random() * (cum[-1] + 0.0), 0, len(pop) - 1)]
    # same distribution as random.choices when fed the same uniform
    class Fixed(random.Random):
        def __init__(self, u): super().__init__(); self.u = u
        def random(self): return self.u
    for u in (0.0, 0.1, 0.5, 0.9999999):
        class One:
            def random(self_inner): return u
        r = S.CounterRng(1)
        r.random = lambda u=u: u
        assert r.choices(pop, weights=w, k=1) == Fixed(u).choices(pop, weights=w, k=1)


def test_polish_and_optimizer_config_match_reference():
    """The reference's own polish() (run unmodified by tests/golden/make_golden_polish.py) and the derived
    fields of its OptimizerConfig."""
    from rpeg_amd.search.optimizer import OptimizerConfig
    with open(os.path.join(GOLDEN, "ref_polish.json")) as f:
        g = json.load(f)
    oc = g["optimizer_config"]
    for name, cfg in (("default", OptimizerConfig()),
                      ("cfg5", OptimizerConfig(K_x=6, T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=10)),
                      ("e800", OptimizerConfig(E_struct=800, K_x=4))):
        assert [cfg.I_max, cfg.T_cool.hex()] == oc[name]
    cfg, batch, rpeg0, cost, mem = _world(1, 64)
    p = cfg.problem
    table, index = S.build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, cost, mem)
    ev = S.oracle_evaluator(rpeg0, p.device_space, p.suite, p.workload, p.hw, p.K_eval, p.memory_policy)
    for case in g["cases"]:
        _, plan_m, _ = batch.configuration(p, case["i"])
        by_id = {v.id: v for v in rpeg0.vertices}
        plan = ExecutionPlan(sigma={by_id[v.id]: a for v, a in plan_m.sigma.items()},
                             pi={by_id[v.id]: x for v, x in plan_m.pi.items()},
                             mb={by_id[v.id]: x for v, x in plan_m.mb.items()})
        assert ev(plan).gated.hex() == case["start_score"]
        out, score, rounds, n_eval = S.polish(rpeg0, plan, p.device_space, p.suite, p.workload, ev, table, index,
                                              g["T_min"], g["T_init"])
        assert _rows(rpeg0, out) == case["plan"], case["i"]
        assert score.hex() == case["final_score"], case["i"]
        assert n_eval - 1 == case["evaluations"], case["i"]


def test_chain_loop_matches_reference_optimize():
    """The reference's own optimize() (run unmodified, for one structural setting, on the counter-based
    generator by tests/golden/make_golden_optimize.py) against `serial_chain`, which is built from the
    same `propose` / `mh_accept` / elite functions as the population loop `run_chains`: every plan is
    evaluated in the same order, the same number of draws is consumed, the same plan is returned."""
    with open(os.path.join(GOLDEN, "ref_optimize.json")) as f:
        g = json.load(f)
    cfg, batch, rpeg0, cost, mem = _world(1, 8)
    p = cfg.problem
    table, index = S.build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, cost, mem)
    cases = [c for c in g["cases"] if not c.get("families")]
    assert [c.get("transfer") for c in cases] == [None, None, ["both_endpoints", "both_endpoints"]]
    for case in cases:
        ev = S.oracle_evaluator(rpeg0, p.device_space, p.suite, p.workload, p.hw, p.K_eval, p.memory_policy,
                                tuple(case.get("transfer", ("destination_only", "destination_only"))))
        _, plan_m, _ = batch.configuration(p, case["plan"])
        by_id = {v.id: v for v in rpeg0.vertices}
        plan = ExecutionPlan(sigma={by_id[v.id]: a for v, a in plan_m.sigma.items()},
                             pi={by_id[v.id]: x for v, x in plan_m.pi.items()},
                             mb={by_id[v.id]: x for v, x in plan_m.mb.items()})
        params = S.SaParams(K_x=6, T_max=50, T_init=case["T_init"], T_warm=case["T_warm"], T_min=case["T_min"],
                            stag_window=case["stag_window"], E_struct=case["E_struct"])
        assert params.T_cool.hex() == case["T_cool"]
        rng = S.CounterRng(*case["stream"])
        best, order = S.serial_chain(rng, rpeg0, plan, p.device_space, p.suite, p.workload, ev, (table, index),
                                     params, case["E_max"], case["E_struct"])
        log = [_rows(rpeg0, q) for q in order]
        assert log[:8] == case["first"]
        assert len(log) == case["n_eval"]
        assert zlib.crc32(json.dumps(log, separators=(",", ":")).encode()) == case["eval_crc"]
        assert rng.k == case["n_draws"]
        assert _rows(rpeg0, best) == case["final"]
