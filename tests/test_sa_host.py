"""The shipped annealing host logic (rpeg_amd/csrc/rpeg_sa.h) and the critical-chain mass of the shared
scheduler code, run through the CPU build of the kernels' headers:

* its proposal kernels against the vectors written by the reference's own move_gen / multi_move_pair /
  sample_expl_in_region (same counter-based draws),
* its critical-chain masses against the Python restatement,
* a whole population of chains against the Python restatement of the chain loop: identical
  trajectories, step by step.
"""

import ctypes as C
import json
import os

import numpy as np
import pytest

from oracle import rpeg_oracle as O
from oracle import sa_oracle as S
from oracle.cpu_port import CpuPort
from rpeg_amd import configs
from rpeg_amd.core.types import Allocation
from rpeg_amd.engine import abi
from rpeg_amd.ir.plan import ExecutionPlan
from rpeg_amd.search.optimizer import OptimizerConfig, plan_row, sa_params
from tests.helpers import (GOLDEN, check_family_case, family_case_setup, family_problem, seeded_batch,
                           with_transfer_policy)


def _directory(p, rpeg0):
    cost = O.CostModel(p.hw, p.suite, p.workload, p.memory_policy.optimizer_stage, p.memory_policy.activation_checkpointing)
    mem = O.make_mem_model(rpeg0, p.suite, p.workload, p.hw, p.memory_policy)
    table, index = S.build_candidate_directory(rpeg0, p.suite, p.device_space, p.workload, cost, mem)
    arrays = [np.asarray([c[:6] for c in table[v]], np.int16).reshape(-1, 6) for v in rpeg0.vertices]
    return table, index, arrays


def _rows6(rows, nv):
    return [[int(x) for x in rows[v * 10:(v + 1) * 10]] for v in range(nv)]


@pytest.mark.parametrize("c", [1, 5])
def test_cxx_proposals_match_reference_vectors(c):
    with open(os.path.join(GOLDEN, "ref_sa.json")) as f:
        cases = json.load(f)["configs"][str(c)]["cases"]
    cfg, batch = seeded_batch(c, len(cases))
    p = cfg.problem
    sp = p.device_space
    rpeg0 = p.template(0, ())
    nv = len(rpeg0.vertices)
    _, _, arrays = _directory(p, rpeg0)
    port = CpuPort(p)
    for rec in cases:
        i = rec["i"]
        mg = rec["move_gen"]
        opt = OptimizerConfig(T_init=mg["T_init"], T_min=min(0.01, mg["T_init"]))
        params = sa_params(opt, 1, 1, [(0, 0)])
        _, plan_m, _ = batch.configuration(p, i)
        row = plan_row(rpeg0, ExecutionPlan(sigma={v: plan_m.sigma[u] for v, u in zip(rpeg0.vertices, plan_m.sigma)},
                                            pi={v: plan_m.pi[u] for v, u in zip(rpeg0.vertices, plan_m.pi)},
                                            mb={v: plan_m.mb[u] for v, u in zip(rpeg0.vertices, plan_m.mb)}))
        mass = np.zeros(abi.MAX_V)
        mass[:nv] = [float.fromhex(x) for x in rec["mass"]]
        out, draws, fb = port.sa_propose(params, arrays, 0, (42, c, i, 1), plan=row, mass=mass, T=mg["T"])
        assert [_rows6(r, nv) for r in out] == mg["plans"], i
        assert draws == mg["n_draws"] and fb == mg["fallback"], i
        out, draws, _ = port.sa_propose(params, arrays, 1, (42, c, i, 2), plan=row)
        assert ([_rows6(r, nv) for r in out] or [None])[0] == rec["pair"]["plan"], i
        assert draws == rec["pair"]["n_draws"], i
        draws, rows = 0, []
        for v in range(nv):
            lo = i % sp.R
            hi = min(sp.R, lo + 1 + (i // 3) % sp.R)
            out, draws, _ = port.sa_propose(params, arrays, 2, (42, c, i, 3), v=v, r_lo=lo, r_hi=hi, skip=draws)
            rows.append([int(x) for x in out[0]] if len(out) else None)
        assert rows == rec["sample"]["rows"], i
        assert draws == rec["sample"]["n_draws"], i


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_critical_mass_matches_restatement(c):
    n = 40
    cfg, batch = seeded_batch(c, n)
    p = cfg.problem
    got = CpuPort(p).eval(batch, want_mass=True)
    for i in range(n):
        rpeg, plan, wl = batch.configuration(p, i)
        r = O.evaluate_plan(rpeg, plan, p.device_space, p.suite, wl, p.hw, p.K_eval, p.memory_policy,
                            check_stale=False, want_trace=True)
        chain = S.critical_chain(r["nodes"], r["edges"], r["finish"])
        mass = S.critical_mass(chain, rpeg, r["start"], r["finish"])
        want = [mass[v] for v in rpeg.vertices]
        assert [x.hex() for x in got["mass"][i, :len(want)]] == [x.hex() for x in want], i
        assert not got["mass"][i, len(want):].any()


def _log_byte(entry):
    step, kind, nc, acc = entry
    b = (1 if kind == "pair" else 0) | nc << 1
    if acc is not None:
        b |= (2 if acc else 1) << 4
    return b


def test_groups_of_chains_that_step_in_turn_change_nothing():
    """SaRun deals the chains to groups whose steps interleave (so that a GPU evaluates one group while the host works
    on another): every chain draws from its own (seed, chain, step) streams, so any grouping gives the same run."""
    p = configs.config(1).problem
    opt = OptimizerConfig(T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=4)
    rpeg0 = p.template(0, ())
    _, _, arrays = _directory(p, rpeg0)
    n_tau = len(p.structures[0].tau_models)
    variants = [(0,) * n_tau, (1,) + (0,) * (n_tau - 1)]
    params = sa_params(opt, 10, 60, variants, 0, 1 if p.workload.gen_quantiles else 0, 42)
    one = CpuPort(p).sa_run(params, arrays, threads=4)
    assert ((one["log"] >> 6) & 1).sum() > 0, "no restart in the run"
    for groups in (2, 3, 7, 10, 16):
        got = CpuPort(p).sa_run(params, arrays, threads=4, groups=groups)
        for k in ("log", "cur_plan", "best_plan", "best_step", "best_feasible", "restarts", "n_eval", "dead"):
            assert np.array_equal(got[k], one[k]), (groups, k)
        for k in ("cur_score", "best_score"):
            assert np.array_equal(got[k].view(np.uint64), one[k].view(np.uint64)), (groups, k)


@pytest.mark.parametrize("c,n_chains,n_steps,kw", [
    (1, 6, 40, dict(T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=4)),
    (5, 4, 12, dict(T_init=0.05, T_min=0.05, T_warm=0.10, stag_window=10)),
    (2, 3, 25, dict(T_init=0.30, T_min=0.01, T_warm=0.05, stag_window=3, geometric_cooling=True)),
])
def test_chain_trajectories_match_restatement(c, n_chains, n_steps, kw):
    cfg = configs.config(c)
    p = cfg.problem
    opt = OptimizerConfig(**kw)
    n_tau = len(p.structures[0].tau_models)
    variants = [(0,) * n_tau, (1,) + (0,) * (n_tau - 1)]
    rpeg0 = p.template(0, ())
    _, _, arrays = _directory(p, rpeg0)
    split = 1 if p.workload.gen_quantiles else 0
    params = sa_params(opt, n_chains, n_steps, variants, 0, split, 42)
    got = CpuPort(p).sa_run(params, arrays, threads=4)
    sp = S.SaParams(K_x=opt.K_x, T_max=opt.T_max, T_init=opt.T_init, T_warm=opt.T_warm, T_min=opt.T_min,
                    K_elite=opt.K_elite, alpha_pair=opt.alpha_pair, stag_window=opt.stag_window,
                    score_eps=opt.score_eps, E_struct=opt.E_struct, geometric_cooling=opt.geometric_cooling, seed=42)
    assert sp.T_cool == opt.T_cool
    rpegs = [p.template(0, v) for v in variants]
    table, index, _ = _directory(p, rpegs[0])
    nv = len(rpeg0.vertices)
    for cid in range(n_chains):
        rpeg = rpegs[cid % len(variants)]
        tabs = ({v: table[v0] for v, v0 in zip(rpeg.vertices, rpegs[0].vertices)},
                {v: index[v0] for v, v0 in zip(rpeg.vertices, rpegs[0].vertices)})
        ev = S.oracle_evaluator(rpeg, p.device_space, p.suite, p.workload, p.hw, p.K_eval, p.memory_policy)
        ch = S.run_chains(lambda _c: rpeg, ExecutionPlan, Allocation, p.device_space, p.suite, p.workload,
                          lambda _c: ev, tabs, 1, n_steps, sp, first_chain=cid)[0]
        assert bool(got["dead"][cid]) == ch.dead, cid
        if ch.dead:
            continue
        want_log = np.zeros(n_steps, np.uint8)
        for e in ch.log:
            want_log[e[0]] = _log_byte(e)
        assert [int(x) & 0x3F for x in got["log"][cid]] == [int(x) for x in want_log], cid
        assert _rows6(got["cur_plan"][cid], nv) == _rows6(plan_row(rpeg, ch.cur.plan), nv), cid
        assert got["cur_score"][cid].hex() == float(ch.score).hex(), cid
        assert got["restarts"][cid] == ch.r and got["n_eval"][cid] == ch.n_eval, cid
        feas = ch.best_feasible is not None
        assert bool(got["best_feasible"][cid]) == feas, cid
        best = ch.best_feasible if feas else ch.best
        assert _rows6(got["best_plan"][cid], nv) == _rows6(plan_row(rpeg, best.plan), nv), cid
        assert got["best_score"][cid].hex() == float(ch.best_feasible_score if feas else ch.best_score).hex(), cid
        assert got["best_step"][cid] == (ch.best_feasible_step if feas else ch.best_step), cid


def test_cxx_optimize_matches_reference_optimize():
    """The shipped reference-style loop (SaSerial in rpeg_amd/csrc/rpeg_sa.h, here over the CPU evaluator)
    against the trajectory of the reference's own optimize() on the same generator
    (tests/golden/make_golden_optimize.py): same plans evaluated in the same order, same number of draws,
    same returned plan."""
    import zlib
    with open(os.path.join(GOLDEN, "ref_optimize.json")) as f:
        g = json.load(f)
    cfg, batch = seeded_batch(1, 8)
    p = cfg.problem
    rpeg0 = p.template(0, ())
    nv = len(rpeg0.vertices)
    _, _, arrays = _directory(p, rpeg0)
    for case in [c for c in g["cases"] if not c.get("families")]:
        port = CpuPort(with_transfer_policy(p, *case["transfer"]) if "transfer" in case else p)
        _, plan_m, _ = batch.configuration(p, case["plan"])
        row = plan_row(rpeg0, ExecutionPlan(sigma={v: plan_m.sigma[u] for v, u in zip(rpeg0.vertices, plan_m.sigma)},
                                            pi={v: plan_m.pi[u] for v, u in zip(rpeg0.vertices, plan_m.pi)},
                                            mb={v: plan_m.mb[u] for v, u in zip(rpeg0.vertices, plan_m.mb)}))
        opt = OptimizerConfig(K_x=6, T_max=50, E_max=case["E_max"], E_struct=case["E_struct"], T_init=case["T_init"],
                              T_warm=case["T_warm"], T_min=case["T_min"], stag_window=case["stag_window"])
        assert opt.T_cool.hex() == case["T_cool"]
        params = sa_params(opt, 1, 1, [(0, 0)], 0, 1, case["stream"][0])
        res = port.sa_optimize(params, arrays, row, case["E_max"], case["E_struct"], stream_key=case["stream"][1:],
                               log_cap=4096, threads=4)
        log = [_rows6(r, nv) for r in res["eval_log"]]
        assert log[:8] == case["first"]
        assert res["n_eval_log"] == case["n_eval"] == len(log)
        assert zlib.crc32(json.dumps(log, separators=(",", ":")).encode()) == case["eval_crc"]
        assert res["n_draws"] == case["n_draws"]
        assert _rows6(res["best_plan"], nv) == case["final"]


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_start_plan_host_logic_against_reference_vectors(c):
    """The start-plan constructors are host logic over a candidate directory.  Fed the directory of the
    Python restatement, the greedy plan and the cascade of the concurrent constructor (groups by depth,
    partition enumeration, ranking, demotion order) equal what the reference built and lowered; every
    partition with several allocations is pairwise disjoint and inside the device space."""
    from rpeg_amd.search import baselines as B
    with open(os.path.join(GOLDEN, "ref_baselines.json")) as f:
        g = json.load(f)["configs"][str(c)]
    p = configs.config(c).problem
    rpeg0 = p.template(0, ())
    table, _, _ = _directory(p, rpeg0)

    def rows(plan):
        return [[*plan.pi[v], plan.mb[v], *plan.sigma[v].origin, *plan.sigma[v].extent] for v in rpeg0.vertices]

    assert rows(B.build_valid_baseline_plan(rpeg0, p.device_space, p.suite, p.workload, None, table=table)) \
        == g["build_valid_baseline_plan"]["rows"]
    tried = g["build_concurrent_baseline_plan"]["tried"]
    cascade = B.concurrent_plan_cascade(rpeg0, p.device_space, table)
    assert [rows(pl) for pl, _, _ in cascade[:len(tried)]] == [t["rows"] for t in tried]

    sp = p.device_space
    for group in B._find_concurrent_groups(rpeg0):
        for part in B._enumerate_group_partitions(group, sp):
            assert len(part) == len(group)
            seen = set()
            for a in set(part):
                devs = {(r, n, d) for r in range(a.origin[0], a.origin[0] + a.extent[0])
                        for n in range(a.origin[1], a.origin[1] + a.extent[1])
                        for d in range(a.origin[2], a.origin[2] + a.extent[2])}
                assert all(r < sp.R and n < sp.N and d < sp.G for r, n, d in devs)
                assert not (devs & seen)
                seen |= devs


def test_cxx_optimize_over_structural_families_matches_reference_optimize():
    """SaSerial over the separate template's staleness variants and then the AC-share template's, on the CPU
    evaluator, against the reference's optimize() with structural_candidates {"separate", "ac_share"}: every
    evaluated (template, staleness, plan) in order -- including the random restarts that start the AC-share
    settings, which the reference validates with the memory model of its base configuration --, the number of
    draws, and the returned configuration (an AC-share one in the second and third case).  In the third case
    memory is tight and the two memory models disagree on the restarts: the run equals the reference's only
    with the base configuration's view, which the last lines check."""
    with open(os.path.join(GOLDEN, "ref_optimize.json")) as f:
        g = json.load(f)
    cases = [c for c in g["cases"] if c.get("families") and not c.get("max_throughput_loss")]   # no traces on this evaluator
    assert len(cases) == 4 and cases[3]["transfer"] == ["destination_only", "both_endpoints"]
    cases = cases[3:] + cases[:3]                 # the lines after the loop are about the tight-memory case
    for case in cases:
        p = family_problem(case)
        port = CpuPort(p)

        def directory_of(structure):
            return _directory(p, p.template(structure, ()))[2]

        families, row, opt = family_case_setup(p, case, directory_of)
        res = port.sa_optimize_families(families, case["base_tau"], row, case["E_max"], case["E_struct"],
                                        stream_key=case["stream"][1:], log_cap=4096, threads=4)
        check_family_case(p, case, families, res)
    families[1] = families[1][:4] + (None,)      # the template's own memory model for is_valid: another run
    res = port.sa_optimize_families(families, case["base_tau"], row, case["E_max"], case["E_struct"],
                                    stream_key=case["stream"][1:], log_cap=4096, threads=4)
    assert res["n_draws"] != case["n_draws"]


class _TickingClock:
    """A clock that advances by one second at every reading, as the one the deadline cases of
    tests/golden/make_golden_optimize.py put in perf_counter's place."""

    def __init__(self):
        self.reads = 0
        self.fn = abi.CLOCK_FN(self._read)

    def _read(self, _ctx):
        self.reads += 1
        return float(self.reads)

    def install(self, params, deadline):
        params.timed, params.deadline_s = 1, float(deadline)
        params.clock = C.cast(self.fn, C.c_void_p)


def flag_cases():
    with open(os.path.join(GOLDEN, "ref_optimize.json")) as f:
        return json.load(f)["flag_cases"]


def flag_config(case, **kw):
    return OptimizerConfig(K_x=6, T_max=50, E_max=case["E_max"], E_struct=case["E_struct"], T_init=case["T_init"],
                           T_warm=case["T_warm"], T_min=case["T_min"], stag_window=case["stag_window"],
                           fixed_mb=case.get("fixed_mb", False), uniform_vertex=case.get("uniform_vertex", False),
                           hard_oom=case.get("hard_oom", False), **kw)


def check_flag_case_scores(case, res):
    import zlib
    got = [float(x).hex() for x in res["eval_log_score"]]
    assert zlib.crc32(json.dumps(got).encode()) == case["eval_scores_crc"]


@pytest.mark.parametrize("k", range(8))
def test_cxx_optimize_ablations_and_deadlines_match_reference_optimize(k):
    """OptimizerConfig's ablation switches (fixed_mb, uniform_vertex, hard_oom; RPEG/search/optimizer.py:404-410,
    moves.py:182-188, 688, evaluate.py:392, 437) and its wall-clock deadline (optimizer.py:571-579, 703-720,
    848-865) in the shipped loop, against the reference's own optimize() run with the same switches on the same
    generator and -- for the deadlines -- the same ticking clock: same plans in the same order, same scores,
    same number of draws and of clock readings, same returned configuration."""
    import zlib
    case = flag_cases()[k]
    S.ABLATION_FIXED_MB = bool(case.get("fixed_mb"))
    try:
        clock = _TickingClock()
        if case.get("families"):
            p = family_problem(case)
            port = CpuPort(p)
            families, row, opt = family_case_setup(p, case, lambda s: _directory(p, p.template(s, ()))[2],
                                                   fixed_mb=case.get("fixed_mb", False), hard_oom=case.get("hard_oom", False),
                                                   uniform_vertex=case.get("uniform_vertex", False))
            if "deadline" in case:
                clock.install(families[0][0], case["deadline"])
            res = port.sa_optimize_families(families, case["base_tau"], row, case["E_max"], case["E_struct"],
                                            stream_key=case["stream"][1:], log_cap=4096, threads=4)
            check_family_case(p, case, families, res)
        else:
            cfg, batch = seeded_batch(1, 8)
            p = cfg.problem
            rpeg0 = p.template(0, ())
            nv = len(rpeg0.vertices)
            port = CpuPort(p)
            _, plan_m, _ = batch.configuration(p, case["plan"])
            row = plan_row(rpeg0, ExecutionPlan(sigma={v: plan_m.sigma[u] for v, u in zip(rpeg0.vertices, plan_m.sigma)},
                                                pi={v: plan_m.pi[u] for v, u in zip(rpeg0.vertices, plan_m.pi)},
                                                mb={v: plan_m.mb[u] for v, u in zip(rpeg0.vertices, plan_m.mb)}))
            opt = flag_config(case)
            assert opt.T_cool.hex() == case["T_cool"]
            params = sa_params(opt, 1, 1, [(0, 0)], 0, 1, case["stream"][0])
            if "deadline" in case:
                clock.install(params, case["deadline"])
            res = port.sa_optimize(params, _directory(p, rpeg0)[2], row, case["E_max"], case["E_struct"],
                                   stream_key=case["stream"][1:], log_cap=4096, threads=4)
            log = [_rows6(r, nv) for r in res["eval_log"]]
            assert log[:8] == case["first"]
            assert res["n_eval_log"] == case["n_eval"] == len(log)
            assert zlib.crc32(json.dumps(log, separators=(",", ":")).encode()) == case["eval_crc"]
            assert res["n_draws"] == case["n_draws"]
            assert _rows6(res["best_plan"], nv) == case["final"]
    finally:
        S.ABLATION_FIXED_MB = False
    check_flag_case_scores(case, res)
    assert clock.reads == case["clock_reads"]
    # the run ended on its deadline exactly when the deadline, not the budget, is what stopped the reference
    assert res["timed_out"] == ("deadline" in case and case["n_eval"] < case["E_max"])


def test_a_deadline_run_is_a_prefix_of_the_budget_run():
    """With one structural setting the wall clock only ends the search: what a run under a deadline evaluates is
    the beginning of what the same run evaluates under its budgets alone, whatever the deadline; and its result is
    the best of that beginning."""
    cfg, batch = seeded_batch(1, 8)
    p = cfg.problem
    rpeg0 = p.template(0, ())
    port = CpuPort(p)
    _, plan_m, _ = batch.configuration(p, 0)
    row = plan_row(rpeg0, ExecutionPlan(sigma={v: plan_m.sigma[u] for v, u in zip(rpeg0.vertices, plan_m.sigma)},
                                        pi={v: plan_m.pi[u] for v, u in zip(rpeg0.vertices, plan_m.pi)},
                                        mb={v: plan_m.mb[u] for v, u in zip(rpeg0.vertices, plan_m.mb)}))
    arrays = _directory(p, rpeg0)[2]
    opt = OptimizerConfig(K_x=6, T_max=50, E_max=400, E_struct=10 ** 6, T_init=0.05, T_warm=0.10, T_min=0.05, stag_window=4)

    def run(deadline=None):
        params = sa_params(opt, 1, 1, [(0, 0)], 0, 1, 42)
        clock = _TickingClock()
        if deadline is not None:
            clock.install(params, deadline)
        res = port.sa_optimize(params, arrays, row, opt.E_max, opt.E_struct, stream_key=(78, 9, 0), log_cap=4096, threads=4)
        return res, clock
    full, clock = run()
    assert clock.reads == 0 and not full["timed_out"] and full["n_eval_log"] >= opt.E_max
    seen = []
    for deadline in (0.0, 3.0, 40.0, 41.0, 97.0, 10 ** 6):
        res, clock = run(deadline)
        n = res["n_eval_log"]
        assert np.array_equal(res["eval_log"], full["eval_log"][:n])
        assert np.array_equal(res["eval_log_score"].view(np.uint64), full["eval_log_score"][:n].view(np.uint64))
        assert res["timed_out"] == (deadline < 10 ** 6) and (res["timed_out"] or n == full["n_eval_log"])
        # the clock is read before every iteration and after every evaluated batch: the run ends on the reading that
        # reaches the deadline
        assert clock.reads == (deadline if 1.0 <= deadline < 10 ** 6 else clock.reads)
        feasible = res["eval_log_feasible"]
        if feasible.any():
            assert res["best_feasible"] and res["best_score"] == res["eval_log_score"][feasible].max()
        seen.append(n)
    assert seen == sorted(seen) and seen[0] == 1 and seen[1] < seen[3] < seen[4] < seen[5]
