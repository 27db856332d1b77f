"""GPU parity tests: every call goes through the C ABI (librpeg_eval.so) on a real MI355X.

Bars: feasibility masks, ranking and best plan bit-exact; makespan, peak and score bit-exact
(stricter than the 1e-12 relative the workload description allows)."""

import math

import numpy as np
import pytest

from oracle import rpeg_oracle as oracle
from oracle.cpu_port import CpuPort
from rpeg_amd import configs
from rpeg_amd.engine import abi
from rpeg_amd.engine.problem import PlanBatch
from tests.helpers import load_golden, seeded_batch

pytestmark = pytest.mark.gpu

_engines = {}


def engine(c):
    from rpeg_amd.engine.runtime import Engine
    if c not in _engines:
        _engines[c] = Engine(configs.config(c).problem)
    return _engines[c]


def same_bits(a, b):
    return np.array_equal(np.asarray(a, np.float64).view(np.uint64), np.asarray(b, np.float64).view(np.uint64))


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_reference_vectors(c):
    gold = load_golden(c)
    cfg, batch = seeded_batch(c, gold["n"])
    out = engine(c).eval(batch, gate_stale=False)
    for i, want in enumerate(gold["plans"]):
        assert float(out["makespan"][i]).hex() == want["makespan"], i
        assert float(out["peak"][i]).hex() == want["peak"], i
        assert float(out["score"][i]).hex() == want["score"], i
        assert bool(out["mask"][i] & abi.MASK_MEM_OK) == want["feasible"], i
        assert out["mask"][i] & abi.MASK_VALID and not out["mask"][i] & abi.MASK_ERROR


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_python_oracle_beyond_fixtures(c):
    cfg, batch = seeded_batch(c, 40, start=200_000)
    p = cfg.problem
    out = engine(c).eval(batch, gate_stale=True)
    for i in range(40):
        rpeg, plan, wl = batch.configuration(p, i)
        want = oracle.evaluate_plan(rpeg, plan, p.device_space, p.suite, wl, p.hw, p.K_eval, p.memory_policy,
                                    check_stale=True)
        assert out["makespan"][i] == want["makespan"] and out["peak"][i] == want["peak"], i
        assert out["score"][i] == want["score"], i
        assert bool(out["mask"][i] & abi.MASK_STALE_OK) == want["stale_ok"], i
        assert bool(out["mask"][i] & abi.MASK_MEM_OK) == (not want["peak"] > want["cap"]), i


@pytest.mark.parametrize("c,n", [(1, 4096), (2, 65536), (3, 262144), (4, 1048576)])
def test_full_candidate_sets_rank_and_argmax(c, n):
    """Whole seeded sets at the sizes the workload description names (4,096 / 65,536 / 262,144 / 1,048,576
    plans): masks, every score, the ranking and the best plan equal the host build of the same arithmetic,
    which the CPU suite ties to the reference vectors."""
    cfg, batch = seeded_batch(c, n)
    out = engine(c).eval(batch, gate_stale=True)
    ref = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE, threads=16)
    assert np.array_equal(out["mask"], ref["mask"])
    assert same_bits(out["makespan"], ref["makespan"])
    assert same_bits(out["peak"], ref["peak"])
    assert same_bits(out["score"], ref["score"])
    assert np.array_equal(np.argsort(-out["score"], kind="stable"), np.argsort(-ref["score"], kind="stable"))
    assert int(np.argmax(out["score"])) == int(np.argmax(ref["score"]))
    # size-independent properties
    assert np.all(out["makespan"] > 0) and np.all(out["peak"] > 0)
    feasible = (out["mask"] & abi.MASK_MEM_OK) != 0
    stale_ok = (out["mask"] & abi.MASK_STALE_OK) != 0
    raw = cfg.problem.K_eval * cfg.problem.workload.B * cfg.problem.workload.K * \
        (cfg.problem.workload.S + cfg.problem.workload.T) / out["makespan"]
    assert same_bits(out["score"][feasible & stale_ok], raw[feasible & stale_ok])
    assert np.all(out["score"][~stale_ok] == 0.0)
    assert np.all(out["score"][~feasible & stale_ok] < raw[~feasible & stale_ok])


def test_config4_is_mostly_infeasible():
    cfg, batch = seeded_batch(4, 262144)
    out = engine(4).eval(batch)
    frac = 1.0 - np.mean((out["mask"] & abi.MASK_MEM_OK) != 0)
    assert 0.6 < frac < 0.85


def test_permutation_duplicates_and_stride():
    from rpeg_amd.engine.runtime import DeviceBatch
    import torch
    cfg, batch = seeded_batch(2, 5000)
    eng = engine(2)
    base = eng.eval(batch)
    perm = np.random.default_rng(0).permutation(5000)
    shuffled = eng.eval(batch.take(perm))
    for k in ("makespan", "peak", "score", "mask"):
        assert np.array_equal(shuffled[k], base[k][perm]), k
    dup = eng.eval(batch.take(np.repeat(np.arange(100), 7)))
    assert same_bits(dup["score"], np.repeat(base["score"][:100], 7))
    # stride larger than n: evaluate the first 1000 plans of the 5000-plan tensors
    db = DeviceBatch(batch)
    out = eng.eval_device(db, n=1000)
    torch.cuda.synchronize()
    assert same_bits(out["score"].cpu().numpy(), base["score"][:1000])


def test_empty_single_and_invalid():
    cfg, batch = seeded_batch(2, 8)
    eng = engine(2)
    assert eng.eval(batch.slice(0, 0))["score"].shape == (0,)
    one = eng.eval(batch.slice(3, 4))
    assert same_bits(one["score"], eng.eval(batch)["score"][3:4])
    batch.vert[0, 1] = 3
    batch.vert[3, 2] = 5
    batch.head[1, 3] = 7
    batch.vert[7, 4] = 99
    out = eng.eval(batch)
    assert list(out["mask"][1:5]) == [0, 0, 0, 0] and np.all(np.isnan(out["score"][1:5]))
    assert out["mask"][0] & abi.MASK_VALID and out["mask"][5] & abi.MASK_VALID
    allbad = PlanBatch.empty(3)
    assert list(eng.eval(allbad)["mask"]) == [0, 0, 0]


def test_empty_single_and_invalid_device_tensors_and_argument_errors():
    """The same edge cases through rpeg_eval_batch on device tensors (a batch of 8 plans and one of 3,000:
    one plan per wavefront and the main kernel), and the argument checks of rpeg_eval_host."""
    import ctypes as C
    from rpeg_amd.engine.runtime import EngineError
    eng = engine(2)
    for n in (8, 3000, 40000):
        cfg, batch = seeded_batch(2, n)
        batch.vert[0, 1] = 3
        batch.vert[3, 2] = 5
        batch.head[1, 3] = 7
        batch.vert[7, 4] = 99
        out = eng.eval_resident(batch)
        host = eng.eval(batch)
        assert list(out["mask"][1:5]) == [0, 0, 0, 0] and np.all(np.isnan(out["score"][1:5]))
        assert np.array_equal(out["mask"], host["mask"]) and same_bits(out["score"], host["score"])
        assert same_bits(out["makespan"], host["makespan"]) and same_bits(out["peak"], host["peak"])
    assert list(eng.eval_resident(PlanBatch.empty(3))["mask"]) == [0, 0, 0]
    cfg, batch = seeded_batch(2, 16)
    vert = np.ascontiguousarray(batch.vert)
    head = np.ascontiguousarray(batch.head)
    score = np.empty(16)
    bad_stride = abi.PlanSoaT(vert.ctypes.data, head.ctypes.data, 8)        # stride below n
    assert eng.lib.rpeg_eval_host(eng._h, 16, C.addressof(bad_stride), 0, None, None, score.ctypes.data, None, None, None) < 0
    assert b"bad plan tensors" in eng.lib.rpeg_last_error(eng._h)
    no_vert = abi.PlanSoaT(None, head.ctypes.data, 16)
    assert eng.lib.rpeg_eval_host(eng._h, 16, C.addressof(no_vert), 0, None, None, score.ctypes.data, None, None, None) < 0
    assert eng.lib.rpeg_eval_host(eng._h, 16, None, 0, None, None, score.ctypes.data, None, None, None) < 0
    ok = abi.PlanSoaT(vert.ctypes.data, head.ctypes.data, 16)               # only the score is asked for
    assert eng.lib.rpeg_eval_host(eng._h, 16, C.addressof(ok), 0, None, None, score.ctypes.data, None, None, None) == 0
    assert same_bits(score, eng.eval(batch, gate_stale=False)["score"])


def test_plans_that_outgrow_the_learned_ready_list_are_redone():
    """The main kernel sizes its ready lists by the longest list it has seen.  An engine that has only seen
    chain-like graphs (every vertex on vertex 0's allocation and strategy) then meets the seeded set: the plans
    whose lists outgrow the short capacity are flagged and redone with the full one."""
    from rpeg_amd.engine.runtime import Engine
    n = 40000                                       # above the one-plan-per-wavefront range
    cfg, batch = seeded_batch(2, n)
    chains = PlanBatch(batch.vert.copy(), batch.head.copy())
    for v in range(1, 4):
        chains.vert[v * 10:(v + 1) * 10, :] = chains.vert[0:10, :]
    port = CpuPort(cfg.problem)
    eng = Engine(cfg.problem)
    lds = []
    for b in (chains, batch, chains, batch):
        out = eng.eval_resident(b)
        ref = port.eval(b, flags=abi.GATE_STALE, threads=16)
        assert np.array_equal(out["mask"], ref["mask"])
        assert same_bits(out["makespan"], ref["makespan"]) and same_bits(out["score"], ref["score"])
        assert eng.stats()["state_lanes"] == 0
        lds.append(eng.stats()["lds_bytes"])
    # the second call ran with the capacity learned from the chains (the area of the ready lists also holds the ring of
    # the rank pass, which keeps it from shrinking below 32 rows: the two short capacities may need the same LDS)
    assert lds[1] < lds[0] and lds[1] <= lds[3]
    assert (ref["mask"] & abi.MASK_VALID).sum() > n // 2
    eng.close()


def test_plans_beyond_a_short_ready_list_are_redone_and_nothing_is_left_behind():
    """With the main kernel's ready list lowered to 8 entries thousands of plans of config 2 outgrow it.  They are
    redone by the launch that ends the call and come back with the host build's bits; afterwards, with the list
    back at 32 entries, the same engine evaluates the set exactly again -- in the launch that learns the short
    capacity and in the next ones, whose fix-up launches must find no flag or count left over."""
    from rpeg_amd.engine.runtime import Engine
    n = 40000
    cfg, batch = seeded_batch(2, n)
    ref = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE, threads=16)
    assert ref["max_ready"] > 8
    eng = Engine(cfg.problem)
    eng.set_quad_share(0)      # (every class in the main kernel or, the largest graphs, one plan per wavefront)
    for cap in (8, 32, 8, 16):
        eng.set_ready_cap(cap)
        for _ in range(2):
            out = eng.eval_resident(batch)
            assert not np.any(out["mask"] & abi.MASK_LIMIT)
            assert np.array_equal(out["mask"], ref["mask"]), cap
            assert same_bits(out["score"], ref["score"]) and same_bits(out["makespan"], ref["makespan"]), cap
    with pytest.raises(Exception, match="8, 16, 24 or 32"):
        eng.set_ready_cap(12)
    eng.close()


def test_the_drop_in_names_an_engine_limit():
    """evaluate_batch raises EngineLimitError for a mask with RPEG_MASK_LIMIT (no evaluation path sets it for a plan the
    reference evaluates; the bit stays in the ABI for limits a later kernel may have) instead of a division by zero."""
    from rpeg_amd.search import evaluate as ev
    cfg, batch = seeded_batch(2, 4)

    class Limited:
        def eval(self, b, gate_stale=True):
            m = np.full(b.n, abi.MASK_VALID | abi.MASK_ERROR | abi.MASK_LIMIT, np.uint8)
            nan = np.full(b.n, np.nan)
            return dict(mask=m, score=nan, makespan=nan, peak=nan)
    p = cfg.problem
    rpeg, plan, wl = batch.configuration(p, 0)
    real = ev._engine_for
    ev._engine_for = lambda *a, **k: (Limited(), real(*a, **k)[1])
    try:
        with pytest.raises(ev.EngineLimitError):
            ev.evaluate_batch([ev.Configuration(rpeg, plan, p.device_space)], p.suite, wl, p.hw, p.K_eval, p.memory_policy)
    finally:
        ev._engine_for = real


def test_mixed_structures_config3():
    cfg, batch = seeded_batch(3, 2000, start=500_000)
    out = engine(3).eval(batch)
    ref = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE, threads=16)
    assert set(np.unique(batch.head[0])) == {0, 1}
    assert same_bits(out["score"], ref["score"]) and np.array_equal(out["mask"], ref["mask"])


@pytest.mark.parametrize("c", [1, 3, 4])
def test_op_time_batch_is_the_candidate_directory_arithmetic(c):
    from rpeg_amd.search.candidates import strategy_space
    p = configs.config(c).problem
    eng = engine(c)
    rpeg = p.template(0)
    sp = p.device_space
    cost = oracle.CostModel(p.hw, p.suite, p.workload)
    mm = oracle.make_mem_model(rpeg, p.suite, p.workload, p.hw, p.memory_policy)
    from rpeg_amd.core.types import Allocation
    for vi, v in enumerate(rpeg.vertices):
        space = strategy_space(p.suite.specs[v.kind.model].L, p.workload.B, sp.R, sp.N, sp.G)
        pick = np.linspace(0, len(space) - 1, 60).astype(int)
        strat = np.zeros((7, len(pick)), np.int16)
        for j, s in enumerate(pick):
            dp, pp, tp, er, en, eg = space[s]
            mb = 1 if pp == 1 else max(m for m in (1, 2, 4, 8, 16, 32, 64) if (p.workload.B // dp) % m == 0)
            strat[:, j] = (dp, pp, tp, mb, er, en, eg)
        t, pk = eng.op_time(0, vi, strat)
        for j in range(len(pick)):
            dp, pp, tp, mb, er, en, eg = (int(x) for x in strat[:, j])
            node = oracle.XNode("_approx", oracle.OP, (Allocation((0, 0, 0), (er, en, eg)),), tpl=v, k=0,
                                model=v.kind.model, pi=(dp, pp, tp), mb=mb)
            assert t[j] == cost.time(node), (v.id, j)
            assert pk[j] == float(mm.peak_bytes(node)), (v.id, j)


@pytest.mark.parametrize("c", [1, 2, 4])
def test_trace_equals_oracle_schedule(c):
    cfg, batch = seeded_batch(c, 12)
    p = cfg.problem
    eng = engine(c)
    for i in range(12):
        rpeg, plan, wl = batch.configuration(p, i)
        nodes, edges = oracle.lower(rpeg, plan, p.suite, p.K_eval, wl)
        cost = oracle.CostModel(p.hw, p.suite, wl)
        start, finish, _ = oracle.schedule(nodes, edges, cost, p.device_space)
        tr = eng.trace(batch, i)
        assert [start[n.id] for n in nodes] == list(tr["start"])
        assert [finish[n.id] for n in nodes] == list(tr["finish"])
        idx = {n.id: j for j, n in enumerate(nodes)}
        assert [(idx[a.id], idx[b.id]) for a, b in edges] == [tuple(e) for e in tr["edges"]]


def test_device_exp_equals_host_libm():
    rng = np.random.default_rng(11)
    x = np.concatenate([-28.0 * rng.random(1_000_000), -np.logspace(-12, 1.5, 5000), [0.0, -40.0, -64.0]])
    y = engine(4).device_exp(x)
    want = np.array([math.exp(v) for v in x.tolist()])
    assert same_bits(y, want)


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_trace_utilization_and_active_devices_equal_reference(c):
    """Trace.utilization() and Trace.n_active() of the drop-in evaluate(): the engine's start/finish times and
    reserved allocations, folded on the host as the reference folds them, against the values the reference
    computed from its own traces (tests/golden/ref_cfg*.json)."""
    from rpeg_amd.search.evaluate import Configuration, evaluate
    gold = load_golden(c)
    cfg, batch = seeded_batch(c, gold["n"])
    p = cfg.problem
    for i in range(0, gold["n"], 16):
        rpeg, plan, wl = batch.configuration(p, i)
        score, trace, lowered = evaluate(Configuration(rpeg, plan, p.device_space), p.suite, wl, p.hw, p.K_eval,
                                         p.memory_policy)
        want = gold["plans"][i]
        assert float(trace.utilization()).hex() == want["utilization"], i
        assert trace.n_active() == want["n_active"], i
        assert trace.makespan().hex() == want["makespan"], i
    # the same two metrics folded by the library (rpeg_eval_trace_metrics), every plan of the vectors
    eng = engine(c)
    for i in range(gold["n"]):
        util, act = eng.trace_metrics(batch, i)
        assert float(util).hex() == gold["plans"][i]["utilization"] and act == gold["plans"][i]["n_active"], i


def test_drop_in_calls():
    from rpeg_amd.search.evaluate import Configuration, _eval_worker, evaluate, evaluate_batch, evaluate_cached
    from rpeg_amd.search.cache import EvalCache
    cfg, batch = seeded_batch(1, 6)
    p = cfg.problem
    cache = EvalCache()
    cfgs = []
    for i in range(6):
        rpeg, plan, wl = batch.configuration(p, i)
        want = oracle.evaluate_plan(rpeg, plan, p.device_space, p.suite, wl, p.hw, p.K_eval, p.memory_policy,
                                    check_stale=True, want_trace=True)
        conf = Configuration(rpeg, plan, p.device_space)
        score, trace, lowered = evaluate(conf, p.suite, wl, p.hw, p.K_eval)
        assert score == want["raw"] and trace.makespan() == want["makespan"]
        assert [n.id for n in lowered.nodes] == [n.id for n in want["nodes"]]
        assert {n.id: t for n, t in trace.finish.items()} == want["finish"]
        s2, tr2, feasible, miss = evaluate_cached(conf, cache, p.suite, wl, p.hw, p.K_eval)
        assert miss and s2 == want["score"] and feasible == want["feasible"]
        s3, _, _, miss2 = evaluate_cached(conf, cache, p.suite, wl, p.hw, p.K_eval)
        assert not miss2 and s3 == s2
        worker = oracle.evaluate_plan(rpeg, plan, p.device_space, p.suite, wl, p.hw, p.K_eval, p.memory_policy,
                                      check_stale=False)
        s4, _, f4 = _eval_worker((conf, p.suite, wl, p.hw, p.K_eval))
        assert s4 == worker["score"] and f4 == worker["feasible"]
        if wl == batch.configuration(p, 0)[2]:
            cfgs.append((conf, want["score"]))
    wl0 = batch.configuration(p, 0)[2]
    res = evaluate_batch([c for c, _ in cfgs], p.suite, wl0, p.hw, p.K_eval)
    assert list(res.score) == [s for _, s in cfgs]
    bad = Configuration(cfgs[0][0].rpeg, cfgs[0][0].plan, p.device_space, intra_stage_fusion=True)
    with pytest.raises(NotImplementedError):
        evaluate(bad, p.suite, wl0, p.hw, p.K_eval)


@pytest.mark.parametrize("c,n", [(1, 2048), (2, 8192), (5, 1024)])
def test_every_state_layout_gives_the_same_bits(c, n):
    """Scheduler state in the HBM workspace (64 plans per wavefront) or in LDS (8/16/32/64 plans per
    wavefront), one plan per wavefront, four lanes per plan, and the per-batch automatic choice: identical outputs."""
    from rpeg_amd.engine.runtime import Engine, EngineError
    cfg, batch = seeded_batch(c, n)
    eng = Engine(cfg.problem)
    ref = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE, threads=16)
    seen = set()
    for lanes in (0, 1, 4, 8, 16, 32, 64, -1):
        eng.set_state_lanes(lanes)
        try:
            out = eng.eval(batch, gate_stale=True)
        except EngineError as ex:
            assert lanes > 1 and "does not fit in LDS" in str(ex)   # the largest class is too big for that many plans
            continue
        seen.add(eng.stats()["state_lanes"])
        assert (eng.stats()["quad_tasks"] > 0) == (lanes == 4)
        assert np.array_equal(out["mask"], ref["mask"]), lanes
        assert same_bits(out["makespan"], ref["makespan"]) and same_bits(out["score"], ref["score"]), lanes
        assert same_bits(out["peak"], ref["peak"]), lanes
    assert 0 in seen and 1 in seen and 8 in seen
    with pytest.raises(EngineError):
        eng.set_state_lanes(12)


@pytest.mark.parametrize("c,n", [(1, 1500), (2, 3000), (2, 20000), (3, 600), (4, 5000)])
def test_host_and_device_entry_points_agree(c, n):
    """rpeg_eval_host (plans and results in host memory; one plan per wavefront for small batches, staged
    through device memory for larger ones and for classes too large for that kernel), rpeg_eval_batch and
    rpeg_eval_batch_mass on device tensors: identical outputs, equal to the host build."""
    cfg, batch = seeded_batch(c, n)
    eng = engine(c)
    ref = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE, threads=16, want_mass=True)
    for out in (eng.eval(batch, gate_stale=True, mass=True), eng.eval_mass_device(batch, gate_stale=True),
                eng.eval_resident(batch, gate_stale=True)):
        assert np.array_equal(out["mask"], ref["mask"])
        for k in ("makespan", "peak", "score"):
            assert same_bits(out[k], ref[k]), k
        if "mass" in out:
            assert same_bits(out["mass"], ref["mass"])


def test_dense_classes_move_to_four_lanes_per_plan_once_measured():
    """A batch that fills the chip in one round: the first call runs every class in the main kernel, which records how
    long the slowest wavefront of each class took; from the next call on the classes that end last there run four
    lanes per plan beside it.  Outputs equal the host build's bit for bit in every call, also with the share at 0."""
    from rpeg_amd.engine.runtime import Engine
    cfg, batch = seeded_batch(2, 65536)
    ref = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE, threads=16, want_mass=True)
    eng = Engine(cfg.problem)
    quad = []
    for call in range(4):
        if call == 3:
            eng.set_quad_share(0)
        out = eng.eval(batch, gate_stale=True, mass=(call == 2))
        quad.append(eng.stats()["quad_tasks"])
        assert np.array_equal(out["mask"], ref["mask"]), call
        for k in ("makespan", "peak", "score") + (("mass",) if call == 2 else ()):
            assert same_bits(out[k], ref[k]), (call, k)
    assert quad[0] == 0 and quad[1] > 0 and quad[2] > 0 and quad[3] == 0, quad


def test_the_fitted_figures_of_the_split_move_plans_between_kernels_and_no_bit():
    """rpeg_engine_set_split_model: with the single-plan kernel made to look free, or the four-lanes-per-plan kernel,
    or both dear, other classes change kernels (the task counts say so); every call equals the host build."""
    from rpeg_amd.engine.runtime import Engine, EngineError
    cfg, batch = seeded_batch(2, 65536)
    ref = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE, threads=16)
    layouts = []
    for model in ([40.0, 2.2, 40.0, 1.6, 0.45, 0.65, 1.15, 0.97, 0.98],    # the defaults
                  [1.0, 0.1, 40.0, 1.6, 0.45, 1.0, 1.15, 0.97, 0.98],      # a plan costs k_plan next to nothing
                  [40.0, 2.2, 1.0, 0.1, 0.0, 0.65, 1.0, 0.97, 0.98],       # a wavefront of k_quad costs next to nothing
                  [400.0, 20.0, 4000.0, 20.0, 5.0, 0.1, 2.0, 0.5, 0.5]):   # both dear
        eng = Engine(cfg.problem)
        eng.set_split_model(model)
        try:
            for call in range(3):
                out = eng.eval(batch, gate_stale=True)
                assert np.array_equal(out["mask"], ref["mask"]), (model, call)
                for k in ("makespan", "peak", "score"):
                    assert same_bits(out[k], ref[k]), (model, call, k)
            st = eng.stats()
            layouts.append((st["single_plan_tasks"], st["quad_tasks"]))
        finally:
            eng.close()
    assert len(set(layouts)) >= 2, layouts
    assert layouts[1][0] >= layouts[0][0] and layouts[2][1] >= layouts[0][1] and layouts[3][1] == 0, layouts
    eng = Engine(cfg.problem)
    with pytest.raises(EngineError):
        eng.set_split_model([1.0] * 8)
    with pytest.raises(EngineError):
        eng.set_split_model([-1.0] + [1.0] * 8)
    eng.close()


@pytest.mark.parametrize("c,n", [(2, 65536), (4, 200000), (3, 50000)])
def test_the_stream_that_carries_the_layout_changes_no_bit(c, n):
    """rpeg_engine_set_side_layout: cost-model launch, layout and main kernel on the side stream (the default) or on
    the caller's; cold calls (classes lowered, several rounds) and warm ones; two engines that step in turn on two
    threads, of which the one that finds the side streams taken stays on its own; a batch that no plan of is valid.
    Every call equals the host build."""
    import threading
    from rpeg_amd.engine.runtime import Engine
    cfg, batch = seeded_batch(c, n)
    ref = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE, threads=16)

    def check(out, what):
        assert np.array_equal(out["mask"], ref["mask"]), what
        for k in ("makespan", "peak", "score"):
            assert same_bits(out[k], ref[k]), (what, k)

    for on in (True, False):
        eng = Engine(cfg.problem)
        eng.set_side_layout(on)
        try:
            for call in range(3):
                check(eng.eval(batch, gate_stale=True), (on, call))
            bad = batch.slice(0, 30000)
            bad.vert[0, :] = 0   # dp = 0 in every plan: the gate rejects the whole batch
            out = eng.eval(bad, gate_stale=True)
            assert not out["mask"].any() and np.all(np.isnan(out["score"]))
            check(eng.eval(batch, gate_stale=True), (on, "after a batch without a valid plan"))
        finally:
            eng.close()
    engines = [Engine(cfg.problem) for _ in range(2)]
    errors = []

    def work(eng, who):
        try:
            for call in range(4):
                check(eng.eval(batch, gate_stale=True), ("two engines", who, call))
        except Exception as exc:   # noqa: BLE001 - handed to the main thread
            errors.append(exc)

    try:
        threads = [threading.Thread(target=work, args=(e, k)) for k, e in enumerate(engines)]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        assert not errors, errors
    finally:
        for e in engines:
            e.close()


@pytest.mark.parametrize("c,n,what", [(3, 65536, "single_plan_tasks"), (5, 40000, "quad_tasks"), (2, 131072, "quad_tasks"),
                                      (1, 20000, "single_plan_tasks"), (3, 32768, "single_plan_tasks"), (2, 20000, "single_plan_tasks")])
def test_the_measured_split_changes_where_classes_run_and_not_one_bit(c, n, what):
    """Other batches whose layout the engine changes once it has measured its classes -- more than one round of
    wavefronts (the longest classes leave the main kernel for one plan per wavefront, fewer main-kernel wavefronts per
    compute unit), other graphs for four lanes per plan, a single round of wavefronts whose longest classes leave for
    one plan per wavefront --: every call of a fresh engine equals the host build."""
    from rpeg_amd.engine.runtime import Engine
    cfg, batch = seeded_batch(c, n)
    ref = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE, threads=16)
    eng = Engine(cfg.problem)
    seen = []
    for call in range(4):
        out = eng.eval(batch, gate_stale=True)
        seen.append(eng.stats()[what])
        assert np.array_equal(out["mask"], ref["mask"]), call
        for k in ("makespan", "peak", "score"):
            assert same_bits(out[k], ref[k]), (call, k)
    assert seen[-1] != seen[0], seen


def test_small_device_batches_skip_the_layout_and_go_the_long_way_for_new_classes():
    """A small batch of device tensors whose classes the engine knows is two launches and one wait (every plan finds
    its class through the table on the device, no layout on the host); plans of classes not lowered yet send the call
    the long way, which lowers them and evaluates the batch again.  With and without the critical-chain masses, every
    call equals the host build."""
    from rpeg_amd.engine.runtime import Engine
    cfg, a = seeded_batch(2, 1500)
    cfg, b = seeded_batch(2, 1500, start=40000)
    port = CpuPort(cfg.problem)
    eng = Engine(cfg.problem)
    lowered = []
    for call, batch in enumerate((a, a, b, b, a)):
        ref = port.eval(batch, flags=abi.GATE_STALE, threads=16, want_mass=True)
        out = eng.eval_mass_device(batch, gate_stale=True) if call % 2 else eng.eval_resident(batch, gate_stale=True)
        st = eng.stats()
        lowered.append(st["classes_lowered"])
        assert st["state_lanes"] == 1 and st["wave_tasks"] <= batch.n
        out = {k: (v.cpu().numpy() if hasattr(v, "cpu") else v) for k, v in out.items()}
        assert np.array_equal(out["mask"], ref["mask"]), call
        for k in ("makespan", "peak", "score") + (("mass",) if "mass" in out else ()):
            assert same_bits(out[k], ref[k]), (call, k)
    assert lowered[0] > 0 and lowered[1] == 0 and lowered[2] > 0 and lowered[3] == 0 and lowered[4] == 0, lowered


def test_small_batches_pick_the_latency_layout():
    cfg, batch = seeded_batch(2, 512)
    eng = engine(2)
    eng.set_state_lanes(-1)
    eng.eval(batch)
    assert eng.stats()["state_lanes"] > 0
    cfg, batch = seeded_batch(2, 65536)
    eng.eval(batch)
    assert eng.stats()["state_lanes"] == 0


@pytest.mark.parametrize("c", [1, 2, 4])
def test_execution_schedule_artifact_equals_reference(c):
    """evaluate()'s trace is filled in dispatch order, so the schedule section of a plan artifact
    (ir/serialize.py:244-274) lists the nodes as the reference does, with the same times."""
    import json, os, zlib
    from rpeg_amd.ir import serialize as ser
    from rpeg_amd.search.evaluate import Configuration, evaluate
    from tests.helpers import GOLDEN
    with open(os.path.join(GOLDEN, "ref_plans.json")) as f:
        recs = json.load(f)[str(c)]
    cfg, batch = seeded_batch(c, 3)
    p = cfg.problem
    for rec in recs:
        rpeg, plan, wl = batch.configuration(p, rec["i"])
        config = Configuration(rpeg, plan, p.device_space)
        score, trace, lowered = evaluate(config, p.suite, wl, p.hw, p.K_eval, p.memory_policy)
        got = ser.execution_schedule_to_dict(trace, horizon=p.K_eval)
        want = rec["schedule"]
        assert got["policy"] == want["policy"] and got["horizon"] == want["horizon"]
        assert got["predicted_makespan_s"].hex() == want["makespan"] and len(got["nodes"]) == want["n"]
        assert zlib.crc32(",".join(n["node_id"] for n in got["nodes"]).encode()) == want["order_crc"]
        assert [[n["node_id"], n["dispatch_index"], n["predicted_start_s"].hex(), n["predicted_finish_s"].hex()]
                for n in got["nodes"][:6]] == want["head"]


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_is_valid_drop_in_equals_restatement(c):
    """is_valid (RPEG/search/evaluate.py:143-232) through the engine against its restatement on the oracle's
    passes (integer rules, stale-layout rule, memory fit of the K_eval = 1 lowering): seeded plans of every
    structure and staleness of the configuration as they are, then broken one rule at a time; under the
    template's own memory model and under one whose trainable set is another template's (what optimize()
    passes for AC-share plans)."""
    from oracle import rpeg_oracle as O
    from rpeg_amd.core.types import Allocation, Model
    from rpeg_amd.ir.plan import ExecutionPlan
    from rpeg_amd.model.memory import NodeMemoryModel
    from rpeg_amd.search.evaluate import Configuration, is_valid
    cfg, batch = seeded_batch(c, 40)
    p = cfg.problem
    pol = p.memory_policy

    def restated(rpeg, plan, wl, trainable):
        if not O.plan_structurally_valid(rpeg, plan, p.device_space, p.suite, wl):
            return False
        if not O.stale_publication_layout_valid(rpeg, plan):
            return False
        nodes, _ = O.lower(rpeg, plan, p.suite, 1, wl)
        mm = O.MemModel(p.hw, p.suite, wl, trainable, eps_rt=pol.runtime_overhead_fraction,
                        optimizer_stage=pol.optimizer_stage, worker_overhead_bytes=pol.worker_overhead_bytes,
                        semantic_activation_cache_bytes=pol.semantic_activation_cache_bytes,
                        max_worker_groups_per_gpu=pol.max_worker_groups_per_gpu,
                        activation_checkpointing=pol.activation_checkpointing)
        return not (max(O.device_peaks(nodes, mm).values()) > mm.capacity())

    def broken(plan, v, k):
        sigma, pi, mb = dict(plan.sigma), dict(plan.pi), dict(plan.mb)
        dp, pp, tp = pi[v]
        a = sigma[v]
        if k == 0:
            mb[v] = mb[v] + 1                                      # micro-batch rule
        elif k == 1:
            pi[v] = (dp, pp, 3)                                    # tp does not divide G
        elif k == 2:
            sigma[v] = Allocation(origin=(a.origin[0], a.origin[1] + p.device_space.N, a.origin[2]), extent=a.extent)
        elif k == 3:
            sigma[v] = Allocation(origin=a.origin, extent=(a.extent[0], a.extent[1], a.extent[2] + 1))
        elif k == 4:
            del mb[v]                                              # coverage
        return ExecutionPlan(sigma, pi, mb)

    n_true = n_false = n_view = 0
    for i in range(batch.n):
        rpeg, plan, wl = batch.configuration(p, i)
        views = [frozenset(rpeg.trainable)]
        if Model.AC_SHARE in rpeg.trainable:
            views.append(frozenset({Model.ACTOR, Model.CRITIC}))
        for trainable in views:
            mm = NodeMemoryModel.from_policy(p.hw, p.suite, wl, pol, trainable=trainable)
            variants = [plan] + ([broken(plan, rpeg.vertices[i % len(rpeg.vertices)], i % 5)] if trainable == views[0] else [])
            for q in variants:
                got = is_valid(Configuration(rpeg, q, p.device_space), p.suite, wl, mm)
                assert got == restated(rpeg, q, wl, trainable), (i, sorted(m.value for m in trainable))
                n_true += got
                n_false += not got
        if len(views) == 2:
            n_view += restated(rpeg, plan, wl, views[0]) != restated(rpeg, plan, wl, views[1])
    assert n_true > 0 and n_false > 0
    print("valid", n_true, "invalid", n_false, "plans on which the two memory views disagree", n_view)


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_gates_equal_reference_verdicts(c):
    """The drop-in is_valid and evaluate_cached (through the engine: k_signature's gate, the stale rule, the
    memory fit, the penalty) against what the reference's own functions returned for seeded plans and for
    plans broken one rule at a time (tests/golden/ref_validity.json)."""
    import json
    import os
    from rpeg_amd.model.memory import NodeMemoryModel
    from rpeg_amd.search.cache import EvalCache
    from rpeg_amd.search import evaluate as evaluate_mod
    from rpeg_amd.search.evaluate import Configuration, evaluate_cached, is_valid
    from tests.golden.make_golden_validity import validity_cases
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_validity.json")) as f:
        rows = json.load(f)["configs"][str(c)]
    cfg, batch, cases = validity_cases(c)
    p = cfg.problem
    n_valid = n_scored = n_hard = 0
    for want, (i, rule, rpeg, plan, wl) in zip(rows, cases):
        config = Configuration(rpeg, plan, p.device_space)
        mm = NodeMemoryModel.from_policy(p.hw, p.suite, wl, p.memory_policy, trainable=frozenset(rpeg.trainable))
        assert is_valid(config, p.suite, wl, mm) == want["is_valid"], (i, rule)
        n_valid += want["is_valid"]
        if "score" in want and all(want["compatible"]) and rule in (None, 8):
            score, _, feasible, miss = evaluate_cached(config, EvalCache(), p.suite, wl, p.hw, p.K_eval, p.memory_policy)
            assert float(score).hex() == want["score"] and feasible == want["feasible"] and miss, (i, rule)
            n_scored += 1
            if "score_hard_oom" in want:     # the hard-OOM switch, as the reference's evaluate_cached applies it
                evaluate_mod.ABLATION_HARD_OOM = True
                try:
                    hard = evaluate_cached(config, EvalCache(), p.suite, wl, p.hw, p.K_eval, p.memory_policy)
                finally:
                    evaluate_mod.ABLATION_HARD_OOM = False
                assert float(hard[0]).hex() == want["score_hard_oom"] and hard[2] == want["feasible_hard_oom"], (i, rule)
                n_hard += 1
    assert n_valid and n_scored and n_hard


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_transfer_resource_policies_equal_reference(c):
    """Both-endpoints reservations for weights, for activations and for both: makespans of batched launches
    and, through the drop-in evaluate(), dispatch order, finish times and utilisation against the reference
    scheduler's (tests/golden/ref_transfer_policy.json)."""
    from rpeg_amd.core.types import TransferResourcePolicy
    from rpeg_amd.engine.runtime import Engine
    from rpeg_amd.search.evaluate import Configuration, evaluate
    from tests.helpers import load_transfer_policy_golden, order_crc, with_transfer_policy
    gold = load_transfer_policy_golden()
    g = gold["configs"][str(c)]
    cfg, batch = seeded_batch(c, g["n_plans"])
    p = cfg.problem
    for k, pol in enumerate(gold["policies"]):
        eng = Engine(with_transfer_policy(p, *pol))
        out = eng.eval(batch, gate_stale=False)
        for i in range(g["n_plans"]):
            assert float(out["makespan"][i]).hex() == g["rows"][i][k]["makespan"], (i, pol)
            assert not out["mask"][i] & abi.MASK_ERROR
        for i in range(0, g["n_plans"], 8):
            util, _ = eng.trace_metrics(batch, i)
            assert float(util).hex() == g["rows"][i][k]["utilization"], (i, pol)
        tp = TransferResourcePolicy(weight=pol[0], activation=pol[1])
        for i in range(0, g["n_plans"], 24):
            rpeg, plan, wl = batch.configuration(p, i)
            conf = Configuration(rpeg, plan, p.device_space, transfer_resource_policy=tp)
            _, trace, _ = evaluate(conf, p.suite, wl, p.hw, p.K_eval, p.memory_policy)
            want = g["rows"][i][k]
            assert trace.makespan().hex() == want["makespan"], (i, pol)
            assert order_crc([n.id for n in trace.start]) == want["order_crc"], (i, pol)
            assert math.fsum(trace.finish.values()).hex() == want["finish_sum"], (i, pol)
            assert float(trace.utilization()).hex() == want["utilization"], (i, pol)


def test_a_horizon_beyond_the_ready_lists_is_evaluated_all_the_same():
    """DPO's unrolled steps are independent of each other, so every step's first node is ready at time zero: at a
    horizon of 128 steps the ready set holds 128 entries, at 40 steps more than the 32 the four-lanes-per-plan kernel
    keeps in registers.  The reference's heap has no capacity (scheduler.py:423-546), and neither has the call: plans
    that outgrow a kernel's ready set are redone by the launch that ends the call, with a list as long as the graph.
    Whatever the layout, every plan comes back with the host build's bits and no plan with RPEG_MASK_LIMIT."""
    from dataclasses import replace
    from rpeg_amd.engine.runtime import Engine
    cfg, batch = seeded_batch(4, 2048)
    for K, layouts in ((24, (-1, 4)), (33, (-1, 0, 1, 4)), (40, (-1, 0, 4)), (128, (-1, 0))):
        p = replace(cfg.problem, K_eval=K)
        ref = CpuPort(p).eval(batch, flags=abi.GATE_STALE, threads=16)
        assert ref["max_ready"] >= min(K, 33)
        for lanes in layouts:
            eng = Engine(p)
            eng.set_state_lanes(lanes)
            for _ in range(2):
                out = eng.eval(batch)
                assert (eng.stats()["quad_tasks"] > 0) == (lanes == 4)
                assert not np.any(out["mask"] & abi.MASK_LIMIT), (K, lanes)
                assert np.array_equal(out["mask"], ref["mask"]), (K, lanes)
                assert same_bits(out["score"], ref["score"]) and same_bits(out["makespan"], ref["makespan"]), (K, lanes)
            if K == 40:   # the critical-chain masses of redone plans come from the same launch
                m = eng.eval_mass_device(batch)["mass"]
                want = CpuPort(p).eval(batch, flags=0, threads=16, want_mass=True)["mass"]
                assert same_bits(m, want), lanes
            eng.close()
    with pytest.raises(ValueError, match="K_eval"):     # a stated bound: graphs of at most 4,095 lowered nodes
        Engine(replace(cfg.problem, K_eval=5000))


def test_short_ready_lists_and_dense_graphs_in_every_layout():
    """Plans that outgrow a deliberately short ready list of the main kernel (8 entries), and a seeded subset of
    config 3 (ready sets of up to 24 entries, fan-outs of four) in the four-lanes-per-plan kernel: the same bits as
    the host build in every layout, and the same masks from every layout."""
    from rpeg_amd.engine.runtime import Engine
    cfg, batch = seeded_batch(3, 6000, start=40_000)
    ref = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE, threads=16)
    assert ref["max_ready"] > 16
    masks = []
    for lanes, cap in ((0, 8), (0, 32), (4, 32), (1, 32), (-1, 16)):
        eng = Engine(cfg.problem)
        eng.set_state_lanes(lanes)
        eng.set_ready_cap(cap)
        for _ in range(2):
            out = eng.eval(batch)
            assert same_bits(out["score"], ref["score"]) and same_bits(out["peak"], ref["peak"]), (lanes, cap)
            masks.append(out["mask"].copy())
        eng.close()
    assert all(np.array_equal(m, ref["mask"]) for m in masks)


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_utilization_from_the_batched_launch_equals_reference(c):
    """Trace.utilization() as a further output of the batched launch (rpeg_eval_host_util, folded inside k_plan)
    against the reference's own numbers for every plan of tests/golden/ref_transfer_policy.json under the three
    transfer-reservation policies, against the single-plan trace path for other seeded plans, and NaN / mask for
    plans that are not evaluated; the other outputs are those of the plain launch."""
    from rpeg_amd.engine.runtime import Engine, EngineError
    from tests.helpers import load_transfer_policy_golden, with_transfer_policy
    gold = load_transfer_policy_golden()
    g = gold["configs"][str(c)]
    cfg, batch = seeded_batch(c, g["n_plans"])
    p = cfg.problem
    for k, pol in enumerate(gold["policies"]):
        eng = Engine(with_transfer_policy(p, *pol))
        out = eng.eval_util(batch, gate_stale=False)
        plain = eng.eval(batch, gate_stale=False)
        for key in ("makespan", "peak", "score"):
            assert same_bits(out[key], plain[key]), (pol, key)
        assert np.array_equal(out["mask"], plain["mask"])
        for i in range(g["n_plans"]):
            assert float(out["util"][i]).hex() == g["rows"][i][k]["utilization"], (i, pol)
        eng.close()
    eng = engine(c)
    _, more = seeded_batch(c, 300, start=700_000)
    out = eng.eval_util(more)
    valid = np.flatnonzero((out["mask"] & abi.MASK_VALID) != 0)
    assert len(valid) > 100
    for i in valid[::7]:
        assert float(out["util"][i]).hex() == float(eng.trace_metrics(more, int(i))[0]).hex(), i
    assert np.all((out["util"][valid] > 0.0) & (out["util"][valid] <= 1.0))
    more.vert[0, 3] = 3           # tp = 3 divides no G: not evaluated
    bad = eng.eval_util(more.slice(0, 8))
    assert bad["mask"][3] == 0 and np.isnan(bad["util"][3]) and not np.isnan(bad["util"][2])
    # any number of plans: a launch for every 1,024 of them
    _, many = seeded_batch(c, 2600, start=300_000)
    whole = eng.eval_util(many)
    plain = eng.eval(many, gate_stale=False)
    assert same_bits(whole["score"], plain["score"]) and np.array_equal(whole["mask"], plain["mask"])
    for a in (0, 1024, 2048):
        part = eng.eval_util(many.slice(a, min(a + 1024, many.n)))
        assert same_bits(whole["util"][a:a + 1024], part["util"]), a


def test_utilization_of_classes_beyond_a_wavefront_is_traced_plan_by_plan():
    """A problem whose graphs outgrow the plan-per-wavefront kernel (above 384 nodes): eval_util gives the numbers of
    the single-plan trace and the other outputs of the plain call."""
    from rpeg_amd.engine.runtime import Engine
    import dataclasses
    cfg, batch = seeded_batch(1, 24)
    eng = Engine(dataclasses.replace(cfg.problem, K_eval=24))
    out = eng.eval_util(batch, gate_stale=False)
    plain = eng.eval(batch, gate_stale=False)
    assert eng.stats()["classes"] > 0
    assert same_bits(out["score"], plain["score"]) and np.array_equal(out["mask"], plain["mask"])
    ok = np.flatnonzero(((out["mask"] & abi.MASK_VALID) != 0) & ((out["mask"] & abi.MASK_ERROR) == 0))
    assert len(ok) > 8
    for i in ok:
        assert float(out["util"][i]).hex() == float(eng.trace_metrics(batch, int(i))[0]).hex(), i
    assert np.all((out["util"][ok] > 0.0) & (out["util"][ok] <= 1.0))
    eng.close()


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_other_seeds_unroll_depths_and_policies_equal_the_host_build(c):
    """Away from the shipped problems: unroll depths 1, 2, 7 and (three configurations) 32, both-endpoints reservations and two other
    seeds of the candidate generator.  Every makespan, peak, score and mask of the batched launch equals the
    host build of the same arithmetic, whose scheduler is written differently (a push-ordered list, one pop per
    iteration) and is itself checked against the reference vectors."""
    from dataclasses import replace
    from rpeg_amd.core.types import TransferResourcePolicy
    from rpeg_amd.engine.runtime import Engine
    cfg = configs.config(c)
    n = 8192 if c != 5 else 2048
    cases = [(1, ("destination_only", "destination_only")), (2, ("both_endpoints", "destination_only")),
             (7, ("both_endpoints", "both_endpoints"))]
    if c in (1, 2, 4):   # a long horizon, as the runtime's planner schedules (runtime/job_plan.py:174-213)
        cases.append((32, ("destination_only", "destination_only")))
    if c in (1, 2, 3):   # and a longer one: graphs of 1,500-3,000 lowered nodes
        cases.append((100, ("destination_only", "destination_only")))
    for K, pol in cases:
        p = replace(cfg.problem, K_eval=K, transfer_resource_policy=TransferResourcePolicy(*pol))
        eng, port = Engine(p), CpuPort(p)
        for seed in (7, 1234):
            batch = candidates_of(p, cfg, n, seed, c)
            got = eng.eval(batch, gate_stale=True)
            want = port.eval(batch, flags=abi.GATE_STALE, threads=16)
            for k in ("makespan", "peak", "score"):
                assert same_bits(got[k], want[k]), (K, pol, seed, k)
            assert np.array_equal(got["mask"], want["mask"]), (K, pol, seed)


def candidates_of(problem, cfg, n, seed, tag):
    from rpeg_amd.search import candidates
    return candidates.generate(problem, n, cfg.tau_choices, seed=seed, tag=tag)


@pytest.mark.parametrize("c", [1, 2, 3, 4])
def test_memory_policies_equal_reference(c):
    """Optimizer stages 0-2, checkpointing off, runtime overhead fraction, per-worker overhead and cache bytes and
    the worker-group limit: batched launches, and evaluate_cached() with the policy as its argument, against the
    reference's evaluations (tests/golden/ref_memory_policy.json)."""
    from rpeg_amd.engine.runtime import Engine
    from rpeg_amd.model.memory import MemoryPolicy
    from rpeg_amd.search.cache import EvalCache
    from rpeg_amd.search.evaluate import Configuration, evaluate_cached
    from tests.helpers import load_memory_policy_golden, with_memory_policy
    gold = load_memory_policy_golden()
    g = gold["configs"][str(c)]
    cfg, batch = seeded_batch(c, g["n_plans"])
    for k, pol in enumerate(gold["policies"]):
        p = with_memory_policy(cfg.problem, pol)
        out = Engine(p).eval(batch, gate_stale=False)
        for i in range(g["n_plans"]):
            want = g["rows"][i][k]
            assert float(out["makespan"][i]).hex() == want["makespan"], (i, pol)
            assert float(out["peak"][i]).hex() == want["peak"], (i, pol)
            assert float(out["score"][i]).hex() == want["score"], (i, pol)
            assert bool(out["mask"][i] & abi.MASK_MEM_OK) == want["feasible"], (i, pol)
        for i in range(0, g["n_plans"], 16):
            rpeg, plan, wl = batch.configuration(p, i)
            if not oracle.stale_publication_layout_valid(rpeg, plan):
                continue                      # evaluate_cached gates those to 0 (evaluate.py:364-376)
            s, _, feasible, _ = evaluate_cached(Configuration(rpeg, plan, p.device_space), EvalCache(), p.suite, wl,
                                                p.hw, p.K_eval, MemoryPolicy(**pol))
            assert float(s).hex() == g["rows"][i][k]["score"] and feasible == g["rows"][i][k]["feasible"], (i, pol)


@pytest.mark.parametrize("c", [1, 2, 3, 4])
def test_calibrated_hardware_equals_reference(c):
    """Per-role operator scales, weight-transfer and reshard scales, the fixed activation-transfer overhead,
    gemm_k_half and other link / efficiency parameters: batched launches against the reference's evaluations
    (tests/golden/ref_hardware.json)."""
    from rpeg_amd.engine.runtime import Engine
    from tests.helpers import load_hardware_golden, with_hardware
    gold = load_hardware_golden()
    g = gold["configs"][str(c)]
    cfg, batch = seeded_batch(c, g["n_plans"])
    for k, ov in enumerate(gold["overlays"]):
        out = Engine(with_hardware(cfg.problem, ov)).eval(batch, gate_stale=False)
        for i in range(g["n_plans"]):
            want = g["rows"][i][k]
            assert float(out["makespan"][i]).hex() == want["makespan"], (i, k)
            assert float(out["peak"][i]).hex() == want["peak"], (i, k)
            assert float(out["score"][i]).hex() == want["score"], (i, k)
            assert bool(out["mask"][i] & abi.MASK_MEM_OK) == want["feasible"], (i, k)


def test_problems_away_from_the_shipped_configurations_equal_reference():
    """PPO and GRPO without generation quantiles, one and six quantiles, K > 1, meshes with 2 and 8 devices per
    node, 4-byte elements, another head size, a stated parameter count: batched launches against the reference's
    evaluations (tests/golden/ref_variants.json), and 4,096 further plans of each against the host build."""
    from rpeg_amd.engine.runtime import Engine
    from rpeg_amd.search import candidates
    from tests.golden.make_golden_variants import variant_problems
    from tests.helpers import variant_cases
    for name, p, batch, rows in variant_cases():
        eng = Engine(p)
        out = eng.eval(batch, gate_stale=False)
        for i, want in enumerate(rows):
            assert float(out["makespan"][i]).hex() == want["makespan"], (name, i)
            assert float(out["peak"][i]).hex() == want["peak"], (name, i)
            assert float(out["score"][i]).hex() == want["score"], (name, i)
            assert bool(out["mask"][i] & abi.MASK_MEM_OK) == want["feasible"], (name, i)
    for name, p, tau_choices, tag in variant_problems():
        more = candidates.generate(p, 4096, tau_choices, seed=9, tag=tag)
        got, want = Engine(p).eval(more, gate_stale=True), CpuPort(p).eval(more, flags=abi.GATE_STALE, threads=16)
        for k in ("makespan", "peak", "score"):
            assert same_bits(got[k], want[k]), (name, k)
        assert np.array_equal(got["mask"], want["mask"]), name


def test_profile_tool_runs(capsys):
    """python -m rpeg_amd.engine.profile: the per-wavefront clocks of both kernels on a small seeded set."""
    import sys
    from rpeg_amd.engine import profile
    argv = sys.argv
    sys.argv = ["profile", "--config", "2", "--plans", "40000"]
    try:
        profile.main()
    finally:
        sys.argv = argv
    text = capsys.readouterr().out
    assert "k_eval:" in text and "k_plan:" in text and "phases, mean us per task" in text and "longest tasks" in text
