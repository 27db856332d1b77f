"""Pins of the Python oracle that do not come from running the reference: hand tables, closed forms
from the reference's README files, integer identities, special cases that reduce to a textbook
roofline, and an independent brute-force scheduler / per-device memory enumeration."""

import itertools
import math
import random

import pytest

from oracle import rpeg_oracle as oracle
from rpeg_amd import configs
from rpeg_amd.core.types import Allocation, Model
from rpeg_amd.ir.plan import ExecutionPlan
from tests.helpers import oracle_eval, seeded_batch


# ------------------------------------------------------------------ geometry (core/types.py:16-85)
def test_packing_geometry_hand_table():
    table = {(1, 1, 1): (1, 1), (3, 1, 1): (3, 1), (8, 1, 1): (4, 2), (2, 2, 1): (4, 1), (2, 2, 2): (4, 2),
             (1, 8, 4): (4, 8), (4, 2, 2): (4, 4), (1, 4, 2): (4, 2), (3, 1, 2): None}
    for (dp, pp, tp), want in table.items():
        assert oracle.packing_geometry(dp, pp, tp, 4) == want


def test_packing_geometry_device_count_invariant():
    # whenever s*tp divides G the box holds exactly dp*pp*tp devices
    for G in (2, 4, 8):
        for dp, pp, tp in itertools.product(range(1, 33), range(1, 33), (1, 2, 4, 8)):
            if tp > G:
                continue
            geom = oracle.packing_geometry(dp, pp, tp, G)
            s = min(pp, G // tp)
            if geom is not None and s and G % (s * tp) == 0:
                assert geom[0] * geom[1] == dp * pp * tp


def test_rectangular_layouts():
    assert oracle.rectangular_node_layouts(84, 4, 42) == ((2, 42), (3, 28), (4, 21))
    assert oracle.rectangular_node_layouts(0, 4, 4) == ()
    assert oracle.rectangular_node_layouts(7, 4, 4) == ()


def test_disjoint_overlap_consistency():
    rng = random.Random(1)
    for _ in range(2000):
        a = Allocation(tuple(rng.randrange(4) for _ in range(3)), tuple(rng.randrange(1, 4) for _ in range(3)))
        b = Allocation(tuple(rng.randrange(4) for _ in range(3)), tuple(rng.randrange(1, 4) for _ in range(3)))
        da, db = set(oracle.alloc_devices(a)), set(oracle.alloc_devices(b))
        assert oracle.allocs_disjoint(a, b) == (not (da & db))
        assert oracle.allocations_overlap(a, b) == bool(da & db)
        assert oracle.alloc_overlap_size(a, b) == len(da & db)


# ------------------------------------------------------------------ generation phases (lower.py:288-327)
@pytest.mark.parametrize("c,want", [
    (1, [(64, 32, 127, 0, True), (32, 22, 128, 127, False), (10, 10, 256, 255, False)]),
    (2, [(1024, 512, 1023, 0, True), (512, 410, 1024, 1023, False), (102, 102, 2048, 2047, False)]),
    (3, [(256, 77, 1023, 0, True), (179, 102, 3072, 1023, False), (77, 64, 2048, 4095, False), (13, 13, 2048, 6143, False)]),
    (5, [(2048, 1024, 2047, 0, True), (1024, 819, 6144, 2047, False), (205, 205, 8192, 8191, False)]),
])
def test_gen_phases_kat(c, want):
    assert oracle.gen_phases(configs.config(c).problem.workload) == want


# ------------------------------------------------------------------ parameters and work (models.py, cost.py:481-535)
def test_parameter_counts():
    s7, s13, s70 = configs.SPEC_7B, configs.SPEC_13B, configs.SPEC_70B
    assert oracle.transformer_parameter_count(s7, Model.ACTOR) == 5_164_236_800
    assert oracle.transformer_parameter_count(s7, Model.CRITIC) == 5_164_240_896
    assert oracle.transformer_parameter_count(s13, Model.ACTOR) == 10_020_454_400
    assert oracle.transformer_parameter_count(s13, Model.REWARD) == 10_020_459_520
    assert oracle.transformer_parameter_count(s70, Model.ACTOR) == 60_106_473_472
    assert oracle.transformer_parameter_count(s70, Model.AC_SHARE) == 60_106_481_664


def _mock(problem, vid, pi=(1, 1, 1), mb=1, extent=(1, 1, 1), **sub):
    rpeg = problem.template(0)
    v = next(x for x in rpeg.vertices if x.id == vid)
    return oracle.XNode("_mock", oracle.OP, (Allocation((0, 0, 0), extent),), tpl=v, k=0, model=v.kind.model,
                        pi=pi, mb=mb, **sub)


def test_training_work_exact_integers():
    for c, want in ((1, 1_719_704_905_318_400), (2, 217_742_884_718_247_936), (5, 20_396_978_634_221_420_544)):
        p = configs.config(c).problem
        cost = oracle.CostModel(p.hw, p.suite, p.workload)
        assert cost.work_cost(_mock(p, "t_pi")) == want


def test_single_device_is_textbook_roofline():
    # dp=pp=tp=1: every (p-1) factor vanishes, so T = W/(F*eta) (+ optimizer step for training)
    p = configs.config(1).problem
    cost = oracle.CostModel(p.hw, p.suite, p.workload)
    wl, hw = p.workload, p.hw
    for vid in ("i_ref", "i_R", "i_V", "t_pi", "t_V"):
        n = _mock(p, vid)
        assert cost.intra_comm(n) == 0.0 and cost.non_gemm(n) == 0.0
        M = wl.B * wl.K * (wl.S + wl.T)
        eta = M / (M + hw.gemm_m_half)
        want = cost.work_cost(n) / (hw.flops_per_gpu * eta)
        if vid.startswith("t_"):
            sp = p.suite.specs[n.model]
            want += (sp.L * (4 * sp.d ** 2 + 2 * sp.d * sp.d_ff) + sp.V * sp.d) * 18 / hw.memory_bandwidth
        assert cost.op_time(n) == pytest.approx(want, rel=1e-13)


def test_config1_numeric_anchors():
    p = configs.config(1).problem
    cost = oracle.CostModel(p.hw, p.suite, p.workload)
    assert cost.op_time(_mock(p, "i_ref")) == pytest.approx(0.9828302848, rel=1e-12)
    assert cost.op_time(_mock(p, "i_R")) == pytest.approx(0.9582840750894546, rel=1e-12)
    assert cost.op_time(_mock(p, "t_pi")) == pytest.approx(4.0242774016, rel=1e-12)
    assert cost.op_time(_mock(p, "t_V")) == pytest.approx(3.92609562624, rel=1e-12)
    assert cost.op_time(_mock(p, "g_pi")) == pytest.approx(14.571504043340633, rel=1e-12)
    big = dict(pi=(2, 2, 2), mb=4, extent=(1, 2, 4))
    assert cost.op_time(_mock(p, "i_ref", **big)) == pytest.approx(25.3433646144, rel=1e-12)
    assert cost.op_time(_mock(p, "t_pi", **big)) == pytest.approx(281.4369117552, rel=1e-12)
    assert cost.op_time(_mock(p, "g_pi", **big)) == pytest.approx(46.694172971460716, rel=1e-12)
    assert cost.op_time(_mock(p, "i_ref", n_seqs=22, **big)) == pytest.approx(8.729673934800001, rel=1e-12)


def test_breakdown_sums_to_time():
    for c in (1, 2, 3, 4):
        cfg, batch = seeded_batch(c, 24)
        p = cfg.problem
        for i in range(24):
            rpeg, plan, wl = batch.configuration(p, i)
            nodes, _ = oracle.lower(rpeg, plan, p.suite, 1, wl)
            cost = oracle.CostModel(p.hw, p.suite, wl)
            for n in nodes:
                if n.kind == oracle.OP:
                    assert sum(cost.breakdown(n)) == pytest.approx(cost.op_time(n), rel=1e-12)


def test_isolated_peaks_config1():
    p = configs.config(1).problem
    rpeg = p.template(0)
    mm = oracle.make_mem_model(rpeg, p.suite, p.workload, p.hw, p.memory_policy)
    assert mm.peak_bytes(_mock(p, "t_pi")) == 100_495_523_840
    assert mm.peak_bytes(_mock(p, "i_ref")) == 13_547_601_920
    assert mm.peak_bytes(_mock(p, "g_pi")) == 32_656_850_944


# ------------------------------------------------------------------ lowering structure (lower.py)
def _uniform_plan(rpeg, alloc, pi=(1, 1, 1), mb=1, overrides=None):
    overrides = overrides or {}
    sigma = {v: overrides.get(v.id, {}).get("alloc", alloc) for v in rpeg.vertices}
    pis = {v: overrides.get(v.id, {}).get("pi", pi) for v in rpeg.vertices}
    return ExecutionPlan(sigma=sigma, pi=pis, mb={v: mb for v in rpeg.vertices})


def test_colocated_plan_has_no_transfers():
    p = configs.config(1).problem
    rpeg = p.template(0)
    plan = _uniform_plan(rpeg, Allocation((0, 0, 0), (1, 1, 1)))
    nodes, edges = oracle.lower(rpeg, plan, p.suite, p.K_eval, p.workload)
    assert len(nodes) == 6 * p.K_eval and all(n.kind == oracle.OP for n in nodes)


def test_fully_disjoint_ppo_counts():
    p = configs.config(1).problem
    rpeg = p.template(0)
    plan = ExecutionPlan(sigma={v: Allocation((0, i, 0), (1, 1, 1)) for i, v in enumerate(rpeg.vertices)},
                         pi={v: (1, 1, 1) for v in rpeg.vertices}, mb={v: 1 for v in rpeg.vertices})
    nodes, _ = oracle.lower(rpeg, plan, p.suite, p.K_eval, p.workload)
    Q, K = 3, p.K_eval
    assert sum(n.kind == oracle.OP for n in nodes) == (4 * Q + 2) * K
    # 3Q gen->inf transfers + 6 inf->train transfers per step, 2 publications for every step k >= 1
    assert sum(n.kind == oracle.COMM for n in nodes) == (3 * Q + 6) * K + 2 * (K - 1)
    assert sum(n.kind == oracle.RESHARD for n in nodes) == 0


def test_same_alloc_different_pi_reshards():
    p = configs.config(1).problem
    rpeg = p.template(0)
    a = Allocation((0, 0, 0), (1, 1, 2))
    plan = _uniform_plan(rpeg, a, pi=(2, 1, 1), overrides={"g_pi": {"pi": (1, 1, 2)}})
    nodes, edges = oracle.lower(rpeg, plan, p.suite, p.K_eval, p.workload)
    # g_pi@k -> reshard -> t_pi@k in every step; t_pi is then marked resharded, but the publication
    # targets g_pi, whose template is not, so every step k >= 1 also gets a publication reshard
    assert sum(n.kind == oracle.RESHARD for n in nodes) == p.K_eval + (p.K_eval - 1)


def test_unroll_counts():
    p = configs.config(2).problem
    for tau in (0, 1, 2):
        rpeg = p.template(0, [tau])
        nodes, data, pubs = oracle.unroll(rpeg, 5)
        assert len(nodes) == 4 * 5 and len(data) == 4 * 5
        assert len(pubs) == sum(1 for k in range(1, 5) if k > tau)
        assert all(src[1] == max(0, dst[1] - tau - 1) for src, dst, _ in pubs)


# ------------------------------------------------------------------ scheduler (scheduler.py:270-552)
def test_dpo_colocated_dispatch_order():
    p = configs.config(4).problem
    rpeg = p.template(0)
    plan = _uniform_plan(rpeg, Allocation((0, 0, 0), (1, 1, 4)), pi=(4, 1, 1))
    nodes, edges = oracle.lower(rpeg, plan, p.suite, 2, p.workload)
    cost = oracle.CostModel(p.hw, p.suite, p.workload)
    start, finish, order = oracle.schedule(nodes, edges, cost, p.device_space)
    # i_ref@1 overtakes t_pi@0: the sorted-id index precedes the rank in the heap key
    assert order == ["i_pi@0", "i_ref@0", "i_ref@1", "t_pi@0", "i_pi@1", "t_pi@1"]
    # colocated: the makespan is the left fold of the durations in dispatch order
    t = 0.0
    by_id = {n.id: n for n in nodes}
    for nid in order:
        t = t + cost.time(by_id[nid])
    assert max(finish.values()) == t


def _brute_schedule(nodes, edges, dur, rank, prio, tidx, blocked):
    """Independent restatement: scan all ready nodes every round, per-device availability."""
    preds = {n: [] for n in nodes}
    succs = {n: [] for n in nodes}
    for a, b in edges:
        preds[b].append(a)
        succs[a].append(b)
    avail = {}
    fin, key, order = {}, {}, []
    ctr = 0
    left = {n: len(preds[n]) for n in nodes}
    for n in nodes:
        if left[n] == 0:
            key[n] = (0.0, ctr)
            ctr += 1
    while key:
        n = min(key, key=lambda x: (key[x][0], prio[x], tidx[x], -rank[x], key[x][1]))
        est = max([fin[q] for q in preds[n]] + [0.0] + [avail.get(d, 0.0) for d in blocked[n]])
        if est > key[n][0]:
            key[n] = (est, ctr)
            ctr += 1
            continue
        del key[n]
        fin[n] = est + dur[n]
        order.append(n)
        for d in blocked[n]:
            avail[d] = fin[n]
        for w in succs[n]:
            left[w] -= 1
            if left[w] == 0:
                e = max([fin[q] for q in preds[w]] + [avail.get(d, 0.0) for d in blocked[w]])
                key[w] = (e, ctr)
                ctr += 1
    return fin, order


def test_heap_scheduler_equals_brute_force_on_lowered_plans():
    for c in (1, 2, 4):
        cfg, batch = seeded_batch(c, 12)
        p = cfg.problem
        for i in range(12):
            res = oracle_eval(p, batch, i, want_trace=True)
            nodes, edges = res["nodes"], res["edges"]
            rpeg, plan, wl = batch.configuration(p, i)
            cost = oracle.CostModel(p.hw, p.suite, wl)
            ids = [n.id for n in nodes]
            dur = {n.id: cost.time(n) for n in nodes}
            rank = oracle.node_ranks(nodes, edges, dur)
            tpl = sorted({n.tpl.id for n in nodes if n.kind == oracle.OP})
            prio = {n.id: int(n.kind == oracle.OP) for n in nodes}
            tidx = {n.id: (tpl.index(n.tpl.id) if n.kind == oracle.OP else len(tpl)) for n in nodes}
            pr = {n.id: set() for n in nodes}
            su = {n.id: set() for n in nodes}
            for a, b in edges:
                pr[b.id].add(a.id)
                su[a.id].add(b.id)
            by_id = {n.id: n for n in nodes}
            blocked = {n.id: {d for al in oracle.reserved_allocations(n, pr, su, by_id) for d in oracle.alloc_devices(al)}
                       for n in nodes}
            fin, order = _brute_schedule(ids, [(a.id, b.id) for a, b in edges], dur, rank, prio, tidx, blocked)
            assert order == res["order"]
            assert fin == res["finish"]


def test_schedule_invariants():
    cfg, batch = seeded_batch(2, 16)
    p = cfg.problem
    for i in range(16):
        res = oracle_eval(p, batch, i, want_trace=True)
        start, finish = res["start"], res["finish"]
        for a, b in res["edges"]:
            assert start[b.id] >= finish[a.id]
        assert res["makespan"] == max(finish.values())
        assert all(finish[n] >= start[n] for n in start)


# ------------------------------------------------------------------ memory and score (memory.py, evaluate.py)
def test_peaks_independent_of_unroll_depth_and_quantiles():
    cfg, batch = seeded_batch(1, 16)
    p = cfg.problem
    for i in range(16):
        rpeg, plan, wl = batch.configuration(p, i)
        mm = oracle.make_mem_model(rpeg, p.suite, wl, p.hw, p.memory_policy)
        a = oracle.device_peaks(oracle.lower(rpeg, plan, p.suite, 1, wl)[0], mm)
        b = oracle.device_peaks(oracle.lower(rpeg, plan, p.suite, 5, wl)[0], mm)
        assert max(a.values()) == max(b.values())


def test_penalty_closed_form():
    cfg, batch = seeded_batch(2, 64)
    for i in range(64):
        r = oracle_eval(cfg.problem, batch, i)
        if r["feasible"]:
            assert r["score"] == r["raw"]
        else:
            want = r["raw"] * max(math.exp(-40.0 * (r["peak"] / r["cap"] - 1.0)), 1e-12)
            assert r["score"] == want
