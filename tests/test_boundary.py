"""The reference's pipeline call sequence on the drop-in modules (rpeg_amd.compat): unroll -> lower ->
NodeCostModel.time -> schedule -> _device_peaks / mem_worst_violation, against what the reference's own functions
returned for the same seeded plans (tests/golden/ref_boundary.json, written by make_golden_boundary.py)."""

import importlib.util
import json
import os
import sys

import pytest

import rpeg_amd.compat as compat
from tests.helpers import GOLDEN, seeded_batch


def _generator():
    spec = importlib.util.spec_from_file_location("make_golden_boundary", os.path.join(GOLDEN, "make_golden_boundary.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _gold():
    with open(os.path.join(GOLDEN, "ref_boundary.json")) as f:
        return json.load(f)


@pytest.fixture
def names():
    compat.install()
    yield
    compat.uninstall()


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_unroll_and_lower_equal_the_reference_graphs(names, c):
    """Host work only: the unrolled graph and every field of every lowered node and edge, in order."""
    from passes.lower import ExecNodeType, lower
    from passes.unroll import unroll
    gen, gold = _generator(), _gold()
    cfg, batch = seeded_batch(c, gold["n_plans"])
    p = cfg.problem
    for i, want in enumerate(gold["configs"][str(c)]):
        rpeg, plan, wl = batch.configuration(p, i)
        unrolled = unroll(rpeg, p.K_eval, verbose=False)
        lowered = lower(rpeg, unrolled, plan, p.suite, p.K_eval, workload=wl, verbose=False)
        assert [len(unrolled.nodes), len(unrolled.data_edges), len(unrolled.pub_edges)] == want["unroll"][:3]
        assert gen._crc([[e.src.template_vertex.id, e.src.k, e.dst.template_vertex.id, e.dst.k, e.container.name,
                          e.kind.value] for e in unrolled.pub_edges + unrolled.data_edges]) == want["unroll"][3]
        rows = [[n.id, n.kind.value, [gen._alloc(a) for a in n.allocs],
                 None if n.op is None else [n.op.template_vertex.id, n.op.k],
                 None if n.model is None else n.model.value, None if n.pi is None else list(n.pi), n.mb, n.n_seqs,
                 n.n_active, n.phase_steps, n.phase_t_start, bool(n.is_prefill_phase), int(n.payload_in_bytes), n.label]
                for n in lowered.nodes]
        assert rows[:3] + rows[-2:] == want["first_nodes"], i
        assert (len(rows), gen._crc(rows)) == (want["n_nodes"], want["nodes_crc"]), i
        assert gen._crc([[e.src.id, e.dst.id] for e in lowered.edges]) == want["edges_crc"], i
        assert sum(n.kind == ExecNodeType.OP for n in lowered.nodes) >= len(rpeg.vertices) * p.K_eval
        assert all(n.op in unrolled.nodes for n in lowered.nodes if n.kind == ExecNodeType.OP and n.n_seqs is None)


def test_lower_errors_and_plans_without_microbatches(names):
    from ir.plan import ExecutionPlan
    from passes.lower import lower
    from passes.unroll import unroll
    cfg, batch = seeded_batch(2, 4)
    p = cfg.problem
    rpeg, plan, wl = batch.configuration(p, 1)
    with pytest.raises(ValueError, match="K_eval"):
        unroll(rpeg, 0)
    short = ExecutionPlan(sigma={v: a for v, a in list(plan.sigma.items())[1:]}, pi=plan.pi, mb=plan.mb)
    with pytest.raises(KeyError):
        lower(rpeg, unroll(rpeg, 2), short, p.suite, 2, workload=wl)
    with pytest.raises(NotImplementedError):
        lower(rpeg, unroll(rpeg, 2), plan, p.suite, 2, workload=wl, intra_stage_fusion=True)
    bare = lower(rpeg, unroll(rpeg, 2), ExecutionPlan(sigma=plan.sigma, pi=plan.pi, mb={}), p.suite, 2, workload=wl)
    full = lower(rpeg, unroll(rpeg, 2), plan, p.suite, 2, workload=wl)
    assert [n.id for n in bare.nodes] == [n.id for n in full.nodes] and all(n.mb is None for n in bare.nodes)
    # without a workload nothing is split into quantile phases (lower.py:406-408)
    unsplit = lower(rpeg, unroll(rpeg, 2), plan, p.suite, 2)
    assert not any(":" in n.id for n in unsplit.nodes)


@pytest.mark.gpu
@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_pipeline_call_sequence_equals_reference(names, c):
    """pipeline.py:1015-1017, 1422-1497 through the reference's module names: every recorded digest, the violating
    device of mem_worst_violation included."""
    from model.cost import NodeCostModel
    from model.memory import NodeMemoryModel, _device_peaks, mem_worst_violation
    from passes.lower import lower
    from passes.unroll import unroll
    from schedule.scheduler import schedule
    gen, gold = _generator(), _gold()
    api = dict(unroll=unroll, lower=lower, NodeCostModel=NodeCostModel, schedule=schedule,
               NodeMemoryModel=NodeMemoryModel, _device_peaks=_device_peaks, mem_worst_violation=mem_worst_violation)
    cfg, batch = seeded_batch(c, gold["n_plans"])
    p = cfg.problem
    for i, want in enumerate(gold["configs"][str(c)]):
        rpeg, plan, wl = batch.configuration(p, i)
        shadow = [m for m in rpeg.trainable if rpeg.tau.get(m, 0) > 0]
        got = gen.summary(api, rpeg, plan, wl, p.suite, p.hw, p.device_space, p.K_eval, rpeg.trainable, shadow)
        for key in want:
            assert got[key] == want[key], (c, i, key)


@pytest.mark.gpu
def test_time_of_mock_nodes_and_peak_bytes_equal_the_directory(names):
    """NodeCostModel.time and NodeMemoryModel.peak_bytes of a hand-made operator node (the candidate directory's
    mock node, moves.py:439-485) equal rpeg_op_time_batch's figures, with and without an engine in place."""
    import numpy as np
    from core.types import Allocation
    from model.cost import NodeCostModel
    from model.memory import NodeMemoryModel
    from passes.lower import ExecNode, ExecNodeType
    from passes.unroll import UnrolledNode
    from rpeg_amd.engine.runtime import Engine
    from rpeg_amd.search import evaluate as ev
    cfg, batch = seeded_batch(1, 4)
    p = cfg.problem
    rpeg, plan, wl = batch.configuration(p, 0)
    eng = Engine(p)
    saved = dict(ev._engines)
    ev._engines.clear()
    try:
        for slot, v in enumerate(rpeg.vertices):
            dp, pp, tp = plan.pi[v]
            e = plan.sigma[v].extent
            node = ExecNode(id="_approx", kind=ExecNodeType.OP, allocs=(Allocation(origin=(0, 0, 0), extent=e),),
                            op=UnrolledNode(template_vertex=v, k=0), model=v.kind.model, pi=plan.pi[v], mb=plan.mb[v])
            t, pk = eng.op_time(0, slot, np.array([[dp], [pp], [tp], [plan.mb[v]], [e[0]], [e[1]], [e[2]]], np.int16))
            assert NodeCostModel(p.hw, p.suite, wl).time(node) == t[0]
            assert NodeMemoryModel(p.hw, p.suite, wl).peak_bytes(node) == pk[0]
    finally:
        ev._engines.clear()
        ev._engines.update(saved)
        eng.close()
