"""The Python oracle against vectors written by the reference implementation itself
(tests/golden/make_golden.py): bit-exact makespan, raw score, worst device peak, penalised
score, feasibility, lowered graph size, dispatch order, mean device utilisation and number of active
devices."""

import math

import pytest

from oracle import rpeg_oracle as oracle
from tests.helpers import load_golden, oracle_eval, order_crc, seeded_batch


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_plans_match_reference(c):
    gold = load_golden(c)
    cfg, batch = seeded_batch(c, gold["n"])
    import zlib
    assert zlib.crc32(batch.vert.tobytes()) == gold["vert_crc"], "seeded candidate set changed"
    assert zlib.crc32(batch.head.tobytes()) == gold["head_crc"]
    step = 1 if c in (1, 4) else 2   # keep the CPU suite short; every plan of the small configs
    for i in range(0, gold["n"], step):
        want = gold["plans"][i]
        got = oracle_eval(cfg.problem, batch, i, want_trace=True)
        assert len(got["nodes"]) == want["n_nodes"], i
        assert len(got["edges"]) == want["n_edges"], i
        assert order_crc(got["order"]) == want["order_crc"], i
        assert got["makespan"].hex() == want["makespan"], i
        assert got["raw"].hex() == want["raw"], i
        assert float(got["peak"]).hex() == want["peak"], i
        assert got["feasible"] == want["feasible"], i
        assert got["score"].hex() == want["score"], i
        assert math.fsum(got["finish"].values()).hex() == want["finish_sum"], i
        if i % 4 == 0:   # Trace.utilization / Trace.n_active of the reference's own trace
            reserved = oracle.reserved_by_node(got["nodes"], got["edges"])
            util = oracle.utilization(got["start"], got["finish"], got["order"], reserved)
            assert float(util).hex() == want["utilization"], i
            assert oracle.n_active(got["nodes"]) == want["n_active"], i


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_node_times_and_peaks_match_reference(c):
    gold = load_golden(c)
    cfg, batch = seeded_batch(c, len(gold["nodes"]))
    p = cfg.problem
    for i, recs in enumerate(gold["nodes"]):
        rpeg, plan, wl = batch.configuration(p, i)
        nodes, _ = oracle.lower(rpeg, plan, p.suite, p.K_eval, wl)
        by_id = {n.id: n for n in nodes}
        cost = oracle.CostModel(p.hw, p.suite, wl)
        mm = oracle.make_mem_model(rpeg, p.suite, wl, p.hw, p.memory_policy)
        for rec in recs:
            n = by_id[rec["id"]]
            assert cost.time(n).hex() == rec["time"], (i, rec["id"])
            if n.kind == oracle.OP:
                assert float(mm.peak_bytes(n)).hex() == rec["peak_bytes"], (i, rec["id"])
                assert [x.hex() for x in cost.breakdown(n)] == rec["breakdown"], (i, rec["id"])


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_transfer_resource_policies_match_reference(c):
    """Schedules under the three non-default transfer resource policies against the reference scheduler's
    (tests/golden/make_golden_transfer_policy.py): makespan, dispatch order, finish times, utilisation."""
    from tests.helpers import load_transfer_policy_golden
    gold = load_transfer_policy_golden()
    g = gold["configs"][str(c)]
    assert g["n_differ_from_default"] > 0
    cfg, batch = seeded_batch(c, g["n_plans"])
    for i in range(0, g["n_plans"], 1 if c in (1, 4) else 3):
        for pol, want in zip(gold["policies"], g["rows"][i]):
            got = oracle_eval(cfg.problem, batch, i, want_trace=True, transfer_policy=tuple(pol))
            assert got["makespan"].hex() == want["makespan"], (i, pol)
            assert order_crc(got["order"]) == want["order_crc"], (i, pol)
            assert math.fsum(got["finish"].values()).hex() == want["finish_sum"], (i, pol)
            reserved = oracle.reserved_by_node(got["nodes"], got["edges"], tuple(pol))
            util = oracle.utilization(got["start"], got["finish"], got["order"], reserved)
            assert float(util).hex() == want["utilization"], (i, pol)


@pytest.mark.parametrize("c", [1, 2, 3, 4])
def test_memory_policies_match_reference(c):
    """Optimizer stages 0-2, checkpointing off, runtime overhead fraction, per-worker overhead and cache bytes
    and the worker-group limit (inf peaks) against the reference's evaluations
    (tests/golden/make_golden_memory_policy.py): makespan, worst peak, feasibility, penalised score."""
    from tests.helpers import load_memory_policy_golden, with_memory_policy
    gold = load_memory_policy_golden()
    g = gold["configs"][str(c)]
    cfg, batch = seeded_batch(c, g["n_plans"])
    for k, pol in enumerate(gold["policies"]):
        p = with_memory_policy(cfg.problem, pol)
        for i in range(0, g["n_plans"], 1 if c in (1, 4) else 3):
            want = g["rows"][i][k]
            got = oracle_eval(p, batch, i)
            assert got["makespan"].hex() == want["makespan"], (i, pol)
            assert float(got["peak"]).hex() == want["peak"], (i, pol)
            assert got["feasible"] == want["feasible"] and got["score"].hex() == want["score"], (i, pol)


@pytest.mark.parametrize("c", [1, 2, 3, 4])
def test_calibrated_hardware_matches_reference(c):
    """Per-role operator scales, weight-transfer and reshard scales, the fixed activation-transfer overhead,
    gemm_k_half and other link / efficiency parameters against the reference's evaluations
    (tests/golden/make_golden_hardware.py): makespan, dispatch order, worst peak, feasibility, score."""
    from tests.helpers import load_hardware_golden, with_hardware
    gold = load_hardware_golden()
    g = gold["configs"][str(c)]
    cfg, batch = seeded_batch(c, g["n_plans"])
    for k, ov in enumerate(gold["overlays"]):
        p = with_hardware(cfg.problem, ov)
        for i in range(0, g["n_plans"], 1 if c in (1, 4) else 3):
            want = g["rows"][i][k]
            got = oracle_eval(p, batch, i, want_trace=True)
            assert got["makespan"].hex() == want["makespan"], (i, k)
            assert order_crc(got["order"]) == want["order_crc"], (i, k)
            assert float(got["peak"]).hex() == want["peak"], (i, k)
            assert got["feasible"] == want["feasible"] and got["score"].hex() == want["score"], (i, k)


def test_problems_away_from_the_shipped_configurations_match_reference():
    """PPO and GRPO without generation quantiles, one and six quantiles, K > 1, meshes with 2 and 8 devices per
    node, 4-byte elements, another head size, a stated parameter count: the reference's evaluations
    (tests/golden/make_golden_variants.py) -- graph size, dispatch order, makespan, peak, feasibility, score."""
    from tests.helpers import variant_cases
    for name, p, batch, rows in variant_cases():
        for i in range(0, len(rows), 2):
            want = rows[i]
            got = oracle_eval(p, batch, i, want_trace=True)
            assert (len(got["nodes"]), len(got["edges"])) == (want["n_nodes"], want["n_edges"]), (name, i)
            assert order_crc(got["order"]) == want["order_crc"], (name, i)
            assert got["makespan"].hex() == want["makespan"], (name, i)
            assert float(got["peak"]).hex() == want["peak"], (name, i)
            assert got["feasible"] == want["feasible"] and got["score"].hex() == want["score"], (name, i)
