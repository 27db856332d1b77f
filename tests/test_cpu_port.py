"""The host build of the kernels' arithmetic (oracle/cpu_port.cpp compiles rpeg_amd/csrc/*.h with
g++) against the reference vectors and the Python oracle: this checks the code the GPU runs, on the
CPU, including the class lowering and the heap-free scheduler."""

import numpy as np
import pytest

from oracle import rpeg_oracle as oracle
from oracle.cpu_port import CpuPort, exp_libm
from rpeg_amd.engine import abi
from tests.helpers import load_golden, seeded_batch


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_port_matches_reference_vectors(c):
    gold = load_golden(c)
    cfg, batch = seeded_batch(c, gold["n"])
    out = CpuPort(cfg.problem).eval(batch)
    for i, want in enumerate(gold["plans"]):
        assert float(out["makespan"][i]).hex() == want["makespan"], i
        assert float(out["peak"][i]).hex() == want["peak"], i
        assert float(out["score"][i]).hex() == want["score"], i
        assert bool(out["mask"][i] & abi.MASK_MEM_OK) == want["feasible"], i
        assert out["mask"][i] & abi.MASK_VALID and not out["mask"][i] & abi.MASK_ERROR


@pytest.mark.parametrize("c", [1, 2, 3, 4])
def test_port_matches_oracle_beyond_fixtures(c):
    cfg, batch = seeded_batch(c, 48, start=100_000)
    out = CpuPort(cfg.problem).eval(batch, flags=abi.GATE_STALE)
    for i in range(48):
        rpeg, plan, wl = batch.configuration(cfg.problem, i)
        p = cfg.problem
        want = oracle.evaluate_plan(rpeg, plan, p.device_space, p.suite, wl, p.hw, p.K_eval, p.memory_policy,
                                    check_stale=True)
        assert out["makespan"][i] == want["makespan"] and out["peak"][i] == want["peak"]
        assert out["score"][i] == want["score"]
        assert bool(out["mask"][i] & abi.MASK_STALE_OK) == want["stale_ok"]


def test_port_lowering_equals_oracle_lowering():
    for c in (1, 2, 3, 4):
        cfg, batch = seeded_batch(c, 40)
        p = cfg.problem
        port = CpuPort(p)
        for i in range(40):
            rpeg, plan, wl = batch.configuration(p, i)
            nodes, edges = oracle.lower(rpeg, plan, p.suite, p.K_eval, wl)
            low = port.lower(batch, i)
            kinds = {oracle.OP: 0, oracle.COMM: 1, oracle.RESHARD: 2}
            assert [kinds[n.kind] for n in nodes] == list(low["kind"])
            idx = {n.id: j for j, n in enumerate(nodes)}
            assert [(idx[a.id], idx[b.id]) for a, b in edges] == [tuple(e) for e in low["edges"]]
            cost = oracle.CostModel(p.hw, p.suite, wl)
            assert [cost.time(n) for n in nodes] == list(low["dur"])


def test_exp_equals_libm():
    import math
    rng = np.random.default_rng(7)
    x = np.concatenate([-28.0 * rng.random(200_000), -np.logspace(-12, 1.5, 2000), [0.0, -0.0, -40.0, -64.0]])
    y = exp_libm(x)
    for a, b in zip(x.tolist(), y.tolist()):
        assert math.exp(a) == b


def test_invalid_plans_are_masked():
    cfg, batch = seeded_batch(2, 8)
    batch.vert[0, 1] = 3          # dp = 3 does not divide B
    batch.vert[3, 2] = 5          # mb violates the microbatch rule
    batch.head[1, 3] = 7          # split index out of range
    batch.vert[7, 4] = 99         # extent outside the mesh
    out = CpuPort(cfg.problem).eval(batch)
    assert list(out["mask"][1:5] & abi.MASK_VALID) == [0, 0, 0, 0]
    assert out["mask"][0] & abi.MASK_VALID and np.all(np.isnan(out["score"][1:5]))


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_port_transfer_resource_policies_match_reference(c):
    """The lowering's reserved allocations under the three non-default transfer resource policies: makespans
    of the host build against the reference scheduler's (tests/golden/ref_transfer_policy.json)."""
    from tests.helpers import load_transfer_policy_golden, with_transfer_policy
    gold = load_transfer_policy_golden()
    g = gold["configs"][str(c)]
    cfg, batch = seeded_batch(c, g["n_plans"])
    for k, pol in enumerate(gold["policies"]):
        out = CpuPort(with_transfer_policy(cfg.problem, *pol)).eval(batch)
        for i in range(g["n_plans"]):
            assert float(out["makespan"][i]).hex() == g["rows"][i][k]["makespan"], (i, pol)


@pytest.mark.parametrize("c", [1, 2, 3, 4])
def test_port_memory_policies_match_reference(c):
    """Non-default memory policies on the host build of the kernels' arithmetic against the reference's
    evaluations (tests/golden/ref_memory_policy.json), every plan of the vectors."""
    from tests.helpers import load_memory_policy_golden, with_memory_policy
    gold = load_memory_policy_golden()
    g = gold["configs"][str(c)]
    cfg, batch = seeded_batch(c, g["n_plans"])
    for k, pol in enumerate(gold["policies"]):
        out = CpuPort(with_memory_policy(cfg.problem, pol)).eval(batch)
        for i in range(g["n_plans"]):
            want = g["rows"][i][k]
            assert float(out["makespan"][i]).hex() == want["makespan"], (i, pol)
            assert float(out["peak"][i]).hex() == want["peak"], (i, pol)
            assert float(out["score"][i]).hex() == want["score"], (i, pol)
            assert bool(out["mask"][i] & abi.MASK_MEM_OK) == want["feasible"], (i, pol)


@pytest.mark.parametrize("c", [1, 2, 3, 4])
def test_port_calibrated_hardware_matches_reference(c):
    """Calibrated hardware records on the host build of the kernels' arithmetic against the reference's
    evaluations (tests/golden/ref_hardware.json), every plan of the vectors."""
    from tests.helpers import load_hardware_golden, with_hardware
    gold = load_hardware_golden()
    g = gold["configs"][str(c)]
    cfg, batch = seeded_batch(c, g["n_plans"])
    for k, ov in enumerate(gold["overlays"]):
        out = CpuPort(with_hardware(cfg.problem, ov)).eval(batch)
        for i in range(g["n_plans"]):
            want = g["rows"][i][k]
            assert float(out["makespan"][i]).hex() == want["makespan"], (i, k)
            assert float(out["peak"][i]).hex() == want["peak"], (i, k)
            assert float(out["score"][i]).hex() == want["score"], (i, k)
            assert bool(out["mask"][i] & abi.MASK_MEM_OK) == want["feasible"], (i, k)


def test_port_problems_away_from_the_shipped_configurations_match_reference():
    """The host build on the problems of tests/golden/ref_variants.json, every plan of the vectors."""
    from tests.helpers import variant_cases
    for name, p, batch, rows in variant_cases():
        out = CpuPort(p).eval(batch)
        for i, want in enumerate(rows):
            assert float(out["makespan"][i]).hex() == want["makespan"], (name, i)
            assert float(out["peak"][i]).hex() == want["peak"], (name, i)
            assert float(out["score"][i]).hex() == want["score"], (name, i)
            assert bool(out["mask"][i] & abi.MASK_MEM_OK) == want["feasible"], (name, i)


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_bench_flop_constants_follow_a_fresh_count(c):
    """bench.py prices its FP64 roofline with operation counts frozen from oracle/flop_count.cpp: a fresh
    count over the first 4,096 seeded plans stays within 3 % of them (the frozen ones are whole-set means)."""
    import bench
    from oracle.cpu_port import count_flops
    cfg, batch = seeded_batch(c, 4096)
    got = count_flops(cfg.problem, batch)
    assert got["plans"] == 4096
    assert abs(got["total"] - bench.ALG_FLOPS[c]) <= 0.03 * bench.ALG_FLOPS[c], (got, bench.ALG_FLOPS[c])
    # the count is dominated by the scheduler's comparisons, as the kernels' instruction mix is
    assert got["cmp"] > got["add"] + got["mul"] + got["div"]


@pytest.mark.parametrize("c,K", [(1, 100), (2, 100), (4, 128)])
def test_port_matches_oracle_at_long_horizons(c, K):
    """Horizons as the runtime's planner asks for them (runtime/job_plan.py:170-214): the host build of the kernels'
    arithmetic against the Python restatement on graphs of 800-3,000 lowered nodes (for DPO with 128 entries ready at
    once: the host build's list is not bounded as the GPU's is)."""
    import dataclasses
    cfg, batch = seeded_batch(c, 6, start=300_000)
    p = dataclasses.replace(cfg.problem, K_eval=K)
    out = CpuPort(p).eval(batch, flags=abi.GATE_STALE)
    n_checked = 0
    for i in range(6):
        if not out["mask"][i] & abi.MASK_VALID:
            continue
        rpeg, plan, wl = batch.configuration(p, i)
        want = oracle.evaluate_plan(rpeg, plan, p.device_space, p.suite, wl, p.hw, K, p.memory_policy, check_stale=True)
        assert out["makespan"][i] == want["makespan"] and out["peak"][i] == want["peak"] and out["score"][i] == want["score"], i
        n_checked += 1
    assert n_checked >= 2
