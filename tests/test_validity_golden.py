"""The gate functions of RPEG/search/evaluate.py against the reference's OWN verdicts
(tests/golden/ref_validity.json, written by tests/golden/make_golden_validity.py from the part of that
file that parses): is_compatible, allocations_overlap, stale_publication_layout_valid, is_valid,
evaluation_cache_key and the score / feasibility of evaluate_cached, on seeded plans of all five
configurations and on the same plans broken one rule at a time.  Checked here for the Python oracle, the
host build of the kernels' gate and the key text of the drop-in; tests/test_gpu_parity.py checks the GPU."""

import json
import os
import zlib

import numpy as np
import pytest

from oracle import rpeg_oracle as O
from oracle.cpu_port import CpuPort
from rpeg_amd.engine import abi
from rpeg_amd.engine.problem import PlanBatch
from tests.golden.make_golden_validity import validity_cases

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ref_validity.json")


def load():
    with open(GOLD) as f:
        return json.load(f)


def oracle_is_valid(p, rpeg, plan, wl):
    """is_valid (evaluate.py:143-232) on the oracle's passes, with the memory model evaluate_cached builds."""
    if not O.plan_structurally_valid(rpeg, plan, p.device_space, p.suite, wl):
        return False
    if not O.stale_publication_layout_valid(rpeg, plan):
        return False
    nodes, _ = O.lower(rpeg, plan, p.suite, 1, wl)
    mm = O.make_mem_model(rpeg, p.suite, wl, p.hw, p.memory_policy)
    return not (max(O.device_peaks(nodes, mm).values()) > mm.capacity())


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_oracle_gates_equal_reference(c):
    rows = load()["configs"][str(c)]
    cfg, batch, cases = validity_cases(c)
    p = cfg.problem
    assert len(rows) == len(cases)
    seen = dict(valid=0, invalid=0, stale=0, scored=0)
    for want, (i, rule, rpeg, plan, wl) in zip(rows, cases):
        assert (want["plan"], want["rule"]) == (i, rule)
        verts = list(rpeg.vertices)
        assert [O.is_compatible(plan.sigma[v], plan.pi[v], p.device_space) for v in verts] == want["compatible"], (i, rule)
        overlap = 0
        for x, u in enumerate(verts):
            for y, w in enumerate(verts):
                if O.allocations_overlap(plan.sigma[u], plan.sigma[w]):
                    overlap |= 1 << (8 * x + y)
        assert overlap == want["overlap"], (i, rule)
        assert O.stale_publication_layout_valid(rpeg, plan) == want["stale_ok"], (i, rule)
        assert oracle_is_valid(p, rpeg, plan, wl) == want["is_valid"], (i, rule)
        seen["valid" if want["is_valid"] else "invalid"] += 1
        seen["stale"] += not want["stale_ok"]
        if "score" in want:
            got = O.evaluate_plan(rpeg, plan, p.device_space, p.suite, wl, p.hw, p.K_eval, p.memory_policy,
                                  check_stale=True)
            assert float(got["score"]).hex() == want["score"] and got["feasible"] == want["feasible"], (i, rule)
            seen["scored"] += 1
    assert seen["valid"] and seen["invalid"] and seen["stale"] and seen["scored"]


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_host_build_mask_equals_reference(c):
    """The kernels' gate (plan_valid, stale_layout_ok, memory fit: rpeg_core.h / rpeg_plan.h) compiled for the
    host: mask bits against the reference's is_valid and stale rule, scores against evaluate_cached."""
    rows = load()["configs"][str(c)]
    cfg, batch, cases = validity_cases(c)
    p = cfg.problem
    b = PlanBatch.empty(len(cases))
    for k, (i, rule, rpeg, plan, wl) in enumerate(cases):
        b.head[:, k] = batch.head[:, i]
        b.set_plan(k, int(batch.head[0, i]), int(batch.head[1, i]), [], rpeg, plan)
    port = CpuPort(p)
    scored = port.eval(b, flags=abi.GATE_STALE, threads=2)
    import dataclasses
    one = CpuPort(dataclasses.replace(p, K_eval=1)).eval(b, flags=abi.GATE_STALE, threads=2)   # is_valid lowers one step
    for k, want in enumerate(rows):
        m1 = int(one["mask"][k])
        got_valid = bool(m1 & abi.MASK_VALID) and bool(m1 & abi.MASK_STALE_OK) and bool(m1 & abi.MASK_MEM_OK)
        assert got_valid == want["is_valid"], (k, want["plan"], want["rule"])
        if m1 & abi.MASK_VALID:
            assert bool(m1 & abi.MASK_STALE_OK) == want["stale_ok"], k
        if "score" in want and int(scored["mask"][k]) & abi.MASK_VALID:
            assert float(scored["score"][k]).hex() == want["score"], k
            feasible = bool(scored["mask"][k] & abi.MASK_MEM_OK) and bool(scored["mask"][k] & abi.MASK_STALE_OK)
            assert feasible == want["feasible"], k


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_cache_key_text_equals_reference(c):
    from rpeg_amd.search.evaluate import Configuration, evaluation_cache_key
    rows = load()["configs"][str(c)]
    cfg, batch, cases = validity_cases(c)
    p = cfg.problem
    for want, (i, rule, rpeg, plan, wl) in zip(rows, cases):
        key = evaluation_cache_key(Configuration(rpeg, plan, p.device_space), p.memory_policy)
        assert zlib.crc32(key.encode()) == want["key_crc"], (i, rule)
