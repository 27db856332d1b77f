"""The co-resident sum model of the reference's memory model (RPEG/model/memory.py:706-742: a NodeMemoryModel built
without trainable models) against what the reference's own `_device_peaks`, `mem_feasible` and `is_valid` returned
(tests/golden/make_golden_coresident.py): the Python restatement and the host build of the kernels' arithmetic here,
the GPU engine and the drop-in `is_valid` in the GPU test."""

import dataclasses
import json
import os

import numpy as np
import pytest

from oracle import rpeg_oracle as O
from oracle.cpu_port import CpuPort
from rpeg_amd import configs
from rpeg_amd.engine import abi
from rpeg_amd.model.memory import MemoryPolicy, NodeMemoryModel
from tests.helpers import GOLDEN, seeded_batch


def golden():
    with open(os.path.join(GOLDEN, "ref_coresident.json")) as f:
        return json.load(f)


def coresident_problem(p, pol, K):
    """`p` with every structure's memory view emptied of trainable models."""
    return dataclasses.replace(p, K_eval=K, memory_policy=MemoryPolicy(**pol),
                               structures=tuple(dataclasses.replace(s, memory_trainable=frozenset()) for s in p.structures))


def hexpeak(x):
    return "inf" if x == float("inf") else float(x).hex()


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_restatement_and_host_build_equal_reference(c):
    g = golden()
    rows = g["configs"][str(c)]["rows"]
    cfg, batch = seeded_batch(c, len(rows))
    p = cfg.problem
    for k, pol in enumerate(g["policies"]):
        policy = MemoryPolicy(**pol)
        for name, K in (("k1", 1), ("k", p.K_eval)):
            out = CpuPort(coresident_problem(p, pol, K)).eval(batch, flags=0)
            for i, row in enumerate(rows):
                want = row[k][name]
                assert hexpeak(out["peak"][i]) == want["peak"], (i, pol, name)
                assert bool(out["mask"][i] & abi.MASK_MEM_OK) == want["feasible"], (i, pol, name)
        for i in range(0, len(rows), 5):     # the Python restatement on a fifth of them
            rpeg, plan, wl = batch.configuration(p, i)
            mm = O.MemModel(p.hw, p.suite, wl, trainable=frozenset(), eps_rt=policy.runtime_overhead_fraction,
                            optimizer_stage=policy.optimizer_stage, worker_overhead_bytes=policy.worker_overhead_bytes,
                            semantic_activation_cache_bytes=policy.semantic_activation_cache_bytes,
                            max_worker_groups_per_gpu=policy.max_worker_groups_per_gpu,
                            activation_checkpointing=policy.activation_checkpointing)
            nodes, _ = O.lower(rpeg, plan, p.suite, 1, wl)
            peaks = O.device_peaks(nodes, mm)
            assert hexpeak(max(peaks.values())) == rows[i][k]["k1"]["peak"], (i, pol)
            assert (O.mem_worst_violation(nodes, mm) is None) == rows[i][k]["k1"]["feasible"], (i, pol)


def test_the_two_memory_models_differ():
    """The vectors are not the worker-liveness numbers under another name: on the same plans the two models give
    different peaks."""
    cfg, batch = seeded_batch(1, 48)
    p = cfg.problem
    a = CpuPort(coresident_problem(p, {}, 1)).eval(batch, flags=0)["peak"]
    b = CpuPort(dataclasses.replace(p, K_eval=1)).eval(batch, flags=0)["peak"]
    assert np.mean(a != b) > 0.5


@pytest.mark.gpu
@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_engine_and_is_valid_equal_reference(c):
    from rpeg_amd.engine.runtime import Engine
    from rpeg_amd.search.evaluate import Configuration, is_valid
    g = golden()
    rows = g["configs"][str(c)]["rows"]
    cfg, batch = seeded_batch(c, len(rows))
    p = cfg.problem
    for k, pol in enumerate(g["policies"]):
        for name, K in (("k1", 1), ("k", p.K_eval)):
            eng = Engine(coresident_problem(p, pol, K))
            for out in (eng.eval(batch, gate_stale=False), eng.eval_resident(batch.take(np.tile(np.arange(batch.n), 80)))):
                for i, row in enumerate(rows):     # (the second batch is large enough for the plan-per-lane kernel)
                    assert hexpeak(out["peak"][i]) == row[k][name]["peak"], (i, pol, name)
                    assert bool(out["mask"][i] & abi.MASK_MEM_OK) == row[k][name]["feasible"], (i, pol, name)
            eng.close()
        for i, row in enumerate(rows):
            rpeg, plan, wl = batch.configuration(p, i)
            mm = NodeMemoryModel.from_policy(p.hw, p.suite, wl, MemoryPolicy(**pol))
            assert not mm.trainable
            assert is_valid(Configuration(rpeg, plan, p.device_space), p.suite, wl, mm) == row[k]["is_valid"], (i, pol)
