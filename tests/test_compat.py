"""The import-path drop-in (rpeg_amd.compat): the names a call site written for the reference imports."""

import sys

import pytest

import rpeg_amd.compat as compat

# the modules and names the reference's optimizer and pipeline import from the packages this repository mirrors
# (RPEG/search/optimizer.py:16-29, pipeline.py:41-60)
WANTED = {
    "core.types": ["packing_geometry", "Allocation", "DeviceSpace", "Model", "Role", "TemplateVertex"],
    "ir.plan": ["ExecutionPlan"],
    "ir.rpeg": ["RPEG"],
    "ir.ppo": ["build_PPO_RPEG"],
    "ir.grpo": ["build_GRPO_RPEG"],
    "ir.dpo": ["build_DPO_RPEG"],
    "ir.serialize": ["save_plan"],
    "model.cost": ["NodeCostModel"],
    "model.hardware": ["Hardware"],
    "model.memory": ["MemoryPolicy", "NodeMemoryModel", "_device_peaks", "mem_worst_violation", "mem_feasible"],
    "passes.unroll": ["unroll", "UnrolledNode"],
    "passes.lower": ["lower", "ExecNodeType", "ExecNode", "ExecutableRPEG"],
    "schedule.scheduler": ["schedule"],
    "schedule.trace": ["Trace"],
    "model.models": ["ModelSuite", "ModelSpec", "Model"],
    "model.workload": ["Workload"],
    "search.cache": ["EvalCache"],
    "search.evaluate": ["evaluation_cache_key", "evaluate_cached", "is_valid", "_eval_worker", "Configuration", "evaluate"],
    "search.inter_model": ["Iter_inter_model_candidates", "DEFAULT_T_CAND"],
    "search.moves": ["build_candidate_directory", "move_gen", "multi_move_pair", "sample_expl", "MoveStats"],
    "search.optimizer": ["optimize", "polish", "OptimizerConfig"],
}
NOT_MIRRORED = ["passes.transfer_resources", "runtime.job_plan"]


@pytest.fixture
def names():
    compat.install()
    yield
    compat.uninstall()
    assert not any(n in sys.modules for n in compat.PACKAGES + compat.MODULES)


def test_reference_import_statements_resolve_to_this_package(names):
    for module, wanted in WANTED.items():
        scope = {}
        exec(f"from {module} import {', '.join(wanted)}", scope)
        real = sys.modules["rpeg_amd." + module]
        for name in wanted:
            assert scope[name] is getattr(real, name), (module, name)
    import search.optimizer
    import rpeg_amd.search.optimizer
    assert search.optimizer is rpeg_amd.search.optimizer      # one module object: module switches are shared
    import search.moves
    assert search.moves.ABLATION_FIXED_MB is False
    for module in NOT_MIRRORED:
        with pytest.raises(ModuleNotFoundError):
            exec(f"import {module}", {})


def test_install_refuses_to_shadow_and_uninstall_restores():
    import types
    other = types.ModuleType("search")
    sys.modules["search"] = other
    try:
        with pytest.raises(ImportError, match="search"):
            compat.install()
        assert not compat.installed() and sys.modules["search"] is other
        compat.install(force=True)
        import search.cache
        assert search.cache.EvalCache is sys.modules["rpeg_amd.search.cache"].EvalCache
        compat.uninstall()
        assert sys.modules["search"] is other
    finally:
        sys.modules.pop("search", None)


def test_cost_model_record_validates_like_the_reference():
    from rpeg_amd import configs
    from rpeg_amd.model.cost import NodeCostModel
    import dataclasses
    p = configs.config(1).problem
    NodeCostModel(p.hw, p.suite, p.workload)
    with pytest.raises(ValueError, match="optimizer_stage"):
        NodeCostModel(p.hw, p.suite, p.workload, optimizer_stage=3)
    with pytest.raises(ValueError, match="reshard_scale"):
        NodeCostModel(dataclasses.replace(p.hw, reshard_scale=0.0), p.suite, p.workload)


@pytest.mark.gpu
def test_reference_call_sites_run_on_the_engine(names):
    """A call site written for the reference -- cost and memory model records into build_candidate_directory,
    evaluate(), then the proposal functions on its result -- under the reference's module names: the directory
    equals the engine form's, move_gen / multi_move_pair / sample_expl return what the host build of the proposal
    kernels returns for the same stream and masses, and Python's generator seeds them."""
    import random
    import numpy as np
    from core.types import Allocation
    from model.cost import NodeCostModel
    from model.memory import NodeMemoryModel
    from search.evaluate import Configuration, evaluate, is_valid
    from search.moves import MoveStats, build_candidate_directory, move_gen, multi_move_pair, sample_expl
    from oracle.cpu_port import CpuPort
    from rpeg_amd.engine.runtime import Engine
    from rpeg_amd.search import moves as M
    from rpeg_amd.search.optimizer import plan_row
    from tests.helpers import seeded_batch
    cfg, batch = seeded_batch(1, 8)
    p = cfg.problem
    rpeg, plan, wl = batch.configuration(p, 2)
    cost = NodeCostModel(p.hw, p.suite, wl, p.memory_policy.optimizer_stage, p.memory_policy.activation_checkpointing)
    mm = NodeMemoryModel.from_policy(p.hw, p.suite, wl, p.memory_policy, trainable=frozenset(rpeg.trainable))
    table, index = build_candidate_directory(rpeg, p.suite, p.device_space, wl, cost, mm)
    eng = Engine(p)
    table_e, index_e = build_candidate_directory(rpeg, p.suite, p.device_space, wl, eng, 0)
    assert table == table_e and index == index_e and all(len(t) > 10 for t in table.values())

    config = Configuration(rpeg, plan, p.device_space)
    assert is_valid(config, p.suite, wl, mm)
    score, trace, lowered = evaluate(config, p.suite, wl, p.hw, p.K_eval, p.memory_policy)
    mass = M.critical_mass(config, lowered, trace)
    want_mass = eng.eval_mass(batch.slice(2, 3))["mass"][0]
    assert [mass[v] for v in rpeg.vertices] == list(want_mass[:len(rpeg.vertices)])

    port = CpuPort(p)
    arrays = M.directory_arrays(rpeg, table)
    row = plan_row(rpeg, plan)
    for T in (0.3, 0.02):
        random.seed(11)
        key = tuple(random.getrandbits(63) for _ in range(3))
        random.seed(11)
        stats = MoveStats()
        got = move_gen(config, lowered, trace, table, index, 6, 50, T, 0.3, stats)
        want, _, _ = port.sa_propose(M._params_for(None, 0, None, 6, 50, 0.3), arrays, 0, (0,) + key, plan=row,
                                     mass=list(want_mass), T=T)
        assert len(got) == len(want) > 0
        for c, w in zip(got, want):
            assert np.array_equal(plan_row(rpeg, c.plan), w)
            changed = [v for v in rpeg.vertices if (c.plan.pi[v], c.plan.mb[v], c.plan.sigma[v]) !=
                       (plan.pi[v], plan.mb[v], plan.sigma[v])]
            assert len(changed) == 1
        assert stats.n_calls == 1 and stats.n_placement_proposed + stats.n_strategy_proposed == len(got)
        assert "single-vertex" in stats.summary(0, 0, 0)
    random.seed(5)
    key = tuple(random.getrandbits(63) for _ in range(3))
    random.seed(5)
    pair = multi_move_pair(config, p.suite, wl)
    want, _, _ = port.sa_propose(M._params_for(None, 0, None), [], 1, (0,) + key, plan=row)
    assert (pair is None) == (len(want) == 0)
    if pair is not None:
        assert np.array_equal(plan_row(rpeg, pair.plan), want[0])
    v = rpeg.vertices[1]
    random.seed(9)
    key = tuple(random.getrandbits(63) for _ in range(3))
    random.seed(9)
    drawn = sample_expl(v, p.suite, p.device_space, wl)
    want, _, _ = port.sa_propose(M._params_for(None, 0, None), [], 2, (0,) + key, v=1, r_lo=0, r_hi=p.device_space.R)
    assert drawn is not None and len(want) == 1
    f = [int(x) for x in want[0]]
    assert drawn == (Allocation(origin=(f[4], f[5], f[6]), extent=(f[7], f[8], f[9])), (f[0], f[1], f[2]), f[3])
    eng.close()
