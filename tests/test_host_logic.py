"""CPU tests of the host side: candidate generator, plan tensors, problem compiler, the evaluate
shims' integer gates and cache key, and that the C-ABI library loads and exports every symbol the
header declares (no compute calls without a GPU)."""

import ctypes
import os
import re

import numpy as np
import pytest

from oracle import rpeg_oracle as oracle
from rpeg_amd import configs
from rpeg_amd.core.types import Allocation, Model, packing_geometry, rectangular_node_layouts
from rpeg_amd.engine import abi
from rpeg_amd.engine.compile import compile_problem, gen_phases
from rpeg_amd.engine.problem import PlanBatch
from rpeg_amd.search import candidates
from rpeg_amd.search.cache import EvalCache, config_hash
from rpeg_amd.search.evaluate import (Configuration, allocations_overlap, evaluation_cache_key, is_compatible,
                                      stale_publication_layout_valid)
from tests.helpers import seeded_batch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_candidates_are_counter_based():
    cfg, full = seeded_batch(2, 512)
    part = candidates.generate(cfg.problem, 100, cfg.tau_choices, seed=42, tag=2, start=300)
    assert np.array_equal(part.vert, full.vert[:, 300:400]) and np.array_equal(part.head, full.head[:, 300:400])
    other = candidates.generate(cfg.problem, 100, cfg.tau_choices, seed=43, tag=2, start=300)
    assert not np.array_equal(other.vert, part.vert)


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_candidates_are_structurally_valid(c):
    cfg, batch = seeded_batch(c, 300)
    p = cfg.problem
    for i in range(300):
        rpeg, plan, wl = batch.configuration(p, i)
        assert oracle.plan_structurally_valid(rpeg, plan, p.device_space, p.suite, wl)
        for v in rpeg.vertices:
            assert is_compatible(plan.sigma[v], plan.pi[v], p.device_space)


def test_mirror_geometry_equals_oracle():
    for G in (2, 4, 8):
        for dp in range(1, 20):
            for pp in range(1, 20):
                for tp in (1, 2, 4, 8):
                    if tp <= G:
                        assert packing_geometry(dp, pp, tp, G) == oracle.packing_geometry(dp, pp, tp, G)
    for n in range(0, 40):
        assert rectangular_node_layouts(n, 4, 8) == oracle.rectangular_node_layouts(n, 4, 8)


def test_plan_batch_roundtrip():
    cfg, batch = seeded_batch(3, 64)
    p = cfg.problem
    again = PlanBatch.empty(64)
    for i in range(64):
        rpeg, plan, wl = batch.configuration(p, i)
        st = p.structures[int(batch.head[0, i])]
        again.set_plan(i, int(batch.head[0, i]), int(batch.head[1, i]), [rpeg.tau[m] for m in st.tau_models], rpeg, plan)
    assert np.array_equal(again.vert, batch.vert) and np.array_equal(again.head, batch.head)


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_problem_compiler_tables(c):
    p = configs.config(c).problem
    P = compile_problem(p)
    assert P.n_struct == len(p.structures) and P.K_eval == p.K_eval
    wl = p.workload
    assert P.score_num == float(p.K_eval * wl.B * wl.K * (wl.S + wl.T))
    for s in range(P.n_struct):
        rpeg = p.template(s)
        cost = oracle.CostModel(p.hw, p.suite, wl)
        for i, v in enumerate(rpeg.vertices):
            node = oracle.XNode("x", oracle.OP, (Allocation((0, 0, 0), (1, 1, 1)),), tpl=v, k=0, model=v.kind.model,
                                pi=(1, 1, 1), mb=1)
            assert P.st[s].vertex[i].unsplit.W == float(cost.work_cost(node))
            assert P.st[s].vertex[i].topo_idx == sorted(x.id for x in rpeg.vertices).index(v.id)
        order = oracle.template_topo_order(rpeg)
        pairs = oracle.within_step_priors(order, rpeg.trainable)
        assert [(P.st[s].pair[k].u, P.st[s].pair[k].v) for k in range(P.st[s].n_pair)] == \
            [(rpeg.vertices.index(u), rpeg.vertices.index(v)) for u, v, _ in pairs]
    for j in range(1, P.n_split):
        ph = gen_phases(p.workload_for(j))
        assert ph == oracle.gen_phases(p.workload_for(j))
        assert P.n_phase[j] == len(ph)


def test_stale_layout_and_overlap_gates():
    p = configs.config(2).problem
    rpeg = p.template(0, [1])
    a, b = Allocation((0, 0, 0), (1, 2, 4)), Allocation((0, 1, 0), (1, 2, 4))
    far = Allocation((2, 0, 0), (1, 2, 4))
    assert allocations_overlap(a, b) and not allocations_overlap(a, far)
    from rpeg_amd.ir.plan import ExecutionPlan
    def plan(g, t):
        sigma = {v: (g if v.id == "g_pi" else t if v.id == "t_pi" else far) for v in rpeg.vertices}
        return ExecutionPlan(sigma=sigma, pi={v: (2, 1, 4) for v in rpeg.vertices}, mb={v: 1 for v in rpeg.vertices})
    assert not stale_publication_layout_valid(Configuration(rpeg, plan(a, b), p.device_space))
    assert stale_publication_layout_valid(Configuration(rpeg, plan(a, far), p.device_space))
    sync = p.template(0, [0])
    assert stale_publication_layout_valid(Configuration(sync, plan(a, b), p.device_space))


def test_cache_key_and_cache():
    cfg, batch = seeded_batch(1, 2)
    p = cfg.problem
    rpeg, plan, _ = batch.configuration(p, 0)
    rpeg2, plan2, _ = batch.configuration(p, 1)
    k1 = evaluation_cache_key(Configuration(rpeg, plan, p.device_space))
    assert re.fullmatch(r"[0-9a-f]{64}:mem:fusion=0:transfer=destination_only,destination_only:2:1:0:0:"
                        r"activation_cache=0:groups=0", k1)
    assert config_hash(rpeg, plan) != config_hash(rpeg2, plan2)
    assert config_hash(rpeg, plan) == config_hash(*batch.configuration(p, 0)[:2])
    cache = EvalCache()
    assert cache.get(k1) is None and k1 not in cache
    cache.put(k1, 1.5, None, True)
    assert cache.get(k1) == (1.5, None, True) and cache.hits == 1 and cache.misses == 1 and cache.size() == 1


def test_library_exports_every_declared_symbol():
    from rpeg_amd.engine import runtime
    header = open(os.path.join(ROOT, "include", "rpeg_eval.h")).read()
    declared = set(re.findall(r"\b(rpeg_[a-z_]+)\s*\(", header))
    assert declared == set(runtime.EXPORTS)
    lib = runtime.load_library()
    for name in declared:
        assert hasattr(lib, name), name


def test_abi_struct_layout_matches_header():
    # sizes the C compiler reports for the header's structs must equal the ctypes mirror
    import subprocess, tempfile
    src = '#include <stdio.h>\n#include "rpeg_eval.h"\nint main(){printf("%zu %zu %zu %zu %zu\\n", sizeof(rpeg_problem_t),' \
          ' sizeof(rpeg_struct_t), sizeof(rpeg_vertex_t), sizeof(rpeg_edge_t), sizeof(rpeg_model_t));return 0;}\n'
    with tempfile.TemporaryDirectory() as d:
        open(os.path.join(d, "s.c"), "w").write(src)
        subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), "-o", os.path.join(d, "s"), os.path.join(d, "s.c")], check=True)
        out = subprocess.run([os.path.join(d, "s")], capture_output=True, text=True, check=True).stdout.split()
    want = [ctypes.sizeof(t) for t in (abi.ProblemT, abi.StructT, abi.VertexT, abi.EdgeT, abi.ModelT)]
    assert [int(x) for x in out] == want


def test_engine_refuses_without_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from rpeg_amd.engine.runtime import Engine, EngineError
    with pytest.raises(EngineError):
        Engine(configs.config(4).problem)


def test_structural_settings_in_reference_order():
    """Iter_inter_model_candidates against what the reference's yields (tests/golden/make_golden_inter_model.py):
    templates, staleness assignments (models ordered by value string, last fastest), the fused settings
    interleaved, AC-share last; and the families optimize() derives from the same rules."""
    import json
    import os
    from rpeg_amd import configs
    from rpeg_amd.core.types import Model
    from rpeg_amd.search.inter_model import Iter_inter_model_candidates
    from rpeg_amd.search.optimizer import OptimizerConfig, _ac_penalty, optimize_families, penalized_score
    from tests.helpers import GOLDEN, family_problem
    with open(os.path.join(GOLDEN, "ref_inter_model.json")) as f:
        g = json.load(f)
    p = configs.config(1).problem
    for name, cand in g["t_cands"].items():
        t_cand = None if cand is None else {Model(m): set(v) for m, v in cand.items()}
        for algorithm in ("ppo", "grpo", "dpo"):
            got = [dict(vertices=[v.id for v in rpeg.vertices], tau=[[m.value, t] for m, t in cfg.tau.items()],
                        ac_share=cfg.ac_share, fused=cfg.intra_stage_fusion, algorithm=cfg.algorithm)
                   for rpeg, cfg in Iter_inter_model_candidates(p.suite, p.workload, t_cand, algorithm=algorithm)]
            assert got == g[f"{name}/{algorithm}"], (name, algorithm)
        # the families of optimize(): the same settings without the fused ones, grouped by template
        fp = family_problem()
        fams = optimize_families(fp, OptimizerConfig(T_cand=t_cand, lambda_ac=0.15), lambda s: [])
        walked = [(prm.structure, tuple(int(prm.tau[k][i]) for i in range(len(fp.structures[prm.structure].tau_models))))
                  for prm, *_ in fams for k in range(prm.n_variants)]
        want = [(int(s["ac_share"]), tuple(t for _, t in s["tau"])) for s in g[f"{name}/ppo"] if not s["fused"]]
        assert walked == want
        assert [f[2] for f in fams] == [1.0, 0.85][:len(fams)] and [f[4] for f in fams] == [None, 2][:len(fams)]
    assert _ac_penalty(3.0, 0.0) == 3.0 and _ac_penalty(3.0, 0.15) == 3.0 * (1.0 - 0.15)
    assert penalized_score(2.0, None, OptimizerConfig(lambda_ac=0.5), False) == 2.0
    assert penalized_score(2.0, None, OptimizerConfig(lambda_ac=0.5), True) == 1.0


def test_cache_key_text_assembled_from_fragments_equals_one_dump():
    """config_hash puts the key text together from per-template fragments; it must be the text one
    json.dumps of the whole payload gives (RPEG/search/cache.py:160-185), for every template and staleness of
    the five configurations, also when two templates alternate."""
    from rpeg_amd.search.cache import _config_hash_plain, config_hash
    from tests.helpers import seeded_batch
    seen = []
    for c in (1, 2, 3, 4, 5):
        cfg, batch = seeded_batch(c, 24)
        for i in range(24):
            rpeg, plan, _ = batch.configuration(cfg.problem, i)
            seen.append((rpeg, plan))
            assert config_hash(rpeg, plan) == _config_hash_plain(rpeg, plan), (c, i)
    for rpeg, plan in seen[::7]:
        assert config_hash(rpeg, plan) == _config_hash_plain(rpeg, plan)
