"""Drop-in evaluation calls: same names, arguments, return shapes and error behaviour as
RPEG/search/evaluate.py, computed by the GPU engine.

  evaluate(config, suite, workload, hw, K_eval, memory_policy)          -> (score, trace, lowered)
  evaluate_cached(config, cache, suite, workload, hw, K_eval, policy)   -> (score, trace, feasible, miss)
  _eval_worker((config, suite, workload, hw, K_eval[, policy]))         -> (score, trace, feasible)
  is_valid(config, suite, workload, mem_model)                          -> bool
  evaluate_batch(configs, suite, workload, hw, K_eval, policy)          -> BatchResult   (new: the
      batched form of Pool.map(_eval_worker, ...), RPEG/search/optimizer.py:793-798)

The integer gates (`is_compatible`, `allocations_overlap`, `stale_publication_layout_valid`, the
integer part of `is_valid`) are host code as in the reference.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from ..core.types import (Allocation, DeviceSpace, RPEG_TRANSFER_RESOURCE_POLICY, TransferResourcePolicy,
                          packing_geometry, rectangular_node_layouts)
from ..engine import abi
from ..engine.problem import STRUCTURES, EvalProblem, PlanBatch
from ..ir.plan import ExecutionPlan
from ..ir.rpeg import RPEG
from ..model.hardware import Hardware
from ..model.memory import MemoryPolicy, NodeMemoryModel
from ..model.models import ModelSuite
from ..model.workload import Workload
from ..passes.lower import ExecEdge, ExecNode, ExecNodeType, ExecutableRPEG, lower   # noqa: F401  (re-exported)
from ..schedule.trace import Trace   # noqa: F401  (re-exported: the reference's evaluate module names it)
from .cache import EvalCache, config_hash

_OOM_BETA = 40.0
ABLATION_HARD_OOM = False


class EngineLimitError(RuntimeError):
    """A plan the reference would evaluate exceeds a limit of this engine (RPEG_MASK_LIMIT)."""



@dataclass
class Configuration:
    rpeg: RPEG
    plan: ExecutionPlan
    device_space: DeviceSpace
    intra_stage_fusion: bool = False
    transfer_resource_policy: Optional[TransferResourcePolicy] = None


def is_compatible(alloc: Allocation, pi: Tuple[int, int, int], device_space: DeviceSpace) -> bool:
    """Placement feasibility under nested 3D parallelism with stage packing (evaluate.py:50-94)."""
    dp, pp, tp = pi
    if tp > device_space.G:
        return False
    geom = packing_geometry(dp, pp, tp, device_space.G)
    if geom is None or alloc.extent[2] != geom[0]:
        return False
    if tuple(alloc.extent[:2]) not in rectangular_node_layouts(geom[1], device_space.R, device_space.N):
        return False
    bounds = (device_space.R, device_space.N, device_space.G)
    return all(o >= 0 and o + e <= b for o, e, b in zip(alloc.origin, alloc.extent, bounds))


def allocations_overlap(left: Allocation, right: Allocation) -> bool:
    return all(left.origin[k] < right.origin[k] + right.extent[k] and right.origin[k] < left.origin[k] + left.extent[k]
               for k in range(3))


def stale_publication_layout_valid(config: Configuration) -> bool:
    """Every publication with a positive staleness budget needs disjoint endpoints (evaluate.py:115-140)."""
    for e in config.rpeg.pub_edges:
        if int(config.rpeg.tau.get(e.src.kind.model, 0)) > 0 and \
                allocations_overlap(config.plan.sigma[e.src], config.plan.sigma[e.dst]):
            return False
    return True


# ----------------------------------------------------------------------------- engine plumbing
_engines: Dict[tuple, object] = {}   # insertion-ordered: least recently used first
_MAX_ENGINES = 16


def _structure_of(rpeg: RPEG):
    ids = tuple(v.id for v in rpeg.vertices)
    for st in STRUCTURES.values():
        # every shipped template has a distinct vertex-id tuple
        if ids == _TEMPLATE_IDS[st.name]:
            return st
    raise ValueError(f"unsupported template graph with vertices {ids}")


_TEMPLATE_IDS = {"ppo": ("g_pi", "i_ref", "i_R", "i_V", "t_pi", "t_V"), "grpo": ("g_pi", "i_ref", "i_R", "t_pi"),
                 "dpo": ("i_pi", "i_ref", "t_pi"), "ac_share": ("g_ac", "i_ref", "i_R", "i_ac", "t_ac")}


def _engine_for(rpeg: RPEG, suite: ModelSuite, workload: Workload, hw: Hardware, space: DeviceSpace, K_eval: int,
                policy: MemoryPolicy, more_structures=(), memory_trainable=None, transfer_policy=None):
    """(engine, structure of `rpeg`): one engine per problem, kept for the life of the process.  The
    structure of `rpeg` is structure 0 of the engine (with `memory_trainable` as the memory model's set of
    trainable models when that is given and differs from the template's), `more_structures` follow.
    `transfer_policy` (a TransferResourcePolicy, None = the default) is part of the problem: it decides
    which allocations the lowered transfers reserve."""
    from dataclasses import replace
    from ..engine.runtime import Engine
    st = _structure_of(rpeg)
    if memory_trainable is not None and frozenset(memory_trainable) != frozenset(st.tau_models):
        st = replace(st, memory_trainable=frozenset(memory_trainable))
    structures = (st,) + tuple(more_structures)
    transfer_policy = transfer_policy or RPEG_TRANSFER_RESOURCE_POLICY
    rest = (tuple(sorted((m.value, s) for m, s in suite.specs.items())), workload, hw, space, K_eval, policy,
            transfer_policy)
    key = (tuple((s.name, s.memory_trainable) for s in structures),) + rest
    alias = ((st.name, st.memory_trainable), "first") + rest
    hit = key if key in _engines else alias if not more_structures and alias in _engines else None
    if hit is not None:
        # (an engine that holds this template as structure 0 beside others serves as well, and keeps its classes)
        eng = _engines.pop(hit)
        _engines[hit] = eng          # most recently used last
        return eng, st
    problem = EvalProblem(structures=structures, suite=suite, workload=workload, hw=hw, device_space=space,
                          K_eval=K_eval, memory_policy=policy, transfer_resource_policy=transfer_policy)
    eng = _engines[key] = Engine(problem)
    _engines.setdefault(alias, eng)
    while len(_engines) > _MAX_ENGINES:      # a long-lived process that sees many problems keeps the recent ones;
        _engines.pop(next(iter(_engines)))   # an engine frees its device memory when its last holder lets go
    return eng, st


def _engine_like(rpeg, space: Optional[DeviceSpace], suite=None, workload=None, vertex=None, hw=None, policy=None):
    """The most recently used engine that holds the template of `rpeg` as a structure on device space `space`
    (any space when that is None; and, when given, for these models, this workload, this hardware record and this
    (optimizer stage, activation checkpointing) pair), with the index of that structure -- for calls of the
    reference's API that name neither the hardware nor the horizon (the proposal functions of search.moves),
    whose results depend on neither.  With `vertex` in place of `rpeg`: an engine with a template that holds that
    vertex, the structure and the vertex's slot in it."""
    want = None if rpeg is None else _structure_of(rpeg).name
    for eng in reversed(list(_engines.values())):
        p = eng.problem
        if (space is not None and p.device_space != space) or (suite is not None and p.suite.specs != suite.specs) or \
                (workload is not None and p.workload != workload) or (hw is not None and p.hw != hw) or \
                (policy is not None and (p.memory_policy.optimizer_stage, p.memory_policy.activation_checkpointing) != tuple(policy)):
            continue
        for k, st in enumerate(p.structures):
            if vertex is not None:
                ids = [v.id for v in p.template(k, ()).vertices]
                if vertex.id in ids and st.memory_trainable is None:
                    return eng, k, ids.index(vertex.id)
            elif st.name == want and st.memory_trainable is None:
                return eng, k
    raise LookupError("no evaluation engine for this template and device space yet: evaluate a configuration of it "
                      "(evaluate, evaluate_cached, evaluate_batch) before asking for proposals")


def _engine_space_for(rpeg, plan, suite, workload, hw) -> DeviceSpace:
    """A device space for calls of the reference's API that name none (NodeCostModel.time, mem_worst_violation):
    node durations and device peaks do not depend on it, only the engine's validity gate does.  The space of the
    most recently used engine for this template, these models, workload and hardware under which every vertex of
    the plan is placed validly; else the smallest space that encloses the plan, with the devices per node for which
    the plan's packing is valid."""
    def fits(space):
        return all(is_compatible(plan.sigma[v], plan.pi[v], space) for v in rpeg.vertices)
    want = _structure_of(rpeg).name
    for eng in reversed(list(_engines.values())):
        p = eng.problem
        if p.suite.specs == suite.specs and p.workload == workload and p.hw == hw and \
                any(st.name == want for st in p.structures) and fits(p.device_space):
            return p.device_space
    R = max(plan.sigma[v].origin[0] + plan.sigma[v].extent[0] for v in rpeg.vertices)
    N = max(plan.sigma[v].origin[1] + plan.sigma[v].extent[1] for v in rpeg.vertices)
    g_lo = max(plan.sigma[v].origin[2] + plan.sigma[v].extent[2] for v in rpeg.vertices)
    for G in range(g_lo, 8 * g_lo + 1):
        if fits(DeviceSpace(R=R, N=N, G=G)):
            return DeviceSpace(R=R, N=N, G=G)
    raise ValueError("the plan's allocations are no valid packing on any device space")


def _check_supported(config: Configuration):
    if config.intra_stage_fusion:
        raise NotImplementedError("intra_stage_fusion=True is not evaluated by this engine")


def _pack(configs: Sequence[Configuration], st, workload: Workload) -> PlanBatch:
    batch = PlanBatch.empty(len(configs))
    split = 1 if workload.gen_quantiles else 0
    for i, cfg in enumerate(configs):
        for v in cfg.rpeg.vertices:  # a missing vertex raises KeyError as lower() does (lower.py:447-451)
            cfg.plan.sigma[v], cfg.plan.pi[v]
        taus = [int(cfg.rpeg.tau[m]) for m in st.tau_models]
        plan = cfg.plan
        if any(v not in plan.mb for v in cfg.rpeg.vertices):
            raise KeyError("plan.mb misses a template vertex")
        batch.set_plan(i, 0, split, taus, cfg.rpeg, plan)
    return batch


@dataclass
class BatchResult:
    score: np.ndarray      # evaluate_cached semantics (0 where the stale-layout rule fails)
    makespan: np.ndarray
    peak: np.ndarray
    mask: np.ndarray
    feasible: np.ndarray   # memory-feasible and stale-layout valid
    util: Optional[np.ndarray] = None   # Trace.utilization() per configuration, when asked for


def evaluate_batch(configs: Sequence[Configuration], suite: ModelSuite, workload: Workload, hw: Hardware,
                   K_eval: int, memory_policy: MemoryPolicy = MemoryPolicy(), gate_stale: bool = True,
                   with_util: bool = False) -> BatchResult:
    """Scores many configurations of ONE template structure in one GPU launch.  `with_util`: also
    Trace.utilization() of each (trace.py:53-101) from the same launch, 1,024 configurations at a time."""
    if not configs:
        z = np.zeros(0)
        return BatchResult(z, z, z, np.zeros(0, np.uint8), np.zeros(0, bool))
    for c in configs:
        _check_supported(c)
    pol = configs[0].transfer_resource_policy or RPEG_TRANSFER_RESOURCE_POLICY
    if any((c.transfer_resource_policy or RPEG_TRANSFER_RESOURCE_POLICY) != pol for c in configs):
        raise ValueError("the configurations of one batch must share their transfer resource policy")
    eng, st = _engine_for(configs[0].rpeg, suite, workload, hw, configs[0].device_space, K_eval, memory_policy,
                          transfer_policy=pol)
    batch = _pack(configs, st, workload)
    if with_util:
        out = eng.eval_util(batch, gate_stale=gate_stale)
    else:
        out = eng.eval(batch, gate_stale=gate_stale)
    mask = out["mask"]
    if np.any((mask & abi.MASK_VALID) == 0):
        raise ValueError("a configuration violates the integer validity rules of is_valid")
    if np.any(mask & abi.MASK_LIMIT):
        raise EngineLimitError("a configuration exceeds a limit of the evaluation engine: it was not evaluated")
    if np.any(mask & abi.MASK_ERROR):
        raise ZeroDivisionError("a configuration has a degenerate node duration or makespan")
    feasible = ((mask & abi.MASK_MEM_OK) != 0) & ((mask & abi.MASK_STALE_OK) != 0)
    score = out["score"].copy()
    if ABLATION_HARD_OOM:
        score[(mask & abi.MASK_MEM_OK) == 0] = 0.0
    return BatchResult(score, out["makespan"], out["peak"], mask, feasible, out.get("util"))


# ----------------------------------------------------------------------------- trace objects
def _trace_of(eng, st, config: Configuration, batch: PlanBatch, workload=None, suite=None, lowered=None):
    """(Trace, ExecutableRPEG) of the one plan of `batch`: the lowered graph (passes.lower.lower) and the engine's
    start / finish time, dispatch position and reserved vertices of every node of it."""
    from ..schedule.scheduler import trace_on
    if lowered is None:
        lowered = lower(config.rpeg, None, config.plan, suite if suite is not None else eng.problem.suite,
                        eng.problem.K_eval, workload=workload if workload is not None else eng.problem.workload)
    return trace_on(eng, lowered, batch), lowered


# ----------------------------------------------------------------------------- reference API
def evaluate(config: Configuration, suite: ModelSuite, workload: Workload, hw: Hardware, K_eval: int,
             memory_policy: MemoryPolicy = MemoryPolicy()):
    """unroll -> lower -> cost -> schedule -> score of one configuration (evaluate.py:235-290);
    returns (score, trace, lowered)."""
    _check_supported(config)
    eng, st = _engine_for(config.rpeg, suite, workload, hw, config.device_space, K_eval, memory_policy,
                          transfer_policy=config.transfer_resource_policy)
    batch = _pack([config], st, workload)
    trace, lowered = _trace_of(eng, st, config, batch, workload, suite)
    score = trace.throughput(W_step=workload.B * workload.K * (workload.S + workload.T), K=K_eval)
    return score, trace, lowered


def is_valid(config: Configuration, suite: ModelSuite, workload: Workload, mem_model: NodeMemoryModel) -> bool:
    """Drop-in for is_valid (RPEG/search/evaluate.py:143-232): plan coverage, divisibility, micro-batch and
    packing rules, the stale-publication layout rule, and memory fit of the K_eval = 1 lowering under
    `mem_model` -- whose set of trainable models need not be the template's (optimize() passes the model of
    its base configuration).  Coverage is checked here; everything else is the mask of one engine call."""
    _check_supported(config)
    plan = config.plan
    for v in config.rpeg.vertices:
        if v not in plan.sigma or v not in plan.pi or v not in plan.mb:
            return False
    # (a memory model without trainable models is the reference's co-resident sum model, memory.py:706-742)
    eng, st = _engine_for(config.rpeg, suite, workload, mem_model.hw, config.device_space, 1, mem_model.policy,
                          memory_trainable=mem_model.trainable)
    mask = int(eng.eval(_pack([config], st, workload), gate_stale=False)["mask"][0])
    return bool(mask & abi.MASK_VALID) and bool(mask & abi.MASK_STALE_OK) and bool(mask & abi.MASK_MEM_OK)


def evaluation_cache_key(config: Configuration, memory_policy: MemoryPolicy = MemoryPolicy()) -> str:
    """Same key text as evaluate.py:301-326."""
    pol = config.transfer_resource_policy or RPEG_TRANSFER_RESOURCE_POLICY
    return (f"{config_hash(config.rpeg, config.plan)}:mem:"
            f"fusion={int(config.intra_stage_fusion)}:"
            f"transfer={','.join(pol.to_dict().values())}:"
            f"{memory_policy.optimizer_stage}:"
            f"{int(memory_policy.activation_checkpointing)}:"
            f"{memory_policy.runtime_overhead_fraction:.12g}:"
            f"{memory_policy.worker_overhead_bytes:.12g}:"
            f"activation_cache={memory_policy.semantic_activation_cache_bytes:.12g}:"
            f"groups={memory_policy.max_worker_groups_per_gpu}")


def _score_one(config, suite, workload, hw, K_eval, memory_policy, gate_stale):
    _check_supported(config)
    eng, st = _engine_for(config.rpeg, suite, workload, hw, config.device_space, K_eval, memory_policy,
                          transfer_policy=config.transfer_resource_policy)
    batch = _pack([config], st, workload)
    res = evaluate_batch([config], suite, workload, hw, K_eval, memory_policy, gate_stale=gate_stale)
    trace, _ = _trace_of(eng, st, config, batch, workload, suite)
    return float(res.score[0]), trace, res


def evaluate_cached(config: Configuration, cache: EvalCache, suite: ModelSuite, workload: Workload, hw: Hardware,
                    K_eval: int, memory_policy: MemoryPolicy = MemoryPolicy()):
    """Cache lookup, then evaluation with the soft OOM penalty; a plan whose positive-lag
    publication endpoints intersect scores 0 and is infeasible (evaluate.py:329-403).
    Returns (score, trace, feasible, miss)."""
    h = evaluation_cache_key(config, memory_policy)
    if h in cache:
        score, trace, feasible = cache.get(h)
        return score, trace, feasible, False
    score, trace, res = _score_one(config, suite, workload, hw, K_eval, memory_policy, gate_stale=True)
    feasible = bool(res.feasible[0])
    cache.put(h, score, trace, feasible)
    return score, trace, feasible, True


def _eval_worker(args):
    """Pool target of the reference (evaluate.py:406-442): no cache, no stale-layout gate."""
    if len(args) == 5:
        config, suite, workload, hw, K_eval = args
        memory_policy = MemoryPolicy()
    else:
        config, suite, workload, hw, K_eval, memory_policy = args
    score, trace, res = _score_one(config, suite, workload, hw, K_eval, memory_policy, gate_stale=False)
    return score, trace, bool(res.mask[0] & abi.MASK_MEM_OK)
