"""Batched simulated annealing on the GPU evaluator.

`OptimizerConfig` mirrors RPEG/search/optimizer.py:33-128 (same fields, same derived I_max and
T_cool).  The reference runs ONE chain at a time and maps `_eval_worker` over the K_x candidates of
its current step (optimizer.py:793-798); here a population of independent chains advances in
lock-step and the candidates of all chains of a step are scored in one launch (rpeg_sa_run).  The
neighbourhood (move_gen, multi_move_pair), the best-of-K proposal, the acceptance rule, the elite
list and the stagnation restarts are the reference's; the random numbers are a counter-based stream
instead of MT19937, so a run is reproducible but not draw-for-draw equal to a reference run.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass, field
from typing import Dict, FrozenSet, List, Optional, Sequence, Set, Tuple

import numpy as np

from ..core.types import Allocation, Model, packing_geometry
from ..engine import abi
from ..engine.problem import EvalProblem, FIELDS_PER_VERTEX
from ..ir.plan import ExecutionPlan
from ..model.hardware import Hardware
from ..model.memory import MemoryPolicy
from ..model.models import ModelSuite
from ..model.workload import Workload
from .cache import EvalCache
from .evaluate import (Configuration, _check_supported, _engine_for, _structure_of, evaluate_batch, evaluate_cached,
                       evaluation_cache_key)
from .inter_model import DEFAULT_T_CAND, _iter_staleness as _staleness_assignments
from .moves import build_candidate_directory, directory_arrays



@dataclass
class OptimizerConfig:
    """RPEG/search/optimizer.py:33-128.  Fields that steer parts this engine does not run (structural
    outer loop budgets, utilisation objective, ablations) are kept so that existing call sites
    construct it unchanged; they are ignored unless noted."""
    K_x: int = 6
    T_max: int = 50
    E_max: int = 5000
    E_struct: int = 400
    T_cand: Optional[Dict[Model, Set[int]]] = None
    structural_candidates: Optional[FrozenSet[str]] = None
    lambda_ac: float = 0.15
    score_eps: float = 1e-4
    T_init: float = 0.30
    T_warm: float = 0.05
    T_min: float = 0.01
    K_elite: int = 3
    alpha_pair: float = 0.28
    stag_window: int = 20
    max_throughput_loss: float = 0.0
    I_max: int = 0
    R_max: int = 10000
    T_cool: float = 0.0
    algorithm: str = "ppo"
    deadline: Optional[float] = None
    deadline_per_struct: Optional[float] = None
    fixed_mb: bool = False
    uniform_vertex: bool = False
    no_polish: bool = False
    hard_oom: bool = False
    geometric_cooling: bool = False
    memory_optimizer_stage: int = 2
    memory_activation_checkpointing: bool = True
    memory_runtime_overhead_fraction: float = 0.0
    memory_worker_overhead_bytes: float = 0.0
    memory_semantic_activation_cache_bytes: float = 0.0
    memory_max_worker_groups_per_gpu: int = 0

    def __post_init__(self) -> None:
        allowed = frozenset({"separate", "fused", "ac_share"})
        if self.structural_candidates is not None:
            unknown = self.structural_candidates - allowed
            if unknown:
                raise ValueError("unknown structural_candidates: " + ", ".join(sorted(unknown)))
            if not self.structural_candidates:
                raise ValueError("structural_candidates must not be empty")
        self.memory_policy()
        if self.I_max <= 0:
            self.I_max = int(self.E_struct / ((self.K_x + 1) / 2) * 0.5)
        self.T_cool = (self.T_min / self.T_init) ** (1.0 / (0.7 * self.I_max))

    def memory_policy(self) -> MemoryPolicy:
        return MemoryPolicy(optimizer_stage=self.memory_optimizer_stage,
                            activation_checkpointing=self.memory_activation_checkpointing,
                            runtime_overhead_fraction=self.memory_runtime_overhead_fraction,
                            worker_overhead_bytes=self.memory_worker_overhead_bytes,
                            semantic_activation_cache_bytes=self.memory_semantic_activation_cache_bytes,
                            max_worker_groups_per_gpu=self.memory_max_worker_groups_per_gpu)


@dataclass
class ChainResult:
    """Outcome of `optimize_chains` (arrays are indexed by chain)."""
    best_plan: np.ndarray          # int16 [n_chains, MAX_V*10]
    best_score: np.ndarray
    best_step: np.ndarray
    best_time: np.ndarray          # seconds from the start of the run to the first sight of best_plan
    best_feasible: np.ndarray
    cur_plan: np.ndarray
    cur_score: np.ndarray
    restarts: np.ndarray
    n_eval: np.ndarray
    dead: np.ndarray
    log: np.ndarray
    variants: List[Tuple[int, ...]]
    wall_s: float = 0.0
    eval_s: float = 0.0
    n_launch: int = 0
    n_plans: int = 0

    def argbest(self) -> int:
        """Chain holding the best feasible plan (lowest chain index among equals); falls back to the
        best infeasible one as optimize() does (optimizer.py:946)."""
        feas = self.best_feasible.astype(bool)
        pool = np.flatnonzero(feas) if feas.any() else np.flatnonzero(~np.isnan(self.best_score))
        if pool.size == 0:
            raise RuntimeError("no chain holds a plan")
        return int(pool[np.argmax(self.best_score[pool])])


def sa_params(opt: OptimizerConfig, n_chains: int, n_steps: int, variants: Sequence[Sequence[int]], structure: int = 0,
              split: int = 1, seed: int = 42, restart_attempts: int = 50, gate_candidates: bool = False) -> abi.SaParamsT:
    p = abi.SaParamsT()
    p.n_chains, p.n_steps, p.K_x, p.T_max, p.K_elite = n_chains, n_steps, opt.K_x, opt.T_max, opt.K_elite
    p.stag_window, p.restart_attempts = opt.stag_window, restart_attempts
    p.gate_candidates, p.geometric_cooling = int(gate_candidates), int(opt.geometric_cooling)
    p.structure, p.split, p.n_variants = structure, split, len(variants)
    if not 1 <= len(variants) <= 8:
        raise ValueError("between 1 and 8 staleness variants")
    for k, taus in enumerate(variants):
        for t in range(2):
            p.tau[k][t] = int(taus[t]) if t < len(taus) else 0
    p.T_init, p.T_warm, p.T_min, p.T_cool = opt.T_init, opt.T_warm, opt.T_min, opt.T_cool
    p.alpha_pair, p.score_eps, p.seed = opt.alpha_pair, opt.score_eps, seed
    p.max_throughput_loss = float(opt.max_throughput_loss)
    p.fixed_mb, p.uniform_vertex, p.hard_oom = int(opt.fixed_mb), int(opt.uniform_vertex), int(opt.hard_oom)
    return p


def set_deadline(params: abi.SaParamsT, opt: OptimizerConfig, clock=None):
    """Enters OptimizerConfig.deadline / .deadline_per_struct into the parameters of rpeg_sa_optimize*.  Both
    are readings of time.perf_counter() (optimizer.py:78-82) -- or of `clock` when one is given -- and the
    library counts its steady clock from the start of the call, so without `clock` they go in as seconds
    from now.  Returns what must stay alive while the call runs (the callback of `clock`)."""
    params.timed = (1 if opt.deadline is not None else 0) | (2 if opt.deadline_per_struct is not None else 0)
    if not params.timed:
        return None
    import time
    now = 0.0 if clock is not None else time.perf_counter()
    params.deadline_s = (opt.deadline - now) if opt.deadline is not None else 0.0
    params.deadline_struct_s = (opt.deadline_per_struct - now) if opt.deadline_per_struct is not None else 0.0
    if clock is None:
        return None
    fn = abi.CLOCK_FN(lambda _ctx: float(clock()))
    params.clock = C.cast(fn, C.c_void_p)
    return fn


def plan_row(rpeg, plan: ExecutionPlan) -> np.ndarray:
    row = np.zeros(abi.MAX_V * FIELDS_PER_VERTEX, np.int16)
    for slot, v in enumerate(rpeg.vertices):
        a = plan.sigma[v]
        row[slot * FIELDS_PER_VERTEX:(slot + 1) * FIELDS_PER_VERTEX] = [*plan.pi[v], plan.mb[v], *a.origin, *a.extent]
    return row


def row_plan(rpeg, row: np.ndarray) -> ExecutionPlan:
    sigma, pi, mb = {}, {}, {}
    for slot, v in enumerate(rpeg.vertices):
        f = [int(x) for x in row[slot * FIELDS_PER_VERTEX:(slot + 1) * FIELDS_PER_VERTEX]]
        pi[v], mb[v] = (f[0], f[1], f[2]), f[3]
        sigma[v] = Allocation(origin=(f[4], f[5], f[6]), extent=(f[7], f[8], f[9]))
    return ExecutionPlan(sigma=sigma, pi=pi, mb=mb)


def optimize_chains(problem: EvalProblem, opt: OptimizerConfig, n_chains: int, n_steps: int,
                    variants: Sequence[Sequence[int]], seed: int = 42, base_plan: Optional[ExecutionPlan] = None,
                    engine=None, structure: int = 0, directory=None, gate_candidates: bool = False) -> ChainResult:
    """Runs `n_chains` chains of `n_steps` steps on the GPU.  Chain c anneals under staleness variant
    variants[c % len(variants)] (one staleness value per trainable model of the structure)."""
    from ..engine.runtime import Engine
    eng = engine or Engine(problem)
    rpeg0 = problem.template(structure, ())
    if directory is None:
        table, _ = build_candidate_directory(rpeg0, problem.suite, problem.device_space, problem.workload, eng, structure)
        directory = directory_arrays(rpeg0, table)
    split = 1 if problem.workload.gen_quantiles else 0
    params = sa_params(opt, n_chains, n_steps, variants, structure, split, seed, gate_candidates=gate_candidates)
    base = plan_row(rpeg0, base_plan) if base_plan is not None else None
    out = eng.sa_run(params, directory, base)
    return ChainResult(variants=[tuple(int(t) for t in v) for v in variants], **out)


def _iter_staleness(tau_models, t_cand) -> List[Tuple[int, ...]]:
    """The staleness variants in the reference's order (RPEG/search/inter_model.py:43-65), each as one
    value per entry of `tau_models`."""
    return [tuple(tau[m] for m in tau_models) for tau in _staleness_assignments(tau_models, t_cand)]


def _ac_penalty(score: float, lambda_ac: float) -> float:
    """RPEG/search/optimizer.py:132-145."""
    return score if lambda_ac == 0.0 else score * (1.0 - lambda_ac)


def penalized_score(raw_score: float, rpeg, opt_config: "OptimizerConfig", ac_share: bool) -> float:
    """The score optimize() ranks by (RPEG/search/optimizer.py:148-170): only the AC-share penalty."""
    return _ac_penalty(raw_score, opt_config.lambda_ac) if ac_share else raw_score


def optimize_families(problem: EvalProblem, opt_config: OptimizerConfig, engine_directory) -> List[tuple]:
    """The structural families optimize() walks for structure 0 of `problem`, in the reference's order
    (RPEG/search/inter_model.py:68-121 filtered by `structural_candidates`, optimizer.py:541-553): the
    separate template with the staleness variants of T_cand, then -- for a template that trains an actor
    and a critic, when `problem` holds the AC-share template as structure 1 and its view under the base
    configuration's memory model as structure 2 -- AC-share with its own, scored times (1 - lambda_ac).
    The fused settings are not entered (that lowering pass does not run upstream).  Returns the list
    Engine.sa_optimize_families takes; `engine_directory(structure)` supplies the candidate directory."""
    t_cand = opt_config.T_cand if opt_config.T_cand is not None else DEFAULT_T_CAND
    names = opt_config.structural_candidates
    split = 1 if problem.workload.gen_quantiles else 0
    st = problem.structures[0]
    families = []
    if names is None or "separate" in names:
        variants = _iter_staleness(st.tau_models, t_cand)
        if variants:
            families.append((sa_params(opt_config, 1, 1, variants, 0, split, 0), engine_directory(0), 1.0, 0, None))
    shares = set(st.tau_models) >= {Model.ACTOR, Model.CRITIC}      # is_AC_share_applicable (ir/ac_share.py:17-26)
    if shares and len(problem.structures) >= 3 and (names is None or "ac_share" in names):
        ac = problem.structures[1]
        variants = _iter_staleness(ac.tau_models, t_cand)
        if variants:
            scale = 1.0 - opt_config.lambda_ac if opt_config.lambda_ac != 0.0 else 1.0
            families.append((sa_params(opt_config, 1, 1, variants, 1, split, 0), engine_directory(1), scale, 1, 2))
    if not families:
        raise ValueError("structural_candidates exclude every inter-model candidate for "
                         f"algorithm={opt_config.algorithm}")
    return families


def family_structures(rpeg, opt_config: OptimizerConfig) -> tuple:
    """The structures an engine for optimize() on the template of `rpeg` holds besides that template: for a
    template that trains an actor and a critic, unless `structural_candidates` leaves AC-share out, the AC-share
    template and its view under the base configuration's memory model."""
    from ..engine.problem import STRUCTURES, as_seen_from
    st = _structure_of(rpeg)
    names = opt_config.structural_candidates
    if set(st.tau_models) >= {Model.ACTOR, Model.CRITIC} and (names is None or "ac_share" in names):
        return (STRUCTURES["ac_share"], as_seen_from(STRUCTURES["ac_share"], st))
    return ()


def optimize(base_config: Configuration, suite: ModelSuite, workload: Workload, hw: Hardware, K_eval: int,
             opt_config: OptimizerConfig, cache: Optional[EvalCache] = None, seed: int = 42,
             stream_key: Sequence[int] = (0, 0, 0), clock=None) -> Configuration:
    """Drop-in for optimize() (RPEG/search/optimizer.py:365-946) on the template of `base_config`.

    Runs the reference's loop (rpeg_sa_optimize_families): the structural families one after the other --
    the template of `base_config` with the staleness variants of T_cand, then, for a PPO template, the
    AC-share template with its own, scored times (1 - lambda_ac) -- and per variant a sequence of restarts
    of one chain, with the evaluation cache, the budgets E_max / E_struct, the per-family elites and the
    warm restarts of the reference.  The K_x candidates of an iteration are one GPU launch.  Given the same
    random generator the reference evaluates the same plans in the same order and returns the same
    configuration (tests/golden/make_golden_optimize.py); the generator here is the counter-based stream
    (seed, *stream_key), not MT19937.

    With `max_throughput_loss` > 0 plans are ranked by throughput x utilisation above the throughput floor
    (optimizer.py:461-486); every evaluated plan is then traced once more for its utilisation.

    `opt_config.deadline` / `.deadline_per_struct` are readings of time.perf_counter() as in the reference
    (optimizer.py:78-82, 571-579, 703-720, 848-865); `clock`, a callable returning seconds, takes the place of
    perf_counter for both when given.  The ablation switches `fixed_mb`, `uniform_vertex` and `hard_oom` are
    turned into the module switches of search.moves and search.evaluate as the reference does
    (optimizer.py:404-410) and stay set afterwards, as there.

    Not entered: the intra-stage-fusion settings (`structural_candidates` "fused").  The run keeps its own
    cache (keyed by plan, template and staleness); what it evaluated is put into `cache` afterwards under the
    reference's keys, entries `cache` held before are not consulted."""
    _check_supported(base_config)
    from . import evaluate as _eval_mod, moves as _moves_mod
    _moves_mod.ABLATION_FIXED_MB = bool(opt_config.fixed_mb)
    _moves_mod.ABLATION_UNIFORM_VERTEX = bool(opt_config.uniform_vertex)
    _eval_mod.ABLATION_HARD_OOM = bool(opt_config.hard_oom)
    policy = opt_config.memory_policy()
    more = family_structures(base_config.rpeg, opt_config)
    eng, st = _engine_for(base_config.rpeg, suite, workload, hw, base_config.device_space, K_eval, policy, more,
                          transfer_policy=base_config.transfer_resource_policy)

    def directory(structure: int):
        rpeg = eng.problem.template(structure, ())
        table, _ = build_candidate_directory(rpeg, suite, base_config.device_space, workload, eng, structure)
        return directory_arrays(rpeg, table)

    families = optimize_families(eng.problem, opt_config, directory)
    families[0][0].seed = seed
    keep_clock = set_deadline(families[0][0], opt_config, clock)
    # evaluations the run can make: its budget, and per structural setting E_struct, the batch that crosses it,
    # the setting's start plan and the restart that follows the crossing
    n_settings = sum(f[0].n_variants for f in families)
    log_cap = min(opt_config.E_max, n_settings * (opt_config.E_struct + 2 * opt_config.K_x + 2)) + 64
    own = [int(base_config.rpeg.tau.get(m, 0)) for m in st.tau_models]
    res = eng.sa_optimize_families(families, own, plan_row(base_config.rpeg, base_config.plan), opt_config.E_max,
                                   opt_config.E_struct, opt_config.R_max, stream_key,
                                   log_cap=log_cap if cache is not None else 0)
    del keep_clock
    if cache is not None:
        _carry_into(cache, eng.problem, families, res, own, suite, workload, base_config, policy,
                    opt_config.max_throughput_loss > 0.0)
    return configuration_of(eng.problem, families, res, own, suite, workload, base_config)


def _carry_into(cache: EvalCache, problem, families, res, base_tau, suite, workload, base_config, policy, with_util):
    """Puts what the run evaluated into the caller's cache under the reference's keys, so that what runs next on
    the same cache -- polish() in the reference's pipeline (RPEG/pipeline.py:1549-1560) -- finds the entries
    optimize() would have left there: score and feasibility as stored, and in the trace's place the
    utilisation (the one number of a trace that polish reads) when the utilisation objective is on."""
    templates = {}
    for row, var, score, feasible, util in zip(res["eval_log"], res["eval_log_variant"], res["eval_log_score"],
                                               res["eval_log_feasible"], res["eval_log_util"]):
        var = int(var)
        if var not in templates:
            f, k = (0, None) if var == 255 else (var // 8, var % 8)
            st = problem.structures[families[f][0].structure]
            taus = list(base_tau) if k is None else [int(families[f][0].tau[k][i]) for i in range(len(st.tau_models))]
            templates[var] = st.build(suite, workload, tau={m: taus[i] for i, m in enumerate(st.tau_models)})
        rpeg = templates[var]
        config = Configuration(rpeg, row_plan(rpeg, row), base_config.device_space, intra_stage_fusion=False,
                               transfer_resource_policy=base_config.transfer_resource_policy)
        h = evaluation_cache_key(config, policy)
        if h not in cache:
            cache.put(h, float(score), _Utilization(float(util)) if with_util else None, bool(feasible))


def configuration_of(problem: EvalProblem, families, res, base_tau, suite, workload, base_config) -> Configuration:
    """The configuration a result of sa_optimize_families names: template of the best family, staleness of
    its best variant (the base configuration's own when that is what was best), best plan."""
    params = families[res["best_family"]][0]
    st = problem.structures[params.structure]
    k = res["best_variant"]
    taus = list(base_tau) if k >= params.n_variants else [int(params.tau[k][i]) for i in range(len(st.tau_models))]
    rpeg = st.build(suite, workload, tau={m: taus[i] for i, m in enumerate(st.tau_models)})
    return Configuration(rpeg, row_plan(rpeg, res["best_plan"]), base_config.device_space,
                         intra_stage_fusion=False, transfer_resource_policy=base_config.transfer_resource_policy)


class _Utilization:
    """Stands in a cache entry for the trace of a polish candidate: its one number the objective reads."""

    def __init__(self, value: float):
        self.value = value

    def utilization(self) -> float:
        return self.value


def polish(best_config: Configuration, suite: ModelSuite, workload: Workload, hw: Hardware, K_eval: int,
           opt_config: OptimizerConfig, cache: EvalCache, table, index, ac_share: bool = False,
           max_rounds: int = 50) -> Configuration:
    """Drop-in for polish() (RPEG/search/optimizer.py:949-1188): deterministic greedy coordinate descent on
    the plan returned by optimize().  Vertices in id order; for each, every strategy of the directory window
    around the current one, placed at origin (0,0,0), is scored in ONE batched launch (the reference maps
    `_eval_worker` over them, optimizer.py:1138-1148); the best strict improvement among the memory-feasible
    ones is applied; passes repeat until one brings no improvement.  Cache hits are merged before fresh
    results, as in the reference, so equal scores resolve the same way."""
    _check_supported(best_config)
    policy = opt_config.memory_policy()
    config, rpeg = best_config, best_config.rpeg
    G = config.device_space.G
    delta, best_raw = opt_config.max_throughput_loss, [0.0]

    def _score(raw: float, trace=None) -> float:   # optimizer.py:1021-1044
        s = raw
        if delta > 0.0 and trace is not None:
            best_raw[0] = max(best_raw[0], raw)
            s = raw * 1e-12 if raw < (1.0 - delta) * best_raw[0] else raw * max(trace.utilization(), 1e-6)
        return _ac_penalty(s, opt_config.lambda_ac) if ac_share else s

    vertices = sorted(rpeg.vertices, key=lambda v: v.id)
    w_frac = opt_config.T_min / opt_config.T_init
    raw, _trace, _feasible, _miss = evaluate_cached(config, cache, suite, workload, hw, K_eval, policy)
    score = _score(raw, _trace)
    for _round in range(max_rounds):
        improved = False
        for v in vertices:
            best_score, best = score, None
            v_table = table[v]
            n = len(v_table)
            w = max(5, int(n * w_frac))
            dp_c, pp_c, tp_c = config.plan.pi[v]
            r_ext_c, n_ext_c, _g = config.plan.sigma[v].extent
            j_star = index[v].get((dp_c, pp_c, tp_c, r_ext_c, n_ext_c, config.plan.mb[v]), n // 2)
            cands = []
            for j in range(max(0, j_star - w), min(n - 1, j_star + w) + 1):
                if j == j_star:
                    continue
                dp, pp, tp, r_ext, n_ext, mb = v_table[j][:6]
                geom = packing_geometry(dp, pp, tp, G)
                if geom is None:
                    continue
                plan = ExecutionPlan(sigma={**config.plan.sigma, v: Allocation(origin=(0, 0, 0), extent=(r_ext, n_ext, geom[0]))},
                                     pi={**config.plan.pi, v: (dp, pp, tp)}, mb={**config.plan.mb, v: mb})
                cands.append(Configuration(rpeg, plan, config.device_space, intra_stage_fusion=False,
                                           transfer_resource_policy=config.transfer_resource_policy))
            hits, misses = [], []
            for nb in cands:
                h = evaluation_cache_key(nb, policy)
                if h in cache:
                    s, t, f = cache.get(h)
                    hits.append((nb, s, t, f))
                else:
                    misses.append((nb, h))
            fresh = []
            if misses:
                res = evaluate_batch([nb for nb, _ in misses], suite, workload, hw, K_eval, policy, gate_stale=False,
                                     with_util=delta > 0.0)
                for j, ((nb, h), s, m) in enumerate(zip(misses, res.score, res.mask)):
                    f = bool(m & abi.MASK_MEM_OK)
                    # the utilisation objective reads one number of a candidate's trace: keep that (same launch)
                    t = _Utilization(float(res.util[j])) if delta > 0.0 else None
                    cache.put(h, float(s), t, f)
                    fresh.append((nb, float(s), t, f))
            for nb, s, t, f in hits + fresh:
                if not f:
                    continue
                score_n = _score(s, t)
                if score_n > best_score:
                    best_score, best = score_n, nb
            if best is not None:
                config, score, improved = best, best_score, True
        if not improved:
            break
    return config
