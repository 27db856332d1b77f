"""The search part of the reference's pipeline as one call (RPEG/pipeline.py:1405-1560, without the command
line, plots and reports): start plans from the candidate directory, the three evaluations that open the cache,
optimize() over the structural families, polish() on the same cache.  Every step runs on the GPU engine."""

from __future__ import annotations

import dataclasses
import time
from dataclasses import dataclass, field
from typing import Dict, Optional, Sequence

from ..core.types import DeviceSpace, Model
from ..ir.plan import ExecutionPlan
from ..model.hardware import Hardware
from ..model.models import ModelSuite
from ..model.workload import Workload
from .baselines import build_concurrent_baseline_plan, build_valid_baseline_plan
from .cache import EvalCache
from .evaluate import Configuration, _engine_for, evaluate_cached
from .moves import build_candidate_directory
from .inter_model import DEFAULT_T_CAND
from .optimizer import OptimizerConfig, family_structures, optimize, polish

def _template(algorithm: str, suite: ModelSuite, workload: Workload, tau: Optional[Dict[Model, int]]):
    """The synchronous template of an algorithm (RPEG/pipeline.py:1405-1410)."""
    from ..ir.dpo import build_DPO_RPEG
    from ..ir.grpo import build_GRPO_RPEG
    from ..ir.ppo import build_PPO_RPEG
    build = {"dpo": build_DPO_RPEG, "grpo": build_GRPO_RPEG}.get(algorithm, build_PPO_RPEG)
    return build(suite, workload, tau) if tau is not None else build(suite, workload)


@dataclass
class SearchResult:
    start: Configuration                 # what optimize() was seeded with: the concurrent start plan or `seed_plan`
    greedy: Configuration
    concurrent_found: bool               # False: no concurrent plan fits, the start is the greedy plan
    optimized: Configuration
    polished: Configuration              # == optimized when polish was skipped (infeasible result, no_polish)
    scores: Dict[str, float] = field(default_factory=dict)     # greedy, start, optimized, polished
    seconds: Dict[str, float] = field(default_factory=dict)    # directory + start plans, optimize, polish
    cache: Optional[EvalCache] = None


def search_plan(suite: ModelSuite, workload: Workload, hw: Hardware, device_space: DeviceSpace, K_eval: int,
                opt_config: OptimizerConfig, algorithm: Optional[str] = None, tau: Optional[Dict[Model, int]] = None,
                seed_plan: Optional[ExecutionPlan] = None, cache: Optional[EvalCache] = None, seed: int = 42,
                stream_key: Sequence[int] = (0, 0, 0), no_polish: bool = False,
                time_budget: Optional[float] = None) -> SearchResult:
    """Start plans -> optimize -> polish, in the order and on the shared cache of RPEG/pipeline.py:1412-1560.
    `time_budget` is the reference's --time (pipeline.py:1351-1366, 1542-1545): the annealing loop ends that many
    seconds after optimize() is entered and the evaluation budget E_max is lifted; E_struct still bounds a setting.
    The start plans are built and scored on the synchronous template (staleness 0 for every model of `tau`,
    pipeline.py:1398-1410); the optimizer is seeded with the template of staleness `tau` (pipeline.py:1524-1525)."""
    algorithm = algorithm or opt_config.algorithm
    policy = opt_config.memory_policy()
    cache = cache if cache is not None else EvalCache()
    rpeg = _template(algorithm, suite, workload, None if tau is None else {m: 0 for m in tau})
    seed_rpeg = rpeg if tau is None else _template(algorithm, suite, workload, tau)
    t0 = time.perf_counter()
    eng, _ = _engine_for(rpeg, suite, workload, hw, device_space, K_eval, policy, family_structures(rpeg, opt_config))
    table, _ = build_candidate_directory(rpeg, suite, device_space, workload, eng)
    conc_plan, found = build_concurrent_baseline_plan(rpeg, device_space, suite, workload, eng, table=table)
    greedy_plan = build_valid_baseline_plan(rpeg, device_space, suite, workload, eng, table=table)
    t1 = time.perf_counter()
    greedy = Configuration(rpeg, greedy_plan, device_space)
    conc = Configuration(rpeg, conc_plan, device_space)
    start = Configuration(rpeg, seed_plan if seed_plan is not None else conc_plan, device_space)
    scores = {}
    scores["greedy"] = evaluate_cached(greedy, cache, suite, workload, hw, K_eval, policy)[0]
    scores["concurrent"] = evaluate_cached(conc, cache, suite, workload, hw, K_eval, policy)[0]
    scores["start"] = evaluate_cached(start, cache, suite, workload, hw, K_eval, policy)[0]
    t2 = time.perf_counter()
    seed_config = Configuration(seed_rpeg, start.plan, device_space)
    if time_budget is not None:
        opt_config = dataclasses.replace(opt_config, deadline=time.perf_counter() + time_budget, E_max=10 ** 9)
    optimized = optimize(seed_config, suite, workload, hw, K_eval, opt_config, cache, seed=seed, stream_key=stream_key)
    t3 = time.perf_counter()
    scores["optimized"], _, feasible, _ = evaluate_cached(optimized, cache, suite, workload, hw, K_eval, policy)
    polished = optimized
    if feasible and not no_polish:      # pipeline.py:1553-1560
        ac_share = Model.AC_SHARE in optimized.rpeg.trainable
        structure = 1 if ac_share else 0
        p_table, p_index = build_candidate_directory(optimized.rpeg, suite, device_space, workload, eng, structure)
        polished = polish(optimized, suite, workload, hw, K_eval, opt_config, cache, p_table, p_index, ac_share=ac_share)
    t4 = time.perf_counter()
    scores["polished"] = evaluate_cached(polished, cache, suite, workload, hw, K_eval, policy)[0]
    return SearchResult(start=start, greedy=greedy, concurrent_found=found, optimized=optimized, polished=polished,
                        scores=scores, seconds=dict(start_plans=t1 - t0, optimize=t3 - t2, polish=t4 - t3), cache=cache)


def search_from_config(cfg, hw_overlay: Optional[str] = None, seed_plan_file: Optional[str] = None, seed: Optional[int] = None,
                       stream_key: Sequence[int] = (0, 0, 0), time_budget: Optional[float] = None) -> SearchResult:
    """`search_plan` for a configuration in the reference's YAML schema (a path or a loaded dict), with the glue
    of RPEG/pipeline.py:1285-1404, 1431-1436, 1521-1522, 1760-1761: optional calibrated-hardware overlay, algorithm
    and AC-share permission from the policy section, optimizer settings, staleness of the seed template = the first
    candidate of every model, optional seed plan file, base / optimized plan files named in the output section."""
    from .. import config_io
    from ..ir.serialize import load_plan, save_plan
    cfg = config_io.load_config(cfg) if isinstance(cfg, str) else cfg
    if hw_overlay:
        config_io.merge_hardware_overlay(cfg, hw_overlay)
    config_io.validate_config(cfg)
    out, pol, o = cfg.get("output", {}), cfg.get("policy", {}), cfg["optimizer"]
    algorithm = pol.get("algorithm", "ppo")
    allow_ac_share = pol.get("allow_ac_share", False) and algorithm == "ppo"
    device_space, suite = config_io.build_device_space(cfg), config_io.build_suite(cfg)
    workload, hw = config_io.build_workload(cfg), config_io.build_hardware(cfg)
    optim = config_io.build_optimizer_config(cfg, allow_ac_share, algorithm=algorithm)
    # pipeline.py:1367-1371 takes the first candidate of every model with candidates; restricted here to the models
    # the algorithm's template trains (the rest at 0), which is what the template accepts
    t_cand = optim.T_cand if optim.T_cand is not None else DEFAULT_T_CAND
    trained = _template(algorithm, suite, workload, None).tau
    tau = {m: next(iter(t_cand[m])) if t_cand.get(m) else 0 for m in trained}
    seed_plan = load_plan(seed_plan_file, _template(algorithm, suite, workload, tau)) if seed_plan_file else None
    res = search_plan(suite, workload, hw, device_space, o["k_eval"], optim, algorithm=algorithm, tau=tau,
                      seed_plan=seed_plan, seed=seed if seed is not None else out.get("seed") or 42,
                      stream_key=stream_key, no_polish=optim.no_polish, time_budget=time_budget)
    if out.get("base_plan"):
        save_plan(res.start, out["base_plan"])
    if out.get("opt_plan"):
        save_plan(res.polished, out["opt_plan"])
    return res
