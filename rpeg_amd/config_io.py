"""Workload / cluster configuration files in the reference's YAML schema (pipeline.py:65-385).

`load_config` reads a file (bare scientific notation such as 450e9 is a float, as in the
reference's loader), `validate_config` applies the reference's checks, the `build_*` functions
make the records and `problem_from_config` assembles what the engine evaluates.
"""

from __future__ import annotations

import copy
import re
from typing import Dict, Optional

import yaml

from .core.types import DeviceSpace, Model
from .engine.problem import DPO, GRPO, PPO, EvalProblem
from .model.hardware import Hardware
from .model.memory import MemoryPolicy
from .model.models import ModelSpec, ModelSuite
from .model.workload import Workload
from .search.optimizer import DEFAULT_T_CAND, OptimizerConfig

_FLOAT_RE = re.compile(r'''^(?:
    [-+]?(?:[0-9][0-9_]*)\.?[0-9_]*(?:[eE][-+]?[0-9]+)?
    |[-+]?\.(?:inf|Inf|INF)
    |\.(?:nan|NaN|NAN)
)$''', re.X)

_HW_REQUIRED = ("racks", "nodes_per_rack", "gpus_per_node", "flops_per_gpu", "memory_per_gpu", "memory_bandwidth")
_HW_TIERS = ("alpha_coll_g", "beta_coll_g", "alpha_coll_n", "beta_coll_n", "alpha_coll_r", "beta_coll_r",
             "alpha_p2p_g", "beta_p2p_g", "alpha_p2p_n", "beta_p2p_n", "alpha_p2p_r", "beta_p2p_r")


class _Loader(yaml.SafeLoader):
    pass


_Loader.add_implicit_resolver("tag:yaml.org,2002:float", _FLOAT_RE, list("-+0123456789."))


def load_config(path: str) -> Dict:
    with open(path) as f:
        return yaml.load(f, Loader=_Loader)


def merge_hardware_overlay(cfg: Dict, path: str) -> Dict:
    """Overlays the `key: value` lines of a calibrated-hardware file on cfg["hardware"] as the reference's
    `--hw` option does (pipeline.py:1288-1302): comment and blank lines skipped, text after `#` dropped, values
    that do not read as floats ignored.  Returns cfg."""
    overlay = {}
    with open(path) as f:
        for line in f:
            if not line.strip() or line.strip().startswith("#") or ":" not in line:
                continue
            key, val = line.split(":", 1)
            try:
                overlay[key.strip()] = float(val.split("#")[0].strip())
            except ValueError:
                pass
    cfg.setdefault("hardware", {}).update(overlay)
    return cfg


def _require(d: Dict, *keys: str, section: str = "") -> None:
    prefix = f"[{section}] " if section else ""
    for k in keys:
        if k not in d:
            raise ValueError(f"{prefix}Missing required field: '{k}'")


def algorithm_of(cfg: Dict) -> str:
    return cfg.get("policy", {}).get("algorithm", "ppo")


def validate_config(cfg: Dict) -> None:
    """pipeline.py:119-194."""
    _require(cfg, "hardware", "models", "workload", "optimizer")
    hw = cfg["hardware"]
    _require(hw, *_HW_REQUIRED, section="hardware")
    if hw["racks"] < 1 or hw["nodes_per_rack"] < 1 or hw["gpus_per_node"] < 1:
        raise ValueError("[hardware] racks, nodes_per_rack, gpus_per_node must all be >= 1")
    for f in _HW_TIERS:
        _require(hw, f, section="hardware")
    algo = algorithm_of(cfg)
    roles = ("actor",) if algo == "dpo" else ("actor", "reward") if algo == "grpo" else ("actor", "critic", "reward")
    for role in roles:
        _require(cfg["models"], role, section="models")
        _require(cfg["models"][role], "layers", "hidden_dim", "ffn_dim", "vocab_size", section=f"models.{role}")
    _require(cfg["workload"], "batch_size", "samples_per_prompt", "context_length", "generation_length",
             section="workload")
    o = cfg["optimizer"]
    _require(o, "k_eval", section="optimizer")
    if o["k_eval"] < 1:
        raise ValueError("[optimizer] k_eval must be >= 1")
    if algo not in ("ppo", "grpo", "dpo"):
        raise ValueError(f"[policy] Unsupported algorithm '{algo}'. Currently supported: 'ppo', 'grpo', 'dpo'.")
    sc = o.get("staleness_candidates")
    if sc is not None:
        valid = {"actor", "critic", "ac_share"}
        for name in sc:
            if name not in valid:
                raise ValueError(f"[optimizer.staleness_candidates] Unknown model '{name}'. Valid names: {sorted(valid)}")


def build_device_space(cfg: Dict) -> DeviceSpace:
    hw = cfg["hardware"]
    return DeviceSpace(R=hw["racks"], N=hw["nodes_per_rack"], G=hw["gpus_per_node"])


def build_hardware(cfg: Dict) -> Hardware:
    """pipeline.py:211-243 (same optional fields and defaults)."""
    hw = cfg["hardware"]
    return Hardware(
        flops_per_gpu=hw["flops_per_gpu"], memory_per_gpu=hw["memory_per_gpu"], memory_bandwidth=hw["memory_bandwidth"],
        **{f: hw[f] for f in _HW_TIERS},
        gemm_m_half=hw.get("gemm_m_half", 5.0), gemm_k_half=hw.get("gemm_k_half", 0.0),
        decode_bw_eff=hw.get("decode_bw_eff", 0.15), non_gemm_constant=hw.get("non_gemm_constant", 0.0),
        non_gemm_scaling=hw.get("non_gemm_scaling", 0.0), non_gemm_batch_cal=hw.get("non_gemm_batch_cal", 64))


def build_suite(cfg: Dict) -> ModelSuite:
    """pipeline.py:246-294: the reference model shares the actor's architecture, and so does AC-share."""
    m, algo = cfg["models"], algorithm_of(cfg)

    def spec(role: str) -> ModelSpec:
        s = m[role]
        return ModelSpec(L=s["layers"], d=s["hidden_dim"], d_ff=s["ffn_dim"], V=s["vocab_size"],
                         d_head=s.get("head_dim", 128))
    actor = spec("actor")
    specs = {Model.ACTOR: actor, Model.REFERENCE: actor}
    if algo in ("ppo", "grpo"):
        specs[Model.REWARD] = spec("reward")
    if algo == "ppo":
        specs[Model.CRITIC] = spec("critic")
        specs[Model.AC_SHARE] = actor
    return ModelSuite(specs)


def build_workload(cfg: Dict) -> Workload:
    w = cfg["workload"]
    gq = w.get("gen_quantiles", None)
    return Workload(B=w["batch_size"], K=w["samples_per_prompt"], S=w["context_length"], T=w["generation_length"],
                    gen_quantiles=tuple(tuple(q) for q in gq) if gq else None)


def build_optimizer_config(cfg: Dict, allow_ac_share: bool, algorithm: str = "ppo") -> OptimizerConfig:
    """pipeline.py:318-385."""
    o = cfg["optimizer"]
    sc = o.get("staleness_candidates")
    if algorithm in ("grpo", "dpo"):
        t_cand = {Model.ACTOR: {0, 1}}
        if sc is not None and "actor" in sc:
            t_cand[Model.ACTOR] = set(sc["actor"])
    elif sc is None and allow_ac_share:
        t_cand = None
    else:
        names = {"actor": Model.ACTOR, "critic": Model.CRITIC, "ac_share": Model.AC_SHARE}
        t_cand = copy.deepcopy(DEFAULT_T_CAND)
        if sc is not None:
            for name, vals in sc.items():
                t_cand[names[name]] = set(vals)
        if not allow_ac_share:
            t_cand[Model.AC_SHARE] = set()
    return OptimizerConfig(
        K_x=o.get("k_x", 6), T_max=o.get("t_max", 50), E_max=o.get("e_max", 5000), T_init=o.get("t_init", 0.30),
        T_warm=o.get("t_warm", 0.10), T_min=o.get("t_min", 0.03), E_struct=o.get("e_struct", 400), T_cand=t_cand,
        lambda_ac=o.get("lambda_ac", 0.15), score_eps=o.get("score_eps", 1e-4), stag_window=o.get("stag_window", 20),
        alpha_pair=o.get("alpha_pair", 0.28), max_throughput_loss=o.get("max_throughput_loss", 0.0),
        algorithm=algorithm, fixed_mb=o.get("fixed_mb", False), uniform_vertex=o.get("uniform_vertex", False),
        no_polish=o.get("no_polish", False), hard_oom=o.get("hard_oom", False),
        geometric_cooling=o.get("geometric_cooling", False))


def problem_from_config(cfg: Dict, memory_policy: Optional[MemoryPolicy] = None) -> EvalProblem:
    """The evaluation problem of a validated configuration (one template structure: that of its algorithm)."""
    validate_config(cfg)
    structure = {"ppo": PPO, "grpo": GRPO, "dpo": DPO}[algorithm_of(cfg)]
    return EvalProblem(structures=(structure,), suite=build_suite(cfg), workload=build_workload(cfg),
                       hw=build_hardware(cfg), device_space=build_device_space(cfg),
                       K_eval=cfg["optimizer"]["k_eval"], memory_policy=memory_policy or MemoryPolicy())
