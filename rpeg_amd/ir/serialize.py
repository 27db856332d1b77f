"""Plan files: the reference's on-disk schemas, field for field (RPEG/ir/serialize.py:63-340).

`save_plan` / `load_plan` write and read the plain plan schema, `save_optimized_plan` /
`load_optimized_plan` the versioned artifact `rpeg.optimized_plan.v1` with its `plan_hash`
(sha256 of the canonical JSON without the hash), so that plans found by this engine flow to the
reference's runtime unchanged and plans written by the reference can be evaluated here.
"""

from __future__ import annotations

import hashlib
import json
from typing import Optional

from ..core.types import Allocation, Model
from ..model.workload import Workload
from .plan import ExecutionPlan
from .rpeg import RPEG

_MODEL_NAME = {Model.ACTOR: "actor", Model.CRITIC: "critic", Model.REFERENCE: "reference", Model.REWARD: "reward",
               Model.AC_SHARE: "ac_share"}
SCHEMA_VERSION = "rpeg.optimized_plan.v1"


def plan_to_dict(config) -> dict:
    """serialize.py:63-117.  `config` is a Configuration (rpeg, plan, device_space, ...)."""
    rpeg, plan, ds = config.rpeg, config.plan, config.device_space
    structure = {
        "ac_share": Model.AC_SHARE in rpeg.trainable,
        "intra_stage_fusion": bool(config.intra_stage_fusion),
        "tau": {_MODEL_NAME[m]: t for m, t in rpeg.tau.items()},
        "trainable": [_MODEL_NAME[m] for m in sorted(rpeg.trainable, key=lambda m: m.value)],
    }
    if config.transfer_resource_policy is not None:
        structure["transfer_resource_policy"] = config.transfer_resource_policy.to_dict()
    vertices = {}
    for v in rpeg.vertices:
        sigma, pi = plan.sigma[v], plan.pi[v]
        vertices[v.id] = {
            "model": _MODEL_NAME[v.kind.model],
            "role": v.kind.role.value,
            "placement": {"origin": list(sigma.origin), "extent": list(sigma.extent)},
            "parallelism": {"dp": pi[0], "pp": pi[1], "tp": pi[2]},
            "microbatch": plan.mb[v],
        }
    return {
        "device_space": {"racks": ds.R, "nodes_per_rack": ds.N, "gpus_per_node": ds.G},
        "structure": structure,
        "plan": vertices,
    }


def _read(path: str) -> dict:
    with open(path) as f:
        if path.endswith((".yaml", ".yml")):
            import yaml
            return yaml.safe_load(f)
        return json.load(f)


def _write(d: dict, path: str, trailing_newline: bool) -> None:
    if path.endswith((".yaml", ".yml")):
        import yaml
        with open(path, "w") as f:
            yaml.dump(d, f, default_flow_style=False, sort_keys=False, allow_unicode=True)
    else:
        with open(path, "w") as f:
            json.dump(d, f, indent=2)
            if trailing_newline:
                f.write("\n")


def load_plan(path: str, rpeg: RPEG) -> ExecutionPlan:
    """serialize.py:120-157: vertices are matched by id; ids the template does not know are skipped."""
    plan_d = _read(path)["plan"]
    by_id = {v.id: v for v in rpeg.vertices}
    sigma, pi, mb = {}, {}, {}
    for vid, info in plan_d.items():
        v = by_id.get(vid)
        if v is None:
            continue
        p, par = info["placement"], info["parallelism"]
        sigma[v] = Allocation(origin=tuple(p["origin"]), extent=tuple(p["extent"]))
        pi[v] = (par["dp"], par["pp"], par["tp"])
        mb[v] = info["microbatch"]
    return ExecutionPlan(sigma, pi, mb)


def save_plan(config, path: str) -> None:
    """serialize.py:160-183: YAML for .yaml/.yml, JSON otherwise."""
    _write(plan_to_dict(config), path, trailing_newline=False)


def optimized_plan_to_dict(config, algorithm: str, workload: Workload, source_config_hash: Optional[str] = None,
                           execution_schedule: Optional[dict] = None) -> dict:
    """serialize.py:186-241."""
    d = plan_to_dict(config)
    d.update({
        "schema_version": SCHEMA_VERSION,
        "source_config_hash": source_config_hash,
        "algorithm": algorithm.lower(),
        "workload": {
            "batch_size": workload.B,
            "samples_per_prompt": workload.K,
            "context_length": workload.S,
            "generation_length": workload.T,
            "gen_quantiles": [list(x) for x in workload.gen_quantiles] if workload.gen_quantiles else None,
        },
    })
    if execution_schedule is not None:
        d["execution_schedule"] = execution_schedule
    canonical = json.dumps({k: v for k, v in d.items() if k != "plan_hash"}, sort_keys=True, separators=(",", ":"))
    d["plan_hash"] = "sha256:" + hashlib.sha256(canonical.encode()).hexdigest()
    ordered = {k: d[k] for k in ("schema_version", "plan_hash", "source_config_hash", "algorithm", "workload",
                                 "device_space", "structure", "plan")}
    if execution_schedule is not None:
        ordered["execution_schedule"] = d["execution_schedule"]
    return ordered


def execution_schedule_to_dict(trace, *, horizon: int) -> dict:
    """serialize.py:244-274: nodes in dispatch order with their predicted times."""
    if horizon < 1:
        raise ValueError("execution schedule horizon must be >= 1")
    nodes = [{"node_id": node.id, "dispatch_index": i, "predicted_start_s": float(trace.start[node]),
              "predicted_finish_s": float(trace.finish[node])} for i, node in enumerate(trace.start)]
    return {"policy": "rpeg_critical_path_list_v1", "horizon": horizon,
            "predicted_makespan_s": float(trace.makespan()), "nodes": nodes}


def save_optimized_plan(config, path: str, algorithm: str, workload: Workload, source_config_hash: Optional[str] = None,
                        execution_schedule: Optional[dict] = None) -> None:
    """serialize.py:277-319."""
    _write(optimized_plan_to_dict(config, algorithm, workload, source_config_hash, execution_schedule), path,
           trailing_newline=True)


def load_optimized_plan(path: str) -> dict:
    """serialize.py:322-340."""
    d = _read(path)
    if d.get("schema_version") != SCHEMA_VERSION:
        raise ValueError("optimized plan must use schema_version rpeg.optimized_plan.v1")
    return d
