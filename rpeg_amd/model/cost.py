"""The cost-model record of the reference's API (RPEG/model/cost.py:33-63).

The arithmetic of `NodeCostModel.time` (cost.py:66-357) runs inside the evaluation engine, on the GPU; what call
sites construct and pass around -- `NodeCostModel(hw, suite, workload, optimizer_stage, activation_checkpointing)`
handed to `build_candidate_directory` -- is this record, which names the engine that does the work."""

import math
from dataclasses import dataclass


@dataclass(frozen=True)
class NodeCostModel:
    hw: object
    suite: object
    workload: object
    optimizer_stage: int = 2
    activation_checkpointing: bool = True

    def __post_init__(self):
        if self.optimizer_stage not in (0, 1, 2):
            raise ValueError("optimizer_stage must be 0, 1, or 2")
        for name in ("op_generation_scale", "op_inference_scale", "op_training_scale", "weight_comm_scale", "reshard_scale"):
            x = float(getattr(self.hw, name))
            if not math.isfinite(x) or x <= 0.0:
                raise ValueError(f"hardware.{name} must be finite and > 0")
        x = float(self.hw.activation_comm_overhead_s)
        if not math.isfinite(x) or x < 0.0:
            raise ValueError("hardware.activation_comm_overhead_s must be finite and >= 0")

    def engine(self, rpeg, device_space, mem_model=None, K_eval: int = 1):
        """(engine, structure) that evaluates the template of `rpeg` under this cost model and `mem_model`'s
        policy (the policy of this record's two fields when no memory model is given)."""
        from ..search.evaluate import _engine_for
        from .memory import MemoryPolicy
        policy = mem_model.policy if mem_model is not None else MemoryPolicy(
            optimizer_stage=self.optimizer_stage, activation_checkpointing=self.activation_checkpointing)
        if (policy.optimizer_stage, policy.activation_checkpointing) != (self.optimizer_stage, self.activation_checkpointing):
            raise ValueError("the cost model and the memory model disagree on optimizer stage or activation checkpointing")
        trainable = mem_model.trainable if mem_model is not None and mem_model.trainable else None
        eng, _ = _engine_for(rpeg, self.suite, self.workload, self.hw, device_space, K_eval, policy,
                             memory_trainable=trainable)
        return eng, 0

    def time(self, node) -> float:
        raise NotImplementedError("node durations are computed on the GPU: Engine.op_time for mock operator nodes "
                                  "(as build_candidate_directory uses them), evaluate() for the nodes of a plan")
