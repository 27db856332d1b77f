"""Memory policy and memory-model record (mirror of RPEG/model/memory.py:138-250).  The per-device peak
arithmetic itself runs on the GPU; only the records live on the host."""

from dataclasses import dataclass
from typing import FrozenSet


@dataclass(frozen=True)
class MemoryPolicy:
    optimizer_stage: int = 2
    activation_checkpointing: bool = True
    runtime_overhead_fraction: float = 0.0
    worker_overhead_bytes: float = 0.0
    semantic_activation_cache_bytes: float = 0.0
    max_worker_groups_per_gpu: int = 0

    def __post_init__(self):
        if self.optimizer_stage not in (0, 1, 2):
            raise ValueError("optimizer_stage must be 0, 1, or 2")
        if not 0.0 <= self.runtime_overhead_fraction < 1.0:
            raise ValueError("runtime_overhead_fraction must be in [0, 1)")
        if self.worker_overhead_bytes < 0.0:
            raise ValueError("worker_overhead_bytes must be >= 0")
        if self.semantic_activation_cache_bytes < 0.0:
            raise ValueError("semantic_activation_cache_bytes must be >= 0")
        if self.max_worker_groups_per_gpu < 0:
            raise ValueError("max_worker_groups_per_gpu must be >= 0")


def optimizer_stage(name: str) -> int:
    """Numeric ZeRO stage of a distributed-optimizer mode name."""
    key = str(name or "none").strip().lower().replace("-", "_")
    table = {"none": 0, "adamw": 0,
             "zero1": 1, "zero_1": 1, "zero_stage_1": 1, "stage1": 1,
             "zero2": 2, "zero_2": 2, "zero_stage_2": 2, "stage2": 2}
    if key not in table:
        raise ValueError(f"unsupported distributed optimizer mode {name!r}")
    return table[key]


@dataclass(frozen=True)
class NodeMemoryModel:
    """What the reference's NodeMemoryModel is constructed from (RPEG/model/memory.py:188-250): hardware,
    models, workload, the policy's fields and the set of models it treats as trainable.  It is the
    argument `is_valid` takes; the arithmetic behind it is the engine's."""
    hw: object
    suite: object
    workload: object
    policy: MemoryPolicy = MemoryPolicy()
    trainable: FrozenSet = frozenset()
    shadow_models: FrozenSet = frozenset()   # kept as the reference keeps it; no formula reads it

    @classmethod
    def from_policy(cls, hw, suite, workload, policy: MemoryPolicy, trainable=frozenset(), shadow_models=frozenset()):
        return cls(hw, suite, workload, policy, frozenset(trainable), frozenset(shadow_models))
