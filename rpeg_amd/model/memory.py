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
    """The memory-model record of the reference's API, with its fields and defaults (RPEG/model/memory.py:188-250):
    hardware, models, workload, the policy's values and the set of models it treats as trainable.  The arithmetic
    behind `peak_bytes`, `_device_peaks`, `mem_feasible` and `mem_worst_violation` is the engine's."""
    hw: object
    suite: object
    workload: object
    eps_rt: float = 0.0
    trainable: FrozenSet = frozenset()
    shadow_models: FrozenSet = frozenset()   # kept as the reference keeps it; no formula reads it
    optimizer_stage: int = 2
    worker_overhead_bytes: float = 0.0
    semantic_activation_cache_bytes: float = 0.0
    max_worker_groups_per_gpu: int = 0
    activation_checkpointing: bool = True

    def __post_init__(self):
        if self.optimizer_stage not in (0, 1, 2):
            raise ValueError("optimizer_stage must be 0, 1, or 2")

    @classmethod
    def from_policy(cls, hw, suite, workload, policy: MemoryPolicy, trainable=frozenset(), shadow_models=frozenset()):
        return cls(hw, suite, workload, eps_rt=policy.runtime_overhead_fraction, trainable=frozenset(trainable),
                   shadow_models=frozenset(shadow_models), optimizer_stage=policy.optimizer_stage,
                   worker_overhead_bytes=policy.worker_overhead_bytes,
                   semantic_activation_cache_bytes=policy.semantic_activation_cache_bytes,
                   max_worker_groups_per_gpu=policy.max_worker_groups_per_gpu,
                   activation_checkpointing=policy.activation_checkpointing)

    @property
    def policy(self) -> MemoryPolicy:
        return MemoryPolicy(optimizer_stage=self.optimizer_stage, activation_checkpointing=self.activation_checkpointing,
                            runtime_overhead_fraction=self.eps_rt, worker_overhead_bytes=self.worker_overhead_bytes,
                            semantic_activation_cache_bytes=self.semantic_activation_cache_bytes,
                            max_worker_groups_per_gpu=self.max_worker_groups_per_gpu)

    def _eff_capacity(self) -> float:
        return (1 - self.eps_rt) * self.hw.memory_per_gpu

    def peak_bytes(self, node) -> float:
        """Isolated peak of an operator node (memory.py:273-288), from the GPU (`rpeg_op_time_batch`, the call the
        candidate directory makes for its mock nodes, moves.py:539-541)."""
        import numpy as np
        from .cost import NodeCostModel
        cm = NodeCostModel(self.hw, self.suite, self.workload, optimizer_stage=self.optimizer_stage,
                           activation_checkpointing=self.activation_checkpointing)
        v = node.op.template_vertex
        from ..search.evaluate import _engine_like
        try:
            eng, k, slot = _engine_like(None, None, suite=self.suite, workload=self.workload, vertex=v, hw=self.hw,
                                        policy=(self.optimizer_stage, self.activation_checkpointing))
        except LookupError:
            eng, k, slot = cm._engine_for_vertex(v, node)
        ext = node.allocs[0].extent
        row = np.array([[node.pi[0]], [node.pi[1]], [node.pi[2]], [node.mb or 1], [ext[0]], [ext[1]], [ext[2]]], np.int16)
        return float(eng.op_time(k, slot, row)[1][0])

    def is_locally_feasible(self, node) -> bool:
        return self.peak_bytes(node) <= self._eff_capacity()


_alloc_cache: dict = {}


def _alloc_devices(alloc) -> frozenset:
    """The devices of an allocation as the reference holds them (memory.py:582-604): a frozenset built from a set
    filled rack-major.  Its ITERATION order is what orders the reference's device dictionary, and with it which of
    several equally loaded devices `mem_worst_violation` names; building the same object in the same interpreter
    reproduces that order."""
    key = (alloc.origin, alloc.extent)
    hit = _alloc_cache.get(key)
    if hit is None:
        o, e = alloc.origin, alloc.extent
        devices = set()
        for r in range(o[0], o[0] + e[0]):
            for n in range(o[1], o[1] + e[1]):
                for g in range(o[2], o[2] + e[2]):
                    devices.add((r, n, g))
        hit = _alloc_cache[key] = frozenset(devices)
    return hit


def _device_peaks(executable, mem_model: NodeMemoryModel) -> dict:
    """peak(d) of every device that holds an operator node, in the reference's dictionary order
    (memory.py:608-841).  The peak of a device depends only on WHICH template vertices' allocations contain it;
    the GPU evaluates the peak of every such vertex set of the plan in one launch (`rpeg_plan_detail`), the host
    walks the devices in the reference's order -- operator nodes in graph order, each node's allocation in the
    iteration order of its device set -- and looks each one's set up."""
    from .cost import plan_detail_of
    src = getattr(executable, "source", None)
    if src is None:
        raise TypeError("expected the ExecutableRPEG that passes.lower.lower returned")
    key = ("memory", mem_model.hw, tuple(sorted((m.value, sp) for m, sp in mem_model.suite.specs.items())),
           mem_model.workload, mem_model.policy, mem_model.trainable)
    detail = plan_detail_of(executable, key, mem_model.suite, mem_model.workload, mem_model.hw, mem_model.policy,
                            mem_model.trainable)
    peaks_of_set = detail["set_peak"]
    slot = {v: i for i, v in enumerate(src.rpeg.vertices)}
    boxes = [(src.plan.sigma[v].origin, src.plan.sigma[v].extent) for v in src.rpeg.vertices]
    peaks: dict = {}
    seen_vertices = set()
    for node in executable.nodes:
        if node.kind != "op":
            continue
        v = node.op.template_vertex
        if v in seen_vertices:      # a later copy of the vertex inserts no new device
            continue
        seen_vertices.add(v)
        for alloc in node.allocs:
            for d in _alloc_devices(alloc):
                if d in peaks:
                    continue
                members = 0
                for i, (o, e) in enumerate(boxes):
                    if o[0] <= d[0] < o[0] + e[0] and o[1] <= d[1] < o[1] + e[1] and o[2] <= d[2] < o[2] + e[2]:
                        members |= 1 << i
                peaks[d] = float(peaks_of_set[members])
    return peaks


def mem_feasible(executable, mem_model: NodeMemoryModel) -> bool:
    cap = mem_model._eff_capacity()
    return all(not peak > cap for peak in _device_peaks(executable, mem_model).values())


def mem_worst_violation(executable, mem_model: NodeMemoryModel):
    """(device, peak_bytes, capacity_bytes) of the first device of largest peak among those above capacity, or
    None (memory.py:864-887)."""
    cap = mem_model._eff_capacity()
    worst_dev, worst_peak = None, 0.0
    for d, peak in _device_peaks(executable, mem_model).items():
        if peak > cap and peak > worst_peak:
            worst_dev, worst_peak = d, peak
    if worst_dev is None:
        return None
    return worst_dev, worst_peak, cap
