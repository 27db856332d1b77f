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
        """NodeCostModel.time(node) (cost.py:66-88), computed on the GPU.

        A node of a graph that `passes.lower.lower` built: the engine evaluates the duration of every node of that
        plan in one launch (`rpeg_plan_detail`); the result is kept with the graph, so asking for all nodes of a
        graph costs one launch.  An operator node made by hand without quantile fields (the mock node of the
        candidate directory, moves.py:439-485): one `rpeg_op_time_batch` call.  Raises ZeroDivisionError where the
        reference does (a degenerate phase), ValueError for a node the engine cannot place."""
        home = getattr(node, "_home", None)
        if home is not None:
            graph, index = home[0](), home[1]
            if graph is None:
                raise ValueError("the lowered graph this node belongs to no longer exists")
            t = float(_graph_detail(self, graph)["time"][index])
        else:
            t = self._mock_time(node)
        if t != t:
            raise ZeroDivisionError("float division by zero")
        return t

    def _mock_time(self, node) -> float:
        import numpy as np
        from ..core.types import DeviceSpace
        from ..search.evaluate import _engine_like
        kind = getattr(node.kind, "value", node.kind)
        if kind != "op":
            raise ValueError("time() of a COMM or RESHARD node needs the graph it was lowered into: take the node "
                             "from passes.lower.lower(...).nodes")
        if node.n_seqs is not None or node.n_active is not None:
            raise ValueError("time() of a quantile sub-node needs the graph it was lowered into: take the node from "
                             "passes.lower.lower(...).nodes")
        v = node.op.template_vertex
        ext = node.allocs[0].extent
        dp, pp, tp = node.pi
        try:
            eng, k, slot = _engine_like(None, None, suite=self.suite, workload=self.workload, vertex=v, hw=self.hw,
                                        policy=(self.optimizer_stage, self.activation_checkpointing))
        except LookupError:
            eng, k, slot = self._engine_for_vertex(v, node)
        row = np.array([[dp], [pp], [tp], [node.mb or 1], [ext[0]], [ext[1]], [ext[2]]], np.int16)
        return float(eng.op_time(k, slot, row)[0][0])


    def _engine_for_vertex(self, v, node):
        """An engine (a new one) for the first shipped template that holds vertex `v` and that this cost model's
        suite can build: the duration of an operator node depends on its vertex, not on the template around it."""
        from ..core.types import DeviceSpace
        from ..engine.problem import STRUCTURES
        from ..search.evaluate import _TEMPLATE_IDS, _engine_for
        from .memory import MemoryPolicy
        o, e = node.allocs[0].origin, node.allocs[0].extent
        space = DeviceSpace(R=o[0] + e[0], N=o[1] + e[1], G=max(o[2] + e[2], node.pi[2]))
        policy = MemoryPolicy(optimizer_stage=self.optimizer_stage, activation_checkpointing=self.activation_checkpointing)
        for name, ids in _TEMPLATE_IDS.items():
            if v.id not in ids:
                continue
            st = STRUCTURES[name]
            try:
                rpeg = st.build(self.suite, self.workload, tau={m: 0 for m in st.tau_models})
            except (KeyError, ValueError):
                continue
            eng, _ = _engine_for(rpeg, self.suite, self.workload, self.hw, space, 1, policy)
            return eng, 0, ids.index(v.id)
        raise ValueError(f"no shipped template holds vertex {v.id!r} for this model suite")


def _graph_detail(cost_model: NodeCostModel, graph):
    """Per-node durations (and vertex-set peaks) of a lowered graph under `cost_model`, kept with the graph."""
    from ..model.memory import MemoryPolicy
    key = ("cost", cost_model.hw, tuple(sorted((m.value, sp) for m, sp in cost_model.suite.specs.items())),
           cost_model.workload, cost_model.optimizer_stage, cost_model.activation_checkpointing)
    return plan_detail_of(graph, key, cost_model.suite, cost_model.workload, cost_model.hw,
                          MemoryPolicy(optimizer_stage=cost_model.optimizer_stage,
                                       activation_checkpointing=cost_model.activation_checkpointing), None)


_detail_cache: dict = {}     # id(graph) -> (graph, {key: detail}); graphs are kept alive by their own entries only briefly


def plan_detail_of(graph, key, suite, workload, hw, policy, trainable):
    """rpeg_plan_detail of the plan behind `graph` on an engine for (suite, workload, hw, policy); one launch per
    (graph, key), remembered for the last few graphs."""
    from ..schedule.scheduler import plan_batch_of
    from ..search.evaluate import _engine_for, _engine_space_for
    src = getattr(graph, "source", None)
    if src is None:
        raise TypeError("expected the ExecutableRPEG that passes.lower.lower returned")
    slot = _detail_cache.get(id(graph))
    if slot is None or slot[0] is not graph:
        slot = _detail_cache[id(graph)] = (graph, {})
        while len(_detail_cache) > 8:
            _detail_cache.pop(next(iter(_detail_cache)))
    hit = slot[1].get(key)
    if hit is None:
        if src.workload is not None and src.workload != workload:
            raise ValueError("the graph was lowered for another workload than the model's")
        space = _engine_space_for(src.rpeg, src.plan, suite, workload, hw)
        eng, st = _engine_for(src.rpeg, suite, workload, hw, space, src.K_eval, policy, memory_trainable=trainable)
        hit = slot[1][key] = eng.plan_detail(plan_batch_of(graph, st), 0, cap=max(4096, len(graph.nodes)))
        hit["space"] = space
    return hit
