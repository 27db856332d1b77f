"""`schedule(executable, cost_model, device_space, *, transfer_resource_policy)` under the reference's name
(RPEG/schedule/scheduler.py:270-552; called at pipeline.py:1479, 1497 and runtime/job_plan.py:183-213).

`executable` is the graph `passes.lower.lower` returned.  The list scheduling itself -- durations, ranks, the
heap's dispatch order, device availability -- runs on the GPU (`rpeg_eval_trace`); this function hands the plan
behind the graph to the engine for the cost model's hardware and the caller's device space and keys the times by
the graph's own nodes, in dispatch order as the reference fills its dictionaries."""

from __future__ import annotations

from ..core.types import DeviceSpace, RPEG_TRANSFER_RESOURCE_POLICY, TransferResourcePolicy
from ..engine.problem import PlanBatch
from .trace import Trace


def plan_batch_of(executable, st):
    """The one-plan tensor of the plan a lowered graph was built from."""
    src = executable.source
    batch = PlanBatch.empty(1)
    split = 1 if src.workload is not None and src.workload.gen_quantiles else 0
    if any(v not in src.plan.mb for v in src.rpeg.vertices):
        raise KeyError("plan.mb misses a template vertex")
    batch.set_plan(0, 0, split, [int(src.rpeg.tau[m]) for m in st.tau_models], src.rpeg, src.plan)
    return batch


def trace_on(eng, executable, batch) -> Trace:
    """Trace of the one plan of `batch` on engine `eng`, keyed by the nodes of `executable` (its lowered graph)."""
    tr = eng.trace(batch, 0, cap=max(4096, len(executable.nodes)))
    nodes = executable.nodes
    if len(tr["start"]) != len(nodes):
        raise ValueError("the lowered graph does not belong to this plan")
    by_dispatch = sorted(range(len(nodes)), key=lambda i: int(tr["order"][i]))   # scheduler.py:517-518
    start = {nodes[i]: float(tr["start"][i]) for i in by_dispatch}
    finish = {nodes[i]: float(tr["finish"][i]) for i in by_dispatch}
    # the allocations the scheduler reserved: of a node's allocations (source first) those whose vertex the engine
    # reserved, identical allocations once (transfer_resources.py:138-148)
    sigma = executable.source.plan.sigma
    verts = executable.source.rpeg.vertices
    reserved = {}
    for i, node in enumerate(nodes):
        mask = int(tr["reserved"][i])
        owners = (int(tr["vertex"][i]),) if tr["kind"][i] == 0 else (int(tr["src"][i]), int(tr["vertex"][i]))
        reserved[node] = tuple(dict.fromkeys(sigma[verts[x]] for x in owners if (mask >> x) & 1))
    return Trace(start=start, finish=finish, reserved_allocations=reserved)


def schedule(executable, cost_model, device_space: DeviceSpace, *,
             transfer_resource_policy: TransferResourcePolicy = RPEG_TRANSFER_RESOURCE_POLICY) -> Trace:
    from ..model.memory import MemoryPolicy
    from ..search.evaluate import _engine_for
    src = getattr(executable, "source", None)
    if src is None:
        raise TypeError("schedule() takes the ExecutableRPEG that passes.lower.lower returned")
    if src.workload is not None and src.workload != cost_model.workload:
        raise ValueError("the graph was lowered for another workload than the cost model's")
    policy = MemoryPolicy(optimizer_stage=cost_model.optimizer_stage,
                          activation_checkpointing=cost_model.activation_checkpointing)
    eng, st = _engine_for(src.rpeg, cost_model.suite, cost_model.workload, cost_model.hw, device_space, src.K_eval,
                          policy, transfer_policy=transfer_resource_policy)
    return trace_on(eng, executable, plan_batch_of(executable, st))
