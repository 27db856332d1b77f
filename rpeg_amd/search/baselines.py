"""Start plans of the reference's pipeline, built from the engine's candidate directory.

Each constructor takes the place of the reference function of the same name; the reference's
`(cost_model, mem_model)` pair becomes the `engine` (an rpeg_amd.engine.runtime.Engine for the same
models, workload and hardware), whose candidate directory holds per vertex the memory-feasible
strategies ascending by operator time.  A constructor may be handed that directory as `table` when the
caller already has it; otherwise it builds it with one batched launch per vertex.

  build_valid_baseline_plan            RPEG/pipeline.py:389-435
  build_fullycolocated_baseline_plan   RPEG/pipeline.py:1051-1108
  build_naive_concurrent_plan          RPEG/pipeline.py:1111-1201
"""

from __future__ import annotations

from ..core.types import Allocation, DeviceSpace, Model, Role, packing_geometry
from ..ir.plan import ExecutionPlan
from ..ir.rpeg import RPEG
from ..model.models import ModelSuite
from ..model.workload import Workload
from .moves import build_candidate_directory


def _directory(rpeg, suite, device_space, workload, engine, table):
    if table is not None:
        return table
    return build_candidate_directory(rpeg, suite, device_space, workload, engine)[0]


def build_valid_baseline_plan(rpeg: RPEG, device_space: DeviceSpace, suite: ModelSuite, workload: Workload,
                              engine, table=None) -> ExecutionPlan:
    """Greedy start plan: every vertex takes its fastest memory-feasible strategy, placed at the origin
    of the device space (RPEG/pipeline.py:389-435).  RuntimeError when a vertex has no candidate."""
    table = _directory(rpeg, suite, device_space, workload, engine, table)
    sigma, pi, mb = {}, {}, {}
    for v in rpeg.vertices:
        if not table[v]:
            raise RuntimeError(f"No valid candidates for vertex {v.id}; cannot construct baseline plan")
        dp, pp, tp, r_ext, n_ext, mb_v, _ = table[v][0]
        geom = packing_geometry(dp, pp, tp, device_space.G)
        g_ext = geom[0] if geom else min(pp, device_space.G // tp) * tp
        sigma[v] = Allocation(origin=(0, 0, 0), extent=(r_ext, n_ext, g_ext))
        pi[v] = (dp, pp, tp)
        mb[v] = mb_v
    return ExecutionPlan(sigma, pi, mb)


def build_fullycolocated_baseline_plan(rpeg: RPEG, device_space: DeviceSpace, suite: ModelSuite,
                                       workload: Workload, engine, table=None) -> ExecutionPlan:
    """Every vertex on the whole device space, hence no two vertices at a time: per vertex the fastest
    directory entry whose extent is all racks, all nodes and all devices of a node
    (RPEG/pipeline.py:1051-1108).  RuntimeError when a vertex has no such entry."""
    table = _directory(rpeg, suite, device_space, workload, engine, table)
    R, N, G = device_space.R, device_space.N, device_space.G
    sigma, pi, mb = {}, {}, {}
    for v in rpeg.vertices:
        for dp, pp, tp, r_ext, n_ext, mb_v, _ in table[v]:
            geom = packing_geometry(dp, pp, tp, G)
            if geom is not None and (r_ext, n_ext, geom[0]) == (R, N, G):
                break
        else:
            raise RuntimeError(f"No valid full-device strategy for vertex {v.id} in "
                               f"({R}×{N}×{G}); cannot construct fully-colocated baseline")
        sigma[v] = Allocation(origin=(0, 0, 0), extent=(R, N, G))
        pi[v] = (dp, pp, tp)
        mb[v] = mb_v
    return ExecutionPlan(sigma, pi, mb)


def _hand_partition(rpeg: RPEG, device_space: DeviceSpace):
    """The fixed split of RPEG/pipeline.py:1150-1173: generation and the reference model's inference on
    every device, the reward model's inference and the actor's training on the lower half of each node's
    devices, the critic's inference and every other training on the upper half."""
    R, N, G = device_space.R, device_space.N, device_space.G
    half = G // 2
    full = Allocation(origin=(0, 0, 0), extent=(R, N, G))
    lo = Allocation(origin=(0, 0, 0), extent=(R, N, half))
    hi = Allocation(origin=(0, 0, half), extent=(R, N, half))
    assign = {}
    for v in rpeg.vertices:
        role, model = v.kind.role, v.kind.model
        if role == Role.GENERATION:
            assign[v] = full
        elif role == Role.INFERENCE:
            assign[v] = lo if model == Model.REWARD else hi if model == Model.CRITIC else full
        elif role == Role.TRAINING:
            assign[v] = lo if model == Model.ACTOR else hi
    return assign


def build_naive_concurrent_plan(rpeg: RPEG, device_space: DeviceSpace, suite: ModelSuite, workload: Workload,
                                engine, table=None) -> ExecutionPlan:
    """Hand-partitioned concurrent plan: each vertex is given the allocation of `_hand_partition` and the
    fastest directory entry whose extent fits inside it; the plan records the whole assigned allocation,
    not the entry's own extent (RPEG/pipeline.py:1111-1201).  RuntimeError when nothing fits."""
    table = _directory(rpeg, suite, device_space, workload, engine, table)
    G = device_space.G
    assign = _hand_partition(rpeg, device_space)
    sigma, pi, mb = {}, {}, {}
    for v in rpeg.vertices:
        alloc = assign[v]
        for dp, pp, tp, r_ext, n_ext, mb_v, _ in table[v]:
            geom = packing_geometry(dp, pp, tp, G)
            if geom is not None and r_ext <= alloc.extent[0] and n_ext <= alloc.extent[1] and geom[0] <= alloc.extent[2]:
                break
        else:
            raise RuntimeError(f"No feasible strategy for {v.id} on allocation "
                               f"{alloc.extent}; cannot build naive concurrent plan")
        sigma[v] = alloc
        pi[v] = (dp, pp, tp)
        mb[v] = mb_v
    return ExecutionPlan(sigma, pi, mb)
