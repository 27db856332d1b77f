"""`lower(rpeg, unrolled, plan, suite, K_eval, workload)` under the reference's name (RPEG/passes/lower.py:330-851),
and the records it returns (`ExecNodeType`, `ExecNode`, `ExecEdge`, `ExecutableRPEG`, lower.py:20-119).

The graph is built by the library's own class lowering (`rpeg_lower_plan`: the plan's pair predicates packed into a
signature, the signature lowered as the engine lowers it for its kernels), so what `schedule()`, `NodeCostModel.time`
and `mem_worst_violation` later see is the graph the GPU evaluates: node order = insertion order of the reference's
`nodes` dict, edge order = append order of its `edges` list, ids, payloads and labels as the reference writes them.
It is integer work on the host and, like the reference's `lower()`, takes no hardware record and no device space."""

from __future__ import annotations

import ctypes as C
import weakref
from dataclasses import dataclass, field
from enum import Enum
from typing import Dict, Optional, Tuple

import numpy as np

from ..core.types import Allocation, DeviceSpace, Model, RPEG_TRANSFER_RESOURCE_POLICY
from ..engine import abi
from ..engine.compile import compile_problem, gen_phases
from ..engine.problem import EvalProblem, PlanBatch
from ..model.hardware import Hardware
from ..model.workload import Workload
from .unroll import UnrolledNode, UnrolledRPEG


class ExecNodeType(str, Enum):
    OP = "op"
    COMM = "comm"
    RESHARD = "reshard"


@dataclass(frozen=True, eq=False)
class ExecNode:
    id: str
    kind: ExecNodeType
    allocs: Tuple[Allocation, ...]
    op: Optional[UnrolledNode] = None
    model: Optional[Model] = None
    pi: Optional[Tuple[int, int, int]] = None
    mb: Optional[int] = None
    n_seqs: Optional[int] = None
    n_active: Optional[int] = None
    phase_steps: Optional[int] = None
    phase_t_start: Optional[int] = None
    is_prefill_phase: bool = False
    fusion_group: Optional[str] = None
    payload_in_bytes: int = 0
    label: Optional[str] = None
    # where the node sits in the graph lower() built it for: (weak reference to the ExecutableRPEG, index); None for a
    # node made by hand
    _home: Optional[tuple] = field(default=None, repr=False, compare=False)

    def __hash__(self):
        return hash(self.id)

    def __eq__(self, other):
        if not isinstance(other, ExecNode):
            return NotImplemented
        return self.id == other.id

    # the names evaluate() used for these before the reference's record was mirrored in full
    @property
    def template_vertex(self):
        return self.op.template_vertex if self.op is not None else None

    @property
    def k(self):
        return self.op.k if self.op is not None else None


@dataclass(frozen=True)
class ExecEdge:
    src: ExecNode
    dst: ExecNode


@dataclass(frozen=True)
class LoweringSource:
    """What lower() was called with: the graph's way back to the plan for schedule(), time() and the memory model."""
    rpeg: object
    plan: object
    suite: object
    K_eval: int
    workload: Optional[Workload]


@dataclass(frozen=True)
class ExecutableRPEG:
    nodes: Tuple[ExecNode, ...]
    edges: Tuple[ExecEdge, ...]
    composite_operators: tuple = ()
    source: Optional[LoweringSource] = field(default=None, repr=False, compare=False)


def node_id(x: UnrolledNode) -> str:
    return f"{x.template_vertex.id}@{x.k}" if x.i is None else f"{x.template_vertex.id}@{x.k}:{x.i}"


# lower() reads neither of these: any values do
_ANY_HW = Hardware(*([1.0] * 15))
_MODEL_BY_CODE = {code: Model(value) for value, code in abi.MODEL.items()}
_problems: Dict[tuple, tuple] = {}


def _lowering_problem(rpeg, plan, suite, K_eval, workload):
    """(compiled problem tables, structure, generation-split index) for the template of `rpeg`."""
    from ..search.evaluate import _structure_of
    st = _structure_of(rpeg)
    wl = workload if workload is not None else Workload(B=1, K=1, S=1, T=1, gen_quantiles=None)
    key = (st.name, tuple(sorted((m.value, s) for m, s in suite.specs.items())), wl, K_eval)
    hit = _problems.get(key)
    if hit is None:
        space = DeviceSpace(R=1 << 14, N=1 << 14, G=1 << 14)     # not read by the lowering
        problem = EvalProblem(structures=(st,), suite=suite, workload=wl, hw=_ANY_HW, device_space=space,
                              K_eval=K_eval, transfer_resource_policy=RPEG_TRANSFER_RESOURCE_POLICY)
        hit = _problems[key] = (compile_problem(problem, check_sizes=False), st)
        while len(_problems) > 32:
            _problems.pop(next(iter(_problems)))
    return hit[0], hit[1], (1 if wl.gen_quantiles else 0)


def lower(rpeg, unrolled: UnrolledRPEG, plan, suite, K_eval: int, workload: Optional[Workload] = None,
          intra_stage_fusion: bool = False, verbose: bool = False) -> ExecutableRPEG:
    from ..engine.runtime import load_library
    if intra_stage_fusion:
        raise NotImplementedError("intra_stage_fusion=True is not lowered by this engine")
    for v in rpeg.vertices:     # a vertex the plan does not cover raises KeyError, as lower.py:447-451 does
        plan.sigma[v], plan.pi[v]
    P, st, split = _lowering_problem(rpeg, plan, suite, K_eval, workload)
    batch = PlanBatch.empty(1)
    full = plan.mb if all(v in plan.mb for v in rpeg.vertices) else None
    if full is None:            # lower() itself takes a plan without micro-batch counts (`plan.mb.get`, lower.py:452)
        from ..ir.plan import ExecutionPlan
        packed = ExecutionPlan(sigma=plan.sigma, pi=plan.pi, mb={v: plan.mb.get(v) or 1 for v in rpeg.vertices})
    else:
        packed = plan
    batch.set_plan(0, 0, split, [int(rpeg.tau[m]) for m in st.tau_models], rpeg, packed)
    vert = np.ascontiguousarray(batch.vert[:, 0])
    head = np.ascontiguousarray(batch.head[:, 0])
    cap = 8192
    while True:
        kind, vertex, step, sub, src, ref = (np.zeros(cap, np.int32) for _ in range(6))
        payload = np.zeros(cap, np.int64)
        edges = np.zeros(2 * cap, np.int32)
        ne = C.c_int32(0)
        n = load_library().rpeg_lower_plan(C.addressof(P), vert.ctypes.data, head.ctypes.data, kind.ctypes.data,
                                           vertex.ctypes.data, step.ctypes.data, sub.ctypes.data, src.ctypes.data,
                                           payload.ctypes.data, ref.ctypes.data, edges.ctypes.data, C.addressof(ne), cap)
        if n != -7 or cap >= 1 << 20:
            break
        cap *= 8
    if n < 0:
        raise ValueError(f"rpeg_lower_plan failed with status {n}")
    phases = gen_phases(workload) if workload is not None and workload.gen_quantiles else []
    verts = rpeg.vertices
    copies: Dict[tuple, UnrolledNode] = {} if unrolled is None else {(x.template_vertex, x.k): x for x in unrolled.nodes}
    graph = ExecutableRPEG.__new__(ExecutableRPEG)
    home = weakref.ref(graph)      # (weak: a graph and its nodes must not keep each other alive in a cycle)
    nodes = []
    n_comm = n_reshard = 0
    for i in range(n):
        v = verts[vertex[i]]
        if kind[i] == 0:
            op = copies.get((v, int(step[i]))) or UnrolledNode(v, int(step[i]))
            more = {}
            tag = ""
            if sub[i] >= 0:
                n_act, n_seq, steps, t0, pf = phases[sub[i]]
                if v.kind.role.value == "GEN":
                    tag = f":g{sub[i]}"
                    more = dict(n_seqs=n_seq, n_active=n_act, phase_steps=steps, phase_t_start=t0, is_prefill_phase=pf)
                else:
                    tag = f":i{sub[i]}"
                    more = dict(n_seqs=n_seq)
            nodes.append(ExecNode(id=f"{v.id}@{step[i]}{tag}", kind=ExecNodeType.OP, allocs=(plan.sigma[v],), op=op,
                                  model=v.kind.model, pi=plan.pi[v], mb=plan.mb.get(v, None), _home=(home, i), **more))
            continue
        allocs = (plan.sigma[verts[src[i]]], plan.sigma[v])
        label = rpeg.data_edges[ref[i]].container.name if ref[i] < 16 else f"W_{_MODEL_BY_CODE[ref[i] - 16].value}"
        if kind[i] == 1:
            n_comm += 1
            nodes.append(ExecNode(id=f"comm{n_comm}", kind=ExecNodeType.COMM, allocs=allocs,
                                  payload_in_bytes=int(payload[i]), label=label, _home=(home, i)))
        else:
            n_reshard += 1
            nodes.append(ExecNode(id=f"reshard{n_reshard}", kind=ExecNodeType.RESHARD, allocs=allocs,
                                  model=_MODEL_BY_CODE[ref[i] - 16], payload_in_bytes=int(payload[i]), label=label,
                                  _home=(home, i)))
    pairs = edges[:2 * ne.value].reshape(-1, 2)
    object.__setattr__(graph, "nodes", tuple(nodes))
    object.__setattr__(graph, "edges", tuple(ExecEdge(nodes[a], nodes[b]) for a, b in pairs))
    object.__setattr__(graph, "composite_operators", ())
    object.__setattr__(graph, "source", LoweringSource(rpeg, plan, suite, K_eval, workload))
    if verbose:
        print(f"RPEG lowered successfully: {len(nodes)} nodes, {len(graph.edges)} edges.")
    return graph
