"""Start plans of the reference's pipeline, built from the engine's candidate directory.

Each constructor takes the place of the reference function of the same name; the reference's
`(cost_model, mem_model)` pair becomes the `engine` (an rpeg_amd.engine.runtime.Engine for the same
models, workload and hardware), whose candidate directory holds per vertex the memory-feasible
strategies ascending by operator time.  A constructor may be handed that directory as `table` when the
caller already has it; otherwise it builds it with one batched launch per vertex.

  build_valid_baseline_plan            RPEG/pipeline.py:389-435
  build_fullycolocated_baseline_plan   RPEG/pipeline.py:1051-1108
  build_naive_concurrent_plan          RPEG/pipeline.py:1111-1201
  build_concurrent_baseline_plan       RPEG/pipeline.py:437-1048
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


# ----------------------------------------------------------------------------- topology-aware concurrent plan
def _find_concurrent_groups(rpeg: RPEG):
    """Vertices grouped by their longest-path depth over the data edges; the vertices of one depth do
    not depend on one another (RPEG/pipeline.py:437-487)."""
    parents = {v: [] for v in rpeg.vertices}
    for e in rpeg.data_edges:
        if e.src in parents and e.dst in parents:
            parents[e.dst].append(e.src)
    depth = {}

    def depth_of(v):
        if v not in depth:
            depth[v] = 1 + max((depth_of(p) for p in parents[v]), default=-1)
        return depth[v]

    groups = [[] for _ in range(1 + max((depth_of(v) for v in rpeg.vertices), default=0))]
    for v in rpeg.vertices:
        groups[depth[v]].append(v)
    return groups


def _pack_disjoint(sizes, R, N, G):
    """First-fit placement of blocks of `sizes` nodes, each aligned to its own size: along the nodes of a
    rack, then on to the next rack; blocks larger than a rack take whole racks (RPEG/pipeline.py:686-744).
    None when they do not fit."""
    out, rack, node = [], 0, 0
    for n_nodes in sizes:
        if n_nodes > N:
            racks = -(-n_nodes // N)
            if node > 0:
                rack, node = rack + 1, 0
            rack += -rack % racks
            if rack + racks > R:
                return None
            out.append(Allocation(origin=(rack, 0, 0), extent=(racks, N, G)))
            rack, node = rack + racks, 0
        else:
            node += -node % n_nodes
            if node + n_nodes > N:
                rack, node = rack + 1, 0
            if rack >= R:
                return None
            out.append(Allocation(origin=(rack, node, 0), extent=(1, n_nodes, G)))
            node += n_nodes
    return out


def _enumerate_group_partitions(group, device_space: DeviceSpace):
    """Candidate device partitions of one group, one allocation per member and in the reference's order:
    everybody on the whole space; for two or three members every split into power-of-two node counts
    (each extent pattern once), for two also the two halves of every node, for three also one member
    alone beside the other two sharing a block; for more, a node each (RPEG/pipeline.py:640-849).
    Members holding the same allocation run one after the other."""
    from itertools import permutations
    R, N, G = device_space.R, device_space.N, device_space.G
    k = len(group)
    partitions = [[Allocation(origin=(0, 0, 0), extent=(R, N, G))] * k]
    if k == 1:
        return partitions
    total = R * N
    sizes = [1 << i for i in range(total.bit_length()) if (1 << i) <= total]
    seen = set()

    def disjoint(sz):
        packed = _pack_disjoint(sz, R, N, G)
        if packed is None:
            return
        for perm in permutations(range(k)):
            key = tuple(packed[perm[i]].extent for i in range(k))
            if key not in seen:
                seen.add(key)
                partitions.append([packed[perm[i]] for i in range(k)])

    def one_alone(s_solo, s_shared):
        packed = _pack_disjoint([s_solo, s_shared], R, N, G)
        if packed is None:
            return
        for solo in range(k):
            part = [packed[1]] * k
            part[solo] = packed[0]
            key = tuple(a.extent for a in part) + (solo,)
            if key in seen:
                continue
            seen.add(key)
            partitions.append(part)
            swapped = _pack_disjoint([s_shared, s_solo], R, N, G)
            if swapped is None:
                continue
            part = [swapped[1]] * k
            part[solo] = swapped[0]
            key = tuple(a.extent for a in part) + (solo,)
            if key not in seen:
                seen.add(key)
                partitions.append(part)

    if k == 2:
        for s1 in sizes:
            for s2 in sizes:
                if s1 + s2 <= total:
                    disjoint([s1, s2])
        if G >= 4 and G % 2 == 0:
            half = G // 2
            for r in range(R):
                for n in range(N):
                    a = Allocation(origin=(r, n, 0), extent=(1, 1, half))
                    b = Allocation(origin=(r, n, half), extent=(1, 1, half))
                    partitions += [[a, b], [b, a]]
    elif k == 3:
        for s1 in sizes:
            for s2 in sizes:
                if s1 + s2 > total:
                    continue
                for s3 in sizes:
                    if s1 + s2 + s3 <= total:
                        disjoint([s1, s2, s3])
        for s_solo in sizes:
            for s_shared in sizes:
                if s_solo + s_shared <= total:
                    one_alone(s_solo, s_shared)
    elif total >= k:
        partitions.append([Allocation(origin=(r, n, 0), extent=(1, 1, G)) for r in range(R) for n in range(N)][:k])
    return partitions


def _best_strategy_in_alloc(v, table, alloc: Allocation, G: int):
    """Fastest directory entry of `v` whose extent fits inside `alloc`, placed at the allocation's origin
    (RPEG/pipeline.py:578-637; its per-entry memory check repeats the test every directory entry has
    already passed, RPEG/search/moves.py:540-542, and is not repeated here)."""
    for dp, pp, tp, r_ext, n_ext, mb_v, t in table[v]:
        if r_ext > alloc.extent[0] or n_ext > alloc.extent[1]:
            continue
        geom = packing_geometry(dp, pp, tp, G)
        if geom is None or geom[0] > alloc.extent[2]:
            continue
        return dp, pp, tp, mb_v, t, Allocation(origin=alloc.origin, extent=(r_ext, n_ext, geom[0]))
    return None


def _score_group_partition(group, allocs, table, G: int):
    """(estimated time, {vertex: (dp, pp, tp, mb, allocation)}) of one partition: members of one
    allocation add up, allocations run side by side (RPEG/pipeline.py:852-905); (inf, None) when a
    member has no entry that fits."""
    by_alloc = {}
    for v, a in zip(group, allocs):
        by_alloc.setdefault(a, []).append(v)
    assign, times = {}, []
    for alloc, members in by_alloc.items():
        serial = 0.0
        for v in members:
            best = _best_strategy_in_alloc(v, table, alloc, G)
            if best is None:
                return float("inf"), None
            assign[v] = best[:4] + (best[5],)
            serial += best[4]
        times.append(serial)
    return max(times), assign


def concurrent_plan_cascade(rpeg: RPEG, device_space: DeviceSpace, table):
    """The plans `build_concurrent_baseline_plan` would try, in its order, or None where a group has no
    feasible partition.  Per group the partitions are ranked by the number of distinct allocations
    (more first), then by estimated time (stable); the first plan takes every group's best one, and each
    further plan moves the first group that still has a next partition one rank down
    (RPEG/pipeline.py:952-1045).  Returns [(ExecutionPlan, estimated time, [label per group])]."""
    groups = _find_concurrent_groups(rpeg)
    ranked = []
    for group in groups:
        cands = []
        for allocs in _enumerate_group_partitions(group, device_space):
            t, assign = _score_group_partition(group, allocs, table, device_space.G)
            if assign is None:
                continue
            ways = len(set(allocs))
            cands.append((-ways, t, assign, "serialized" if ways == 1 else f"{ways}-way concurrent"))
        if not cands:
            return None
        cands.sort(key=lambda c: (c[0], c[1]))
        ranked.append(cands)
    at = [0] * len(groups)
    plans = []
    while True:
        sigma, pi, mb, total = {}, {}, {}, 0.0
        for gi in range(len(groups)):
            _, t, assign, _ = ranked[gi][at[gi]]
            total += t
            for v, (dp, pp, tp, mb_v, alloc) in assign.items():
                sigma[v], pi[v], mb[v] = alloc, (dp, pp, tp), mb_v
        plans.append((ExecutionPlan(sigma, pi, mb), total, [ranked[gi][at[gi]][3] for gi in range(len(groups))]))
        for gi in range(len(groups)):
            if at[gi] + 1 < len(ranked[gi]):
                at[gi] += 1
                break
        else:
            return plans


def build_concurrent_baseline_plan(rpeg: RPEG, device_space: DeviceSpace, suite: ModelSuite, workload: Workload,
                                   engine, table=None, structure: int = 0):
    """(plan, found): the first plan of `concurrent_plan_cascade` that fits in device memory, or the greedy
    plan and False when a group cannot be placed or no plan fits (RPEG/pipeline.py:908-1048).

    The reference lowers and checks one plan after the other and stops at the first that fits; the order
    of its attempts does not depend on their outcome, so here the whole cascade is one batch through the
    engine and the first plan whose memory bit is set is returned.  The memory peak of a plan is a
    property of its template vertices and does not change with the number of unrolled steps, hence the
    engine's K_eval stands in for the reference's K = 1 lowering of this check."""
    from ..engine import abi
    from ..engine.problem import PlanBatch
    table = _directory(rpeg, suite, device_space, workload, engine, table)
    cascade = concurrent_plan_cascade(rpeg, device_space, table)
    if cascade:
        st = engine.problem.structures[structure]
        batch = PlanBatch.empty(len(cascade))
        taus = [int(rpeg.tau[m]) for m in st.tau_models]
        for i, (plan, _, _) in enumerate(cascade):
            batch.set_plan(i, structure, 1 if workload.gen_quantiles else 0, taus, rpeg, plan)
        mask = engine.eval(batch, gate_stale=False)["mask"]
        if ((mask & abi.MASK_VALID) == 0).any():
            raise ValueError("a cascade plan violates the integer validity rules of is_valid")
        fits = (mask & abi.MASK_MEM_OK) != 0
        if fits.any():
            return cascade[int(fits.argmax())][0], True
    return build_valid_baseline_plan(rpeg, device_space, suite, workload, engine, table=table), False
