"""Strategy space and candidate directory of the simulated-annealing neighbourhood.

Mirrors the names of RPEG/search/moves.py for the part that runs before the annealing loop: the
enumeration of the proposal support (moves.py:97-176, 393-426) and `build_candidate_directory`
(moves.py:464-551), whose inner loop over mock nodes (moves.py:532-549) is one call of
rpeg_op_time_batch per vertex on the GPU.  The proposal kernels themselves (`move_gen`,
`multi_move_pair`) run inside rpeg_sa_run.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Tuple

import numpy as np

from ..core.types import DeviceSpace, TemplateVertex, packing_geometry, rectangular_node_layouts
from ..ir.rpeg import RPEG
from ..model.models import ModelSuite
from ..model.workload import Workload

MIN_B_LOCAL = 8  # moves.py:146


def valid_tp_degrees(G: int) -> List[int]:
    return [tp for tp in range(1, G + 1) if G % tp == 0]


def valid_pp_degrees(R: int, N: int, G: int, L: int) -> List[int]:
    """Divisors of L that are 1 or even (moves.py:109-122)."""
    return [d for d in range(1, R * N * G + 1) if L % d == 0 and (d == 1 or d % 2 == 0)]


def valid_dp_degrees(R: int, N: int, B: int, G: int = 1) -> List[int]:
    return [d for d in range(1, R * N * G + 1) if B % d == 0]


# moves.py:155-158: the ablation switches.  optimize() sets them from its OptimizerConfig as the reference does
# (optimizer.py:408-409), so that a directory built afterwards follows the same micro-batch rule as the
# proposals drawn inside rpeg_sa_optimize*.
ABLATION_FIXED_MB = False
ABLATION_UNIFORM_VERTEX = False


def valid_mb_counts(pp: int, dp: int, B: int) -> List[int]:
    """moves.py:162-199."""
    local = B // dp
    if local < MIN_B_LOCAL and dp > 1:
        return []
    if pp == 1:
        return [1]
    if ABLATION_FIXED_MB:
        return [1] if local % pp != 0 else [pp]
    max_mb = local // MIN_B_LOCAL
    return [mb for mb in range(pp, min(max_mb, local) + 1) if local % mb == 0]


def _enumerate_strategies(v: TemplateVertex, suite: ModelSuite, device_space: DeviceSpace,
                          workload: Workload) -> List[Tuple[int, int, int, int, int, int]]:
    """All (dp, pp, tp, r_ext, n_ext, mb) of the proposal support, in the reference's order."""
    R, N, G, B = device_space.R, device_space.N, device_space.G, workload.B
    L = suite.specs[v.kind.model].L
    out = []
    for tp in valid_tp_degrees(G):
        for pp in valid_pp_degrees(R, N, G, L):
            s = min(pp, G // tp)
            if pp % s != 0:
                continue
            for dp in valid_dp_degrees(R, N, B, G):
                mbs = valid_mb_counts(pp, dp, B)
                if not mbs:
                    continue
                geom = packing_geometry(dp, pp, tp, G)
                if geom is None:
                    continue
                for r_ext, n_ext in rectangular_node_layouts(geom[1], R, N):
                    for mb in mbs:
                        out.append((dp, pp, tp, r_ext, n_ext, mb))
    return out


def build_candidate_directory(rpeg: RPEG, suite: ModelSuite, device_space: DeviceSpace, workload: Workload,
                              engine, structure: int = 0, max_per_vertex: int = 1000):
    """(table, index) as the reference returns them: table[v] = [(dp, pp, tp, r_ext, n_ext, mb, time)]
    ascending by time, memory-infeasible strategies dropped; index[v][key] = position.

    `engine` is an rpeg_amd.engine.runtime.Engine for the same models, workload and hardware, and `structure`
    the index of the template of `rpeg` among its structures; together they take the place of the reference's
    (cost_model, mem_model) pair.  That pair -- a model.cost.NodeCostModel and a model.memory.NodeMemoryModel,
    as a call site written for the reference passes it -- is accepted as well and resolved to the engine."""
    from ..model.cost import NodeCostModel
    if isinstance(engine, NodeCostModel):
        engine, structure = engine.engine(rpeg, device_space, structure if not isinstance(structure, int) else None)
    table: Dict[TemplateVertex, List] = {}
    index: Dict[TemplateVertex, Dict] = {}
    cap = float(engine.P.cap)
    for slot, v in enumerate(rpeg.vertices):
        strategies = _enumerate_strategies(v, suite, device_space, workload)
        if not strategies:
            table[v], index[v] = [], {}
            continue
        s = np.asarray(strategies, dtype=np.int64)
        g_ext = np.asarray([packing_geometry(int(a), int(b), int(c), device_space.G)[0] for a, b, c in s[:, :3]])
        strat = np.stack([s[:, 0], s[:, 1], s[:, 2], s[:, 5], s[:, 3], s[:, 4], g_ext]).astype(np.int16)
        time, peak = engine.op_time(structure, slot, strat)
        keep = np.flatnonzero(~(peak > cap))
        order = keep[np.argsort(time[keep], kind="stable")][:max_per_vertex]
        table[v] = [tuple(int(x) for x in s[j]) + (float(time[j]),) for j in order]
        index[v] = {c[:6]: j for j, c in enumerate(table[v])}
    return table, index


def directory_arrays(rpeg: RPEG, table) -> List[np.ndarray]:
    """The directory as rpeg_sa_run takes it: per vertex an int16 array [n, 6]."""
    return [np.asarray([c[:6] for c in table[v]], dtype=np.int16).reshape(-1, 6) for v in rpeg.vertices]


# ----------------------------------------------------------------------------- the proposal kernels, one draw at a time
@dataclass
class MoveStats:
    """Counters a caller's annealing loop keeps across its move_gen / multi_move_pair calls (moves.py:36-95)."""
    n_calls: int = 0
    n_placement_proposed: int = 0
    n_strategy_proposed: int = 0
    n_fallback: int = 0
    n_empty: int = 0
    n_pair_proposed: int = 0
    n_pair_accepted: int = 0
    n_pair_failed: int = 0
    n_pair_rejected: int = 0

    def summary(self, n_accepted_strategy: int, n_accepted_placement: int, n_rejected_sv: int) -> str:
        single = self.n_placement_proposed + self.n_strategy_proposed
        rows = [("single-vertex", single, n_accepted_strategy + n_accepted_placement, n_rejected_sv, self.n_empty),
                ("  strategy", self.n_strategy_proposed, n_accepted_strategy, None, None),
                ("  placement", self.n_placement_proposed, n_accepted_placement, None, None),
                ("multi-vertex (pair)", self.n_pair_proposed, self.n_pair_accepted, self.n_pair_rejected, self.n_pair_failed)]
        out = [f"{'proposals':22s}{'proposed':>10s}{'accepted':>10s}{'rejected':>10s}{'failed':>8s}"]
        for name, a, b, c, d in rows:
            out.append(f"{name:22s}{a:10d}{b:10d}" + (f"{c:10d}{d:8d}" if c is not None else ""))
        return "\n".join(out)


def _stream_key():
    """Three words of Python's generator: the proposal kernels draw from the counter-based stream they name, so a
    caller who seeds `random` gets the same proposals again (not the draws MT19937 would have given the reference)."""
    import random
    return tuple(random.getrandbits(63) for _ in range(3))


def _params_for(eng, structure: int, directory, K_x: int = 6, T_max: int = 50, T_init: float = 0.30):
    from ..engine import abi
    p = abi.SaParamsT()
    p.structure, p.K_x, p.T_max, p.T_init = structure, K_x, T_max, T_init
    p.n_variants, p.seed = 1, 0
    p.fixed_mb, p.uniform_vertex = int(ABLATION_FIXED_MB), int(ABLATION_UNIFORM_VERTEX)
    return p


def critical_mass(config, executable, trace) -> Dict[TemplateVertex, float]:
    """Time per template vertex on the critical chain of a trace (moves.py:590-642): from the first node of
    largest finish time back along first predecessors of largest finish time, summing the operator nodes'
    durations by vertex."""
    preds: Dict[object, list] = {n: [] for n in executable.nodes}
    for e in executable.edges:
        preds[e.dst].append(e.src)
    mass = {v: 0.0 for v in config.rpeg.vertices}
    node = max(executable.nodes, key=lambda n: trace.finish[n])
    seen = set()
    while node not in seen:
        seen.add(node)
        if node.kind == "op":
            mass[node.template_vertex] += trace.finish[node] - trace.start[node]
        if not preds[node]:
            break
        node = max(preds[node], key=lambda n: trace.finish[n])
    return mass


def move_gen(config, executable, trace, table, index, K_x: int, T_max: int, T: float, T_init: float,
             stats: Optional[MoveStats] = None) -> list:
    """Drop-in for move_gen (moves.py:645-826): up to K_x neighbours of `config` that change one vertex -- one
    placement-only move and strategy moves from the temperature-dependent window of the directory `table` around
    the current strategy; the vertex is drawn with probability 0.6 by critical-chain mass of `trace`.  Runs the
    library's proposal kernel (rpeg_sa_propose) on an engine that has evaluated this template on this device
    space before (evaluate / evaluate_cached do that).  `index` is not needed: the kernel finds the position."""
    from .evaluate import Configuration, _engine_like
    from .optimizer import plan_row, row_plan
    eng, structure = _engine_like(config.rpeg, config.device_space)
    mass = critical_mass(config, executable, trace)
    params = _params_for(eng, structure, None, K_x, T_max, T_init)
    rows, _, fallback = eng.sa_propose(params, directory_arrays(config.rpeg, table), 0, _stream_key(),
                                       plan=plan_row(config.rpeg, config.plan),
                                       mass=[mass[v] for v in config.rpeg.vertices] + [0.0] * (8 - len(config.rpeg.vertices)), T=T)
    out = [Configuration(config.rpeg, row_plan(config.rpeg, r), config.device_space,
                         intra_stage_fusion=config.intra_stage_fusion,
                         transfer_resource_policy=config.transfer_resource_policy) for r in rows]
    if stats is not None:
        stats.n_calls += 1
        stats.n_fallback += int(fallback)
        stats.n_empty += not out
        for c in out:
            moved = any(c.plan.pi[v] != config.plan.pi[v] or c.plan.mb[v] != config.plan.mb[v] for v in config.rpeg.vertices)
            stats.n_strategy_proposed += moved
            stats.n_placement_proposed += not moved
    return out


def multi_move_pair(config, suite: ModelSuite, workload: Workload, max_retries: int = 100):
    """Drop-in for multi_move_pair (moves.py:845-1010): a donor vertex shrinks, a receiver grows into the freed
    devices; None when no such pair was found.  `max_retries` is the reference's default inside the library."""
    from .evaluate import Configuration, _engine_like
    from .optimizer import plan_row, row_plan
    if max_retries != 100:
        raise NotImplementedError("the proposal kernel tries 100 donor/receiver pairs, as the reference's default")
    eng, structure = _engine_like(config.rpeg, config.device_space, suite, workload)
    params = _params_for(eng, structure, None)
    rows, _, _ = eng.sa_propose(params, [], 1, _stream_key(), plan=plan_row(config.rpeg, config.plan))
    if len(rows) == 0:
        return None
    return Configuration(config.rpeg, row_plan(config.rpeg, rows[0]), config.device_space,
                         intra_stage_fusion=config.intra_stage_fusion,
                         transfer_resource_policy=config.transfer_resource_policy)


def sample_expl_in_region(v: TemplateVertex, suite: ModelSuite, device_space: DeviceSpace, workload: Workload,
                          r_lo: int = 0, r_hi: Optional[int] = None):
    """Drop-in for sample_expl_in_region (moves.py:202-296): a random valid (allocation, (dp, pp, tp), mb) of vertex
    `v` on racks [r_lo, r_hi), or None."""
    from ..core.types import Allocation
    from .evaluate import _engine_like
    eng, structure, slot = _engine_like(None, device_space, suite, workload, vertex=v)
    params = _params_for(eng, structure, None)
    rows, _, _ = eng.sa_propose(params, [], 2, _stream_key(), v=slot, r_lo=r_lo,
                                r_hi=device_space.R if r_hi is None else r_hi)
    if len(rows) == 0:
        return None
    f = [int(x) for x in rows[0]]
    return Allocation(origin=(f[4], f[5], f[6]), extent=(f[7], f[8], f[9])), (f[0], f[1], f[2]), f[3]


def sample_expl(v: TemplateVertex, suite: ModelSuite, device_space: DeviceSpace, workload: Workload):
    """moves.py:299-322: sample_expl_in_region over all racks."""
    return sample_expl_in_region(v, suite, device_space, workload)
