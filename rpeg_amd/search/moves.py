"""Strategy space and candidate directory of the simulated-annealing neighbourhood.

Mirrors the names of RPEG/search/moves.py for the part that runs before the annealing loop: the
enumeration of the proposal support (moves.py:97-176, 393-426) and `build_candidate_directory`
(moves.py:464-551), whose inner loop over mock nodes (moves.py:532-549) is one call of
rpeg_op_time_batch per vertex on the GPU.  The proposal kernels themselves (`move_gen`,
`multi_move_pair`) run inside rpeg_sa_run.
"""

from __future__ import annotations

from typing import Dict, List, Tuple

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

    `engine` is an rpeg_amd.engine.runtime.Engine for the same models, workload and hardware; it
    takes the place of the reference's (cost_model, mem_model) pair."""
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
