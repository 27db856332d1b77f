"""Seeded candidate plan sets for batched evaluation.

Candidates are drawn with a counter-based generator: every random choice is a pure function
of (seed, configuration tag, plan index, vertex slot, field), so any subset of a candidate
set can be regenerated independently and in any order, on the host or on the device.

Per vertex, the strategy (dp, pp, tp, r_ext, n_ext, g_ext) is uniform over the strategy space
the reference's simulated-annealing neighbourhood enumerates (RPEG/search/moves.py:97-152,
393-436: tp divides G; pp divides L and is 1 or even; dp divides B; packing geometry and
rectangular layouts from RPEG/core/types.py:16-85) without its memory and minimum-local-batch
filters, so memory-infeasible candidates occur.  The origin is uniform over aligned origins
(moves.py:709-722), the microbatch count uniform over the powers of two up to 64 that
`is_valid` (RPEG/search/evaluate.py:186-192) accepts, staleness uniform over the configured
set, and the generation-split index uniform over 0..Q.
"""

from __future__ import annotations

from typing import Dict, Sequence

import numpy as np

from ..core.types import packing_geometry, rectangular_node_layouts
from ..engine.problem import (EvalProblem, PlanBatch, FIELDS_PER_VERTEX, F_DP, F_PP, F_TP, F_MB,
                              F_OR, F_ON, F_OG, F_ER, F_EN, F_EG)

_U64 = np.uint64
_GOLD = _U64(0x9E3779B97F4A7C15)


def mix64(x: np.ndarray) -> np.ndarray:
    """splitmix64 finalizer on uint64 arrays (wrapping arithmetic)."""
    x = np.asarray(x, dtype=_U64)
    with np.errstate(over="ignore"):
        x = (x ^ (x >> _U64(30))) * _U64(0xBF58476D1CE4E5B9)
        x = (x ^ (x >> _U64(27))) * _U64(0x94D049BB133111EB)
        return x ^ (x >> _U64(31))


def draw(seed: int, tag: int, index: np.ndarray, slot: int, fld: int) -> np.ndarray:
    """uint64 random word for (seed, tag, index, slot, field)."""
    with np.errstate(over="ignore"):
        h = mix64(np.asarray([seed], _U64) + _GOLD * _U64(tag + 1))
        h = mix64(h + _GOLD * (np.asarray(index, _U64) + _U64(1)))
        return mix64(h + _GOLD * _U64(slot * 16 + fld + 1))


def pick(word: np.ndarray, n) -> np.ndarray:
    """Uniform index in [0, n) from a random word (multiply-shift on the top 32 bits)."""
    return ((word >> _U64(32)) * np.asarray(n, _U64)) >> _U64(32)


def strategy_space(L: int, B: int, R: int, N: int, G: int) -> np.ndarray:
    """All (dp, pp, tp, r_ext, n_ext, g_ext) the neighbourhood can reach for a model of L layers."""
    total = R * N * G
    out = []
    for tp in (t for t in range(1, G + 1) if G % t == 0):
        for pp in (p for p in range(1, total + 1) if L % p == 0 and (p == 1 or p % 2 == 0)):
            s = min(pp, G // tp)
            if pp % s:
                continue
            for dp in (d for d in range(1, total + 1) if B % d == 0):
                geom = packing_geometry(dp, pp, tp, G)
                if geom is None:
                    continue
                for r_ext, n_ext in rectangular_node_layouts(geom[1], R, N):
                    out.append((dp, pp, tp, r_ext, n_ext, geom[0]))
    return np.asarray(out, dtype=np.int64).reshape(-1, 6)


def generate(problem: EvalProblem, n: int, tau_choices: Dict[str, Sequence[Sequence[int]]],
             seed: int = 42, tag: int = 0, start: int = 0) -> PlanBatch:
    """Candidates start .. start+n-1 of the seeded set `tag` for `problem`."""
    sp = problem.device_space
    B = problem.workload.B
    idx = np.arange(start, start + n, dtype=np.int64)
    batch = PlanBatch.empty(n)
    n_struct = len(problem.structures)
    struct = pick(draw(seed, tag, idx, 15, 0), n_struct).astype(np.int64)
    split = pick(draw(seed, tag, idx, 15, 1), problem.n_splits()).astype(np.int64)
    batch.head[0] = struct
    for s, st in enumerate(problem.structures):
        sel = struct == s
        rpeg = problem.template(s)
        has_gen = any(v.kind.role.value == "GEN" for v in rpeg.vertices)
        batch.head[1, sel] = split[sel] if has_gen else 0
        for t, choices in enumerate(tau_choices[st.name]):
            c = np.asarray(choices, dtype=np.int64)
            batch.head[2 + t, sel] = c[pick(draw(seed, tag, idx, 15, 2 + t), len(c)).astype(np.int64)][sel]
        for slot, v in enumerate(rpeg.vertices):
            space = strategy_space(problem.suite.specs[v.kind.model].L, B, sp.R, sp.N, sp.G)
            strat = space[pick(draw(seed, tag, idx, slot, 0), len(space)).astype(np.int64)]
            dp, pp, tp, er, en, eg = (strat[:, k] for k in range(6))
            o_r = pick(draw(seed, tag, idx, slot, 1), sp.R // er).astype(np.int64) * er
            o_n = pick(draw(seed, tag, idx, slot, 2), sp.N // en).astype(np.int64) * en
            o_g = pick(draw(seed, tag, idx, slot, 3), sp.G // eg).astype(np.int64) * eg
            local = B // dp
            n_mb = np.ones(n, np.int64)
            for e in range(1, 7):
                n_mb += ((local % (1 << e)) == 0) & (n_mb == e)
            mb = np.where(pp == 1, 1, 1 << pick(draw(seed, tag, idx, slot, 4), n_mb).astype(np.int64))
            rows = {F_DP: dp, F_PP: pp, F_TP: tp, F_MB: mb, F_OR: o_r, F_ON: o_n, F_OG: o_g,
                    F_ER: er, F_EN: en, F_EG: eg}
            for f, val in rows.items():
                batch.vert[slot * FIELDS_PER_VERTEX + f, sel] = val[sel]
    return batch
