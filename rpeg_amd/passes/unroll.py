"""`unroll(rpeg, K_eval)` under the reference's name (RPEG/passes/unroll.py:85-152).

The evaluation engine never materialises this graph -- its class lowering goes from the template and the plan to the
lowered graph in one step -- but the reference's call sites build it and hand it to `lower()` (pipeline.py:1422-1426,
runtime/job_plan.py:174-183, search/optimizer.py:744-745), so the records exist here with the reference's fields:
operator copies (v, k) step-major in template order, the data edges of every step, and the publication edges
(u, max(0, k - tau - 1)) -> (v, k) for the steps k >= 1 with k > tau."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

from ..core.types import Container, EdgeKind, Model, TemplateVertex
from ..ir.rpeg import RPEG


@dataclass(frozen=True)
class UnrolledNode:
    template_vertex: TemplateVertex
    k: int
    i: Optional[int] = None


@dataclass(frozen=True)
class UnrolledEdge:
    src: UnrolledNode
    dst: UnrolledNode
    container: Container
    kind: EdgeKind


@dataclass(frozen=True)
class UnrolledRPEG:
    nodes: Tuple[UnrolledNode, ...]
    data_edges: Tuple[UnrolledEdge, ...]
    pub_edges: Tuple[UnrolledEdge, ...]


def publisher_selection(model: Model, tau: Dict[Model, int], k: int) -> int:
    """Step whose training output step k consumes (unroll.py:62-82)."""
    if model not in tau:
        raise ValueError(f"Missing staleness budget for trainable model {model.value}")
    t = tau[model]
    if isinstance(t, bool) or not isinstance(t, int) or t < 0:
        raise ValueError(f"Staleness budget for {model.value} must be a non-negative integer")
    return max(0, k - (t + 1))


def unroll(rpeg: RPEG, K_eval: int, verbose: bool = False) -> UnrolledRPEG:
    if K_eval <= 0:
        raise ValueError(f"K_eval must be >= 1, got {K_eval}.")
    rpeg.well_formed(verbose=False)
    copy = {(v, k): UnrolledNode(v, k) for k in range(K_eval) for v in rpeg.vertices}
    data = tuple(UnrolledEdge(copy[e.src, k], copy[e.dst, k], e.container, EdgeKind.DATA)
                 for k in range(K_eval) for e in rpeg.data_edges)
    pubs = tuple(UnrolledEdge(copy[e.src, publisher_selection(e.src.kind.model, rpeg.tau, k)], copy[e.dst, k],
                              e.container, EdgeKind.PUB)
                 for k in range(1, K_eval) for e in rpeg.pub_edges if k > rpeg.tau[e.src.kind.model])
    out = UnrolledRPEG(nodes=tuple(copy.values()), data_edges=data, pub_edges=pubs)
    if verbose:
        print(f"RPEG unrolled successfully for {K_eval} steps.")
        print(f"    Unrolled nodes: {len(out.nodes)}.")
        print(f"    Unrolled data edges: {len(out.data_edges)}.")
        print(f"    Unrolled publication edges: {len(out.pub_edges)}.")
    return out
