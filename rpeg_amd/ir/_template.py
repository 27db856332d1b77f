"""Table-driven construction of the four shipped step templates.

Each template is a short table: containers, then vertices (id, role, model, reads,
writes) in template order, then data and publication edges in template order.  Vertex
and edge ORDER is part of the semantics: node insertion order and edge order decide
scheduler ties downstream.
"""

from typing import Dict, Optional, Sequence, Tuple

from ..core.types import Container, EdgeKind, Model, OperatorKind, Role, TemplateEdge, TemplateVertex
from .rpeg import RPEG

_ROLE = {"g": Role.GENERATION, "i": Role.INFERENCE, "t": Role.TRAINING}


def assemble(containers: Dict[str, Container],
             listed: Sequence[str], inputs: Sequence[str],
             vertices: Sequence[Tuple[str, Model, Sequence[str], Sequence[str]]],
             data: Sequence[Tuple[str, str, str]], pubs: Sequence[Tuple[str, str, str]],
             trainable, tau: Optional[Dict[Model, int]], verbose: bool, title: str) -> RPEG:
    vs = {}
    for vid, model, reads, writes in vertices:
        kind = OperatorKind(role=_ROLE[vid[0]], model=model,
                            read=tuple(containers[c] for c in reads),
                            write=tuple(containers[c] for c in writes))
        vs[vid] = TemplateVertex(id=vid, kind=kind)
    d_edges = tuple(TemplateEdge(vs[a], vs[b], containers[c], EdgeKind.DATA) for a, b, c in data)
    p_edges = tuple(TemplateEdge(vs[a], vs[b], containers[c], EdgeKind.PUB) for a, b, c in pubs)
    if tau is None:
        tau = {m: 0 for m in sorted(trainable, key=lambda m: m.value)}
    g = RPEG(tuple(vs.values()), d_edges, p_edges, tuple(containers[c] for c in listed),
             tuple(containers[c] for c in inputs), (), tau, set(trainable))
    g.well_formed(verbose)
    if verbose:
        print(f"RPEG instantiated successfully for {title}.")
        print(f"    Template Nodes: {len(g.vertices)}.")
        print(f"    Data edges: {len(g.data_edges)}.")
        print(f"    Publication edges: {len(g.pub_edges)}.")
    return g


def two_byte(**counts: int) -> Dict[str, Container]:
    return {name: Container(name=name, count=n, elem_size_bytes=2) for name, n in counts.items()}
