"""Template graph of one RL post-training step (mirror of RPEG/ir/rpeg.py:23-186)."""

from dataclasses import dataclass
from typing import Dict, Set, Tuple

from ..core.types import Container, EdgeKind, Model, Role, TemplateEdge, TemplateVertex


class RPEGError(ValueError):
    pass


def _names(models) -> list:
    return [m.value for m in sorted(models, key=lambda m: m.value)]


@dataclass(frozen=True)
class RPEG:
    vertices: Tuple[TemplateVertex, ...]
    data_edges: Tuple[TemplateEdge, ...]
    pub_edges: Tuple[TemplateEdge, ...]
    containers: Tuple[Container, ...]
    in_containers: Tuple[Container, ...]
    out_containers: Tuple[Container, ...]
    tau: Dict[Model, int]
    trainable: Set[Model]

    def well_formed(self, verbose: bool) -> None:
        """Raise RPEGError unless interfaces, boundary containers, publication edges and the
        within-step DAG property hold (same checks and order as RPEG/ir/rpeg.py:37-186)."""
        ids = [v.id for v in self.vertices]
        for i, vid in enumerate(ids):
            if vid in ids[:i]:
                raise RPEGError(f"Duplicate vertex id: {vid}")
        known_v, known_c = set(self.vertices), set(self.containers)
        every = self.data_edges + self.pub_edges
        for e in every:
            if e.src not in known_v:
                raise RPEGError(f"Edge src vertex {e.src.id} not in RPEG.vertices")
            if e.dst not in known_v:
                raise RPEGError(f"Edge dst vertex {e.dst.id} not in RPEG.vertices")
            if e.container not in known_c:
                raise RPEGError(f"Undeclared container {e.container} on edge {e.src.id}->{e.dst.id}")
        if set(self.tau) != set(self.trainable):
            raise RPEGError("tau/trainable mismatch: "
                            f"missing={_names(set(self.trainable) - set(self.tau))}, "
                            f"extra={_names(set(self.tau) - set(self.trainable))}")
        for model, budget in self.tau.items():
            if isinstance(budget, bool) or not isinstance(budget, int) or budget < 0:
                raise RPEGError(f"tau[{model.value}] must be a nonnegative integer, got {budget!r}")
        for e in self.data_edges:
            if e.kind != EdgeKind.DATA:
                raise RPEGError(f"Data edge {e.src.id}->{e.dst.id} must have kind DATA, got {e.kind.value}")
        published = set()
        for e in self.pub_edges:
            tag = f"Publication edge {e.src.id}->{e.dst.id}"
            if e.kind != EdgeKind.PUB:
                raise RPEGError(f"{tag} must have kind PUB, got {e.kind.value}")
            if e.src.kind.role != Role.TRAINING:
                raise RPEGError(f"{tag} must originate at a TRAIN vertex")
            if e.src.kind.model not in self.trainable:
                raise RPEGError(f"{tag} publishes frozen model {e.src.kind.model.value}")
            if e.dst.kind.model != e.src.kind.model:
                raise RPEGError(f"{tag} crosses model identity "
                                f"{e.src.kind.model.value}->{e.dst.kind.model.value}")
            if e.container not in e.src.kind.read or e.container not in e.src.kind.write:
                raise RPEGError(f"{tag} container {e.container.name} must be the source TRAIN "
                                "vertex's read/write weight container")
            published.add(e.src.kind.model)
        if set(self.trainable) - published:
            raise RPEGError("trainable models without publication edges: "
                            f"{_names(set(self.trainable) - published)}")
        for e in every:
            if e.container not in e.src.kind.write:
                raise RPEGError(f"Interface violation: {e.container.name} on edge "
                                f"{e.src.id}->{e.dst.id} not in Write({e.src.id})")
            if e.container not in e.dst.kind.read:
                raise RPEGError(f"Interface violation: {e.container.name} on edge "
                                f"{e.src.id}->{e.dst.id} not in Read({e.dst.id})")
        reads, writes = set(), set()
        for v in self.vertices:
            reads |= set(v.kind.read)
            writes |= set(v.kind.write)
        for what, implied, declared in (("A_in", reads - writes, set(self.in_containers)),
                                        ("A_out", writes - reads, set(self.out_containers))):
            if implied != declared:
                raise RPEGError(f"{what} mismatch: missing={[c.name for c in implied - declared]}, "
                                f"extra={[c.name for c in declared - implied]}")
        indeg = {v: 0 for v in self.vertices}
        for e in self.data_edges:
            indeg[e.dst] += 1
        work = [v for v in self.vertices if indeg[v] == 0]
        done = 0
        while work:
            v = work.pop()
            done += 1
            for e in self.data_edges:
                if e.src == v:
                    indeg[e.dst] -= 1
                    if indeg[e.dst] == 0:
                        work.append(e.dst)
        if done != len(self.vertices):
            raise RPEGError("Data-edge graph must be acyclic; cycle involves "
                            f"{sorted(v.id for v, k in indeg.items() if k > 0)}")
        if verbose:
            print("RPEG is well-formed.")
