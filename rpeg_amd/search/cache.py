"""Evaluation cache and canonical configuration hash (mirror of RPEG/search/cache.py:22-185)."""

import hashlib
import json
from dataclasses import dataclass, field
from typing import Dict, Optional, Tuple


@dataclass
class EvalCache:
    _store: Dict[str, Tuple[float, object, bool]] = field(default_factory=dict)
    hits: int = 0
    misses: int = 0   # unique evaluations stored

    def get(self, key: str) -> Optional[Tuple[float, object, bool]]:
        if key in self._store:
            self.hits += 1
            return self._store[key]
        return None

    def put(self, key: str, score: float, trace, feasible: bool) -> None:
        self._store[key] = (score, trace, feasible)
        self.misses += 1

    def __contains__(self, key: str) -> bool:
        return key in self._store

    def size(self) -> int:
        return len(self._store)

    def stats(self) -> str:
        total = self.hits + self.misses
        rate = self.hits / total if total > 0 else 0.0
        return f"hits={self.hits}  misses={self.misses}  total={total}  hit_rate={rate:.1%}"


def _container(c) -> dict:
    return {"name": c.name, "count": c.count, "elem": c.elem_size_bytes}


def _vertex(v) -> dict:
    by_name = lambda x: x["name"]  # noqa: E731
    return {"id": v.id, "role": v.kind.role.value, "model": v.kind.model.value,
            "read": sorted((_container(c) for c in v.kind.read), key=by_name),
            "write": sorted((_container(c) for c in v.kind.write), key=by_name)}


def _edge(e) -> dict:
    return {"src": e.src.id, "dst": e.dst.id, "container": _container(e.container)}


_graph_text = {}   # id(rpeg) -> (rpeg, the four fragments of the key text that depend on the template only)


def _graph_fragments(rpeg):
    hit = _graph_text.get(id(rpeg))
    if hit is not None and hit[0] is rpeg:
        return hit[1]
    ends = lambda x: (x["src"], x["dst"])  # noqa: E731
    dumps = lambda x: json.dumps(x, separators=(",", ":"), sort_keys=True)  # noqa: E731
    frag = (dumps(sorted((_edge(e) for e in rpeg.data_edges), key=ends)),
            dumps(sorted((_edge(e) for e in rpeg.pub_edges), key=ends)),
            dumps({m.value: t for m, t in rpeg.tau.items()}),
            dumps(sorted((_vertex(v) for v in rpeg.vertices), key=lambda x: x["id"])))
    if len(_graph_text) >= 64:
        _graph_text.clear()
    _graph_text[id(rpeg)] = (rpeg, frag)
    return frag


def config_hash(rpeg, plan) -> str:
    """sha256 of the canonical JSON of (template graph, plan); same payload and key order as the
    reference (RPEG/search/cache.py:160-185: keys sorted at every level, no blanks), so keys are
    interchangeable with caches it wrote.  The text is put together from its seven top-level entries in key
    order; the four that depend on the template alone are kept per template object, since a search hashes
    thousands of plans of a few templates."""
    data_edges, pub_edges, tau, vertices = _graph_fragments(rpeg)
    dumps = lambda x: json.dumps(x, separators=(",", ":"), sort_keys=True)  # noqa: E731
    sigma = dumps({v.id: {"origin": list(a.origin), "extent": list(a.extent)} for v, a in plan.sigma.items()})
    pi = dumps({v.id: list(p) for v, p in plan.pi.items()})
    mb = dumps({v.id: m for v, m in plan.mb.items()})
    text = ('{"data_edges":' + data_edges + ',"mb":' + mb + ',"pi":' + pi + ',"pub_edges":' + pub_edges +
            ',"sigma":' + sigma + ',"tau":' + tau + ',"vertices":' + vertices + "}")
    return hashlib.sha256(text.encode("utf-8")).hexdigest()


def _config_hash_plain(rpeg, plan) -> str:
    """The same key from one json.dumps of the whole payload, as the reference writes it; kept to check the
    assembled text against."""
    by_id = lambda kv: kv[0].id  # noqa: E731
    ends = lambda x: (x["src"], x["dst"])  # noqa: E731
    payload = {
        "vertices": sorted((_vertex(v) for v in rpeg.vertices), key=lambda x: x["id"]),
        "data_edges": sorted((_edge(e) for e in rpeg.data_edges), key=ends),
        "pub_edges": sorted((_edge(e) for e in rpeg.pub_edges), key=ends),
        "tau": {m.value: t for m, t in sorted(rpeg.tau.items(), key=lambda kv: kv[0].value)},
        "sigma": {v.id: {"origin": list(a.origin), "extent": list(a.extent)}
                  for v, a in sorted(plan.sigma.items(), key=by_id)},
        "pi": {v.id: list(p) for v, p in sorted(plan.pi.items(), key=by_id)},
        "mb": {v.id: m for v, m in sorted(plan.mb.items(), key=by_id)},
    }
    text = json.dumps(payload, separators=(",", ":"), sort_keys=True)
    return hashlib.sha256(text.encode("utf-8")).hexdigest()
