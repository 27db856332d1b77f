"""Host-side mirror of the reference's geometry helpers and IR atoms.

Same names, fields and argument meaning as RPEG/core/types.py so that plan
objects built for the reference can be passed to this package unchanged.
"""

from __future__ import annotations

import enum
from dataclasses import dataclass
from typing import Optional, Tuple


def packing_geometry(dp: int, pp: int, tp: int, G: int) -> Optional[Tuple[int, int]]:
    """(g_ext, nodes_needed) of a (dp, pp, tp) strategy on nodes of G devices, or
    None when replicas would straddle a node boundary (RPEG/core/types.py:16-57)."""
    stages_per_node = min(pp, G // tp)
    if stages_per_node == 0 or pp % stages_per_node:
        return None
    nodes_per_replica = pp // stages_per_node
    if nodes_per_replica > 1:
        return G, dp * nodes_per_replica
    replica_gpus = stages_per_node * tp
    replicas_per_node = G // replica_gpus
    if dp <= replicas_per_node:
        return dp * replica_gpus, 1
    if dp % replicas_per_node:
        return None
    return G, dp // replicas_per_node


def rectangular_node_layouts(nodes_needed: int, R: int, N: int) -> Tuple[Tuple[int, int], ...]:
    """Exact (racks, nodes-per-rack) rectangles of `nodes_needed` nodes
    (RPEG/core/types.py:60-85)."""
    if min(nodes_needed, R, N) <= 0:
        return ()
    return tuple((r, nodes_needed // r) for r in range(1, min(R, nodes_needed) + 1)
                 if nodes_needed % r == 0 and nodes_needed // r <= N)


class Role(enum.Enum):
    GENERATION = "GEN"
    INFERENCE = "INF"
    TRAINING = "TRAIN"


class Model(enum.Enum):
    ACTOR = "Pi"
    CRITIC = "V"
    REFERENCE = "Ref"
    REWARD = "R"
    AC_SHARE = "AC"


class Collective(enum.Enum):
    ALLREDUCE = "AllReduce"
    ALLGATHER = "AllGather"
    REDUCESCATTER = "ReduceScatter"
    ALLTOALL = "AllToAll"
    P2P = "PointToPoint"


class EdgeKind(enum.Enum):
    DATA = "data"
    PUB = "pub"


_POLICY_VALUES = ("destination_only", "both_endpoints")


@dataclass(frozen=True)
class TransferResourcePolicy:
    """Which endpoints a transfer node keeps busy (RPEG/core/types.py:128-195)."""
    weight: str = "destination_only"
    activation: str = "destination_only"

    def __post_init__(self) -> None:
        if self.weight not in _POLICY_VALUES:
            raise ValueError(f"unsupported weight transfer resource policy {self.weight!r}")
        if self.activation not in _POLICY_VALUES:
            raise ValueError(f"unsupported activation transfer resource policy {self.activation!r}")

    def for_weight(self, is_weight: bool) -> str:
        return self.weight if is_weight else self.activation

    def to_dict(self) -> dict:
        return {"weight": self.weight, "activation": self.activation}

    @classmethod
    def from_dict(cls, value: object) -> "TransferResourcePolicy":
        if not isinstance(value, dict):
            raise ValueError("transfer_resource_policy must be a mapping")
        return cls(weight=str(value.get("weight", _POLICY_VALUES[0])),
                   activation=str(value.get("activation", _POLICY_VALUES[0])))


RPEG_TRANSFER_RESOURCE_POLICY = TransferResourcePolicy()
CONSERVATIVE_TRANSFER_RESOURCE_POLICY = TransferResourcePolicy("both_endpoints", "both_endpoints")


@dataclass(frozen=True)
class DeviceSpace:
    R: int
    N: int
    G: int

    def num_devices(self) -> int:
        return self.R * self.N * self.G

    def device_id(self, r: int, n: int, g: int) -> int:
        return (r * self.N + n) * self.G + g


@dataclass(frozen=True)
class Allocation:
    origin: Tuple[int, int, int]
    extent: Tuple[int, int, int]

    def size(self) -> int:
        return self.extent[0] * self.extent[1] * self.extent[2]


@dataclass(frozen=True)
class Container:
    name: str
    count: int
    elem_size_bytes: int

    def bytes(self) -> int:
        return self.count * self.elem_size_bytes


@dataclass(frozen=True)
class OperatorKind:
    role: Role
    model: Model
    read: Tuple[Container, ...]
    write: Tuple[Container, ...]


@dataclass(frozen=True)
class TemplateVertex:
    id: str
    kind: OperatorKind


@dataclass(frozen=True)
class TemplateEdge:
    src: TemplateVertex
    dst: TemplateVertex
    container: Container
    kind: EdgeKind
