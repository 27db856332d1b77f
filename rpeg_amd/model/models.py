"""Model hyper-parameters (mirror of RPEG/model/models.py:17-82)."""

from dataclasses import dataclass
from typing import Dict, Optional

from ..core.types import Model


@dataclass(frozen=True)
class ModelSpec:
    L: int
    d: int
    d_ff: int
    V: int
    dtype_bytes: int = 2
    d_head: int = 128
    parameter_count: Optional[int] = None


def base_transformer_params(spec: ModelSpec) -> int:
    if spec.parameter_count is not None:
        return int(spec.parameter_count)
    return spec.L * (4 * spec.d * spec.d + 2 * spec.d * spec.d_ff) + spec.V * spec.d


def transformer_parameter_count(spec: ModelSpec, m: Model) -> int:
    """Base parameters plus one scalar head row for critic / reward / shared actor-critic."""
    head = spec.d if m in (Model.CRITIC, Model.REWARD, Model.AC_SHARE) else 0
    return base_transformer_params(spec) + head


@dataclass(frozen=True)
class ModelSuite:
    specs: Dict[Model, ModelSpec]

    def n_params(self, m: Model) -> int:
        return transformer_parameter_count(self.specs[m], m)
