"""Execution plan P = (sigma, pi, mb), keyed by template vertex (mirror of RPEG/ir/plan.py:15-25)."""

from dataclasses import dataclass
from typing import Dict, Tuple

from ..core.types import Allocation, TemplateVertex


@dataclass(frozen=True)
class ExecutionPlan:
    sigma: Dict[TemplateVertex, Allocation]          # vertex -> device box
    pi: Dict[TemplateVertex, Tuple[int, int, int]]   # vertex -> (dp, pp, tp)
    mb: Dict[TemplateVertex, int]                    # vertex -> microbatch count
