"""Workload description (mirror of RPEG/model/workload.py:13-28)."""

from dataclasses import dataclass
from typing import Optional, Tuple


@dataclass(frozen=True)
class Workload:
    B: int  # prompts per step
    K: int  # rollouts per prompt
    S: int  # prompt length
    T: int  # generation length
    gen_quantiles: Optional[Tuple[Tuple[float, int], ...]] = None  # ((cumulative fraction, tokens), ...)
