"""Structural settings the optimizer walks: template, staleness per trainable model, weight sharing,
fusion flag (mirror of RPEG/search/inter_model.py).  Pure host code; `optimize()` takes its families and
their order from the same rules (`rpeg_amd.search.optimizer.optimize_families`)."""

from __future__ import annotations

import dataclasses
import itertools
from dataclasses import dataclass
from typing import Dict, Iterator, Optional, Set, Tuple

from ..core.types import Model
from ..ir.ac_share import build_AC_share_RPEG, is_AC_share_applicable
from ..ir.dpo import build_DPO_RPEG
from ..ir.grpo import build_GRPO_RPEG
from ..ir.ppo import build_PPO_RPEG
from ..ir.rpeg import RPEG
from ..model.models import ModelSuite
from ..model.workload import Workload

DEFAULT_T_CAND: Dict[Model, Set[int]] = {Model.ACTOR: {0, 1}, Model.CRITIC: {0, 1}, Model.AC_SHARE: {0, 1}}


@dataclass
class InterModelConfig:
    """Which structural setting produced a template (RPEG/search/inter_model.py:32-40)."""
    ac_share: bool
    tau: Dict[Model, int]
    algorithm: str = "ppo"
    intra_stage_fusion: bool = False


def _iter_staleness(trainable, T_cand: Dict[Model, Set[int]]) -> Iterator[Dict[Model, int]]:
    """Every staleness assignment: models ordered by their value string, candidates ascending, last model
    fastest (RPEG/search/inter_model.py:43-65)."""
    models = sorted(trainable, key=lambda m: m.value)
    for combo in itertools.product(*[sorted(T_cand[m]) for m in models]):
        yield dict(zip(models, combo))


def Iter_inter_model_candidates(suite: ModelSuite, workload: Workload, T_cand: Optional[Dict[Model, Set[int]]] = None,
                                algorithm: str = "ppo") -> Iterator[Tuple[RPEG, InterModelConfig]]:
    """(template, setting) pairs in the order optimize() walks them (RPEG/search/inter_model.py:68-121): DPO and
    GRPO their staleness variants; PPO per staleness variant the plain and the fused setting, then, as the
    template trains an actor and a critic, the AC-share template with its own variants."""
    if T_cand is None:
        T_cand = {m: set(s) for m, s in DEFAULT_T_CAND.items()}
    if algorithm in ("dpo", "grpo"):
        rpeg = (build_DPO_RPEG if algorithm == "dpo" else build_GRPO_RPEG)(suite, workload)
        for tau in _iter_staleness(rpeg.trainable, T_cand):
            yield dataclasses.replace(rpeg, tau=tau), InterModelConfig(ac_share=False, tau=tau, algorithm=algorithm)
        return
    ppo = build_PPO_RPEG(suite, workload)
    for tau in _iter_staleness(ppo.trainable, T_cand):
        for fused in (False, True):
            yield dataclasses.replace(ppo, tau=tau), InterModelConfig(ac_share=False, tau=tau, intra_stage_fusion=fused)
    if is_AC_share_applicable(ppo):
        ac = build_AC_share_RPEG(suite, workload)
        for tau in _iter_staleness(ac.trainable, T_cand):
            yield dataclasses.replace(ac, tau=tau), InterModelConfig(ac_share=True, tau=tau)
