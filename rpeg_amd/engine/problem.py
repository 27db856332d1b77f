"""Host description of one batched-evaluation problem and of a batch of candidate plans.

An `EvalProblem` fixes everything that does not vary between candidates: the step
templates ("structures", e.g. PPO and its actor-critic-sharing rewrite), models, workload,
cluster parameters, device mesh, unroll depth and memory policy.  A `PlanBatch` holds the
per-candidate variables as structure-of-arrays tensors in the layout the C ABI takes:

  vert[(slot*10 + f), i]  int16   f = dp, pp, tp, mb, origin r/n/g, extent r/n/g of vertex `slot`
  head[0..3, i]           uint8   structure id, generation-split index, tau of trainable slot 0 / 1

The generation-split index j selects the suffix quantiles[j-1:] of the workload's generation
quantiles (0 = no quantile splitting); it enters the reference through `Workload`, which is a
per-call argument of `evaluate` (RPEG/search/evaluate.py:235-241).
"""

from __future__ import annotations

from dataclasses import dataclass, field, replace
from typing import Callable, FrozenSet, Optional, Sequence, Tuple

import numpy as np

from ..core.types import (Allocation, DeviceSpace, Model, RPEG_TRANSFER_RESOURCE_POLICY,
                          TransferResourcePolicy)
from ..ir.plan import ExecutionPlan
from ..ir.rpeg import RPEG
from ..ir.ppo import build_PPO_RPEG
from ..ir.grpo import build_GRPO_RPEG
from ..ir.dpo import build_DPO_RPEG
from ..ir.ac_share import build_AC_share_RPEG
from ..model.hardware import Hardware
from ..model.memory import MemoryPolicy
from ..model.models import ModelSuite
from ..model.workload import Workload

MAX_VERTICES = 6
FIELDS_PER_VERTEX = 10
F_DP, F_PP, F_TP, F_MB, F_OR, F_ON, F_OG, F_ER, F_EN, F_EG = range(10)


@dataclass(frozen=True)
class Structure:
    """One step template plus the order of its trainable models in the plan header."""
    name: str
    build: Callable[..., RPEG]
    tau_models: Tuple[Model, ...]
    # The models the MEMORY model treats as trainable when that is not the template's own set.  The
    # reference's evaluate_cached builds its memory model from the template (evaluate.py:378-385), but
    # optimize() checks restarts (is_valid) with the memory model of its base configuration
    # (optimizer.py:449-458): under that model the AC-share template's shared model counts as frozen.
    memory_trainable: Optional[FrozenSet[Model]] = None


PPO = Structure("ppo", build_PPO_RPEG, (Model.ACTOR, Model.CRITIC))
GRPO = Structure("grpo", build_GRPO_RPEG, (Model.ACTOR,))
DPO = Structure("dpo", build_DPO_RPEG, (Model.ACTOR,))
AC_SHARE = Structure("ac_share", build_AC_share_RPEG, (Model.AC_SHARE,))
STRUCTURES = {s.name: s for s in (PPO, GRPO, DPO, AC_SHARE)}


def as_seen_from(structure: Structure, base: Structure) -> Structure:
    """`structure` under the memory model of a configuration of `base` (what is_valid sees inside
    optimize(), RPEG/search/optimizer.py:449-458, 596-663)."""
    return replace(structure, memory_trainable=frozenset(base.tau_models))


@dataclass(frozen=True)
class EvalProblem:
    structures: Tuple[Structure, ...]
    suite: ModelSuite
    workload: Workload
    hw: Hardware
    device_space: DeviceSpace
    K_eval: int
    memory_policy: MemoryPolicy = field(default_factory=MemoryPolicy)
    transfer_resource_policy: TransferResourcePolicy = RPEG_TRANSFER_RESOURCE_POLICY

    def n_splits(self) -> int:
        """Number of generation-split variants: 0 (unsplit) .. Q."""
        q = self.workload.gen_quantiles
        return 1 + (len(q) if q else 0)

    def workload_for(self, split: int) -> Workload:
        q = self.workload.gen_quantiles
        if split == 0 or not q:
            return replace(self.workload, gen_quantiles=None)
        return replace(self.workload, gen_quantiles=tuple(q[split - 1:]))

    def template(self, structure: int, taus: Sequence[int] = ()) -> RPEG:
        st = self.structures[structure]
        tau = {m: int(taus[i]) if i < len(taus) else 0 for i, m in enumerate(st.tau_models)}
        return st.build(self.suite, self.workload, tau=tau)


@dataclass
class PlanBatch:
    vert: np.ndarray   # int16 [MAX_VERTICES*10, n]
    head: np.ndarray   # uint8 [4, n]

    @property
    def n(self) -> int:
        return int(self.vert.shape[1])

    @classmethod
    def empty(cls, n: int) -> "PlanBatch":
        return cls(np.zeros((MAX_VERTICES * FIELDS_PER_VERTEX, n), np.int16), np.zeros((4, n), np.uint8))

    def slice(self, lo: int, hi: int) -> "PlanBatch":
        return PlanBatch(np.ascontiguousarray(self.vert[:, lo:hi]), np.ascontiguousarray(self.head[:, lo:hi]))

    def take(self, idx) -> "PlanBatch":
        idx = np.asarray(idx)
        return PlanBatch(np.ascontiguousarray(self.vert[:, idx]), np.ascontiguousarray(self.head[:, idx]))

    def set_plan(self, i: int, structure: int, split: int, taus: Sequence[int],
                 rpeg: RPEG, plan: ExecutionPlan) -> None:
        self.head[0, i], self.head[1, i] = structure, split
        for t, tau in enumerate(taus):
            self.head[2 + t, i] = tau
        for s, v in enumerate(rpeg.vertices):
            a = plan.sigma[v]
            row = list(plan.pi[v]) + [plan.mb[v]] + list(a.origin) + list(a.extent)
            self.vert[s * FIELDS_PER_VERTEX:(s + 1) * FIELDS_PER_VERTEX, i] = row

    def configuration(self, problem: EvalProblem, i: int):
        """(rpeg, ExecutionPlan, Workload) of candidate i in the reference's representation."""
        s, split = int(self.head[0, i]), int(self.head[1, i])
        st = problem.structures[s]
        taus = [int(self.head[2 + t, i]) for t in range(len(st.tau_models))]
        rpeg = problem.template(s, taus)
        sigma, pi, mb = {}, {}, {}
        for slot, v in enumerate(rpeg.vertices):
            f = [int(x) for x in self.vert[slot * FIELDS_PER_VERTEX:(slot + 1) * FIELDS_PER_VERTEX, i]]
            pi[v] = (f[F_DP], f[F_PP], f[F_TP])
            mb[v] = f[F_MB]
            sigma[v] = Allocation(origin=(f[F_OR], f[F_ON], f[F_OG]), extent=(f[F_ER], f[F_EN], f[F_EG]))
        return rpeg, ExecutionPlan(sigma=sigma, pi=pi, mb=mb), problem.workload_for(split)
