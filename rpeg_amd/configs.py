"""The five benchmark workloads, as `EvalProblem` builders plus candidate-set sizes.

Cluster parameters are the calibrated values printed in the reference's README
(README.md:131-161), with flops_per_gpu = 4.4e14.  Values the workload descriptions leave
open are fixed here once: DPO uses K=1, S=T=2048; config 5 uses K_eval=5; staleness sets
default to actor {0,1}, critic {0}.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Tuple

from .core.types import DeviceSpace, Model
from .engine.problem import AC_SHARE, DPO, GRPO, PPO, EvalProblem
from .model.hardware import Hardware
from .model.memory import MemoryPolicy
from .model.models import ModelSpec, ModelSuite
from .model.workload import Workload

SPEC_7B = ModelSpec(L=32, d=4096, d_ff=11008, V=32000)
SPEC_13B = ModelSpec(L=40, d=5120, d_ff=13824, V=32000)
SPEC_70B = ModelSpec(L=80, d=8192, d_ff=28672, V=128256)

# memory_per_gpu that makes about 70 % of config 4's seeded candidates infeasible
CFG4_MEMORY_PER_GPU = 1.03e11
# Config 5 does not state its hardware block.  With the README's 1.03e11 B per device no plan of its
# models fits at T = 16384 (the actor's generation stage alone needs 3.8e11 B whatever the strategy), the
# candidate directory (RPEG/search/moves.py:532-541) is empty for four of the six vertices and the
# reference's move_gen raises on the empty range.  8.0e11 is the smallest round figure at which every
# vertex keeps at least 40 memory-feasible strategies.
CFG5_MEMORY_PER_GPU = 8.0e11


def readme_hardware(memory_per_gpu: float = 1.03e11) -> Hardware:
    return Hardware(
        flops_per_gpu=4.4e14, memory_per_gpu=memory_per_gpu, memory_bandwidth=1.0e12,
        alpha_coll_g=7.8e-5, beta_coll_g=4.545e-9, alpha_coll_n=2.2e-4, beta_coll_n=8.0e-8,
        alpha_coll_r=4.4e-4, beta_coll_r=1.6e-7,
        alpha_p2p_g=3.5e-5, beta_p2p_g=4.545e-9, alpha_p2p_n=1.8e-4, beta_p2p_n=8.0e-8,
        alpha_p2p_r=3.6e-4, beta_p2p_r=1.6e-7,
        gemm_m_half=240.0, gemm_k_half=0.0, decode_bw_eff=0.63,
        non_gemm_constant=1.2e-4, non_gemm_scaling=3.5e-4, non_gemm_batch_cal=64)


@dataclass(frozen=True)
class BenchConfig:
    name: str
    problem: EvalProblem
    n_plans: int
    tau_sets: Tuple[Tuple[int, ...], ...]   # per structure: allowed tau per trainable slot, flattened below
    tau_choices: Dict[str, Tuple[Tuple[int, ...], ...]]


def _cfg(name, structures, suite, workload, space, k_eval, n_plans, tau_choices, hw=None):
    problem = EvalProblem(structures=structures, suite=suite, workload=workload,
                          hw=hw or readme_hardware(), device_space=space, K_eval=k_eval,
                          memory_policy=MemoryPolicy())
    return BenchConfig(name=name, problem=problem, n_plans=n_plans, tau_sets=(), tau_choices=tau_choices)


def config(i: int) -> BenchConfig:
    """Benchmark configuration i in 1..5."""
    if i == 1:
        suite = ModelSuite({Model.ACTOR: SPEC_7B, Model.REFERENCE: SPEC_7B, Model.REWARD: SPEC_7B,
                            Model.CRITIC: SPEC_7B, Model.AC_SHARE: SPEC_7B})
        wl = Workload(B=64, K=1, S=128, T=512, gen_quantiles=((0.5, 128), (0.85, 256), (1.0, 512)))
        return _cfg("cfg1_ppo_1x8x4", (PPO,), suite, wl, DeviceSpace(1, 8, 4), 5, 4096,
                    {"ppo": ((0, 1), (0,))})
    if i == 2:
        suite = ModelSuite({Model.ACTOR: SPEC_7B, Model.REFERENCE: SPEC_7B, Model.REWARD: SPEC_7B})
        wl = Workload(B=128, K=8, S=512, T=4096, gen_quantiles=((0.5, 1024), (0.9, 2048), (1.0, 4096)))
        return _cfg("cfg2_grpo_4x8x4", (GRPO,), suite, wl, DeviceSpace(4, 8, 4), 5, 65536,
                    {"grpo": ((0, 1, 2),)})
    if i == 3:
        suite = ModelSuite({Model.ACTOR: SPEC_13B, Model.REFERENCE: SPEC_13B, Model.REWARD: SPEC_7B,
                            Model.CRITIC: SPEC_13B, Model.AC_SHARE: SPEC_13B})
        wl = Workload(B=256, K=1, S=1024, T=8192,
                      gen_quantiles=((0.3, 1024), (0.7, 4096), (0.95, 6144), (1.0, 8192)))
        return _cfg("cfg3_ppo_acshare_8x8x4", (PPO, AC_SHARE), suite, wl, DeviceSpace(8, 8, 4), 8, 262144,
                    {"ppo": ((0, 1), (0, 1)), "ac_share": ((0, 1),)})
    if i == 4:
        suite = ModelSuite({Model.ACTOR: SPEC_70B, Model.REFERENCE: SPEC_70B})
        wl = Workload(B=512, K=1, S=2048, T=2048, gen_quantiles=None)
        return _cfg("cfg4_dpo_16x16x4", (DPO,), suite, wl, DeviceSpace(16, 16, 4), 5, 1048576,
                    {"dpo": ((0, 1),)}, hw=readme_hardware(CFG4_MEMORY_PER_GPU))
    if i == 5:
        suite = ModelSuite({Model.ACTOR: SPEC_70B, Model.REFERENCE: SPEC_70B, Model.REWARD: SPEC_7B,
                            Model.CRITIC: SPEC_7B, Model.AC_SHARE: SPEC_70B})
        wl = Workload(B=512, K=4, S=1024, T=16384, gen_quantiles=((0.5, 2048), (0.9, 8192), (1.0, 16384)))
        return _cfg("cfg5_ppo_sa_4x32x4", (PPO,), suite, wl, DeviceSpace(4, 32, 4), 5, 64 * 2000 * 6,
                    {"ppo": ((0, 1), (0,))}, hw=readme_hardware(CFG5_MEMORY_PER_GPU))
    raise ValueError(f"no benchmark configuration {i}")
