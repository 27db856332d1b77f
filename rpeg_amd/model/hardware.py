"""Cluster parameters of the analytical model (mirror of RPEG/model/hardware.py:17-122)."""

from dataclasses import dataclass
from typing import Tuple

from ..core.types import Allocation


def _span(allocs: Tuple[Allocation, ...]) -> Tuple[int, int]:
    racks = max(a.origin[0] + a.extent[0] for a in allocs) - min(a.origin[0] for a in allocs)
    nodes = max(a.origin[1] + a.extent[1] for a in allocs) - min(a.origin[1] for a in allocs)
    return racks, nodes


@dataclass(frozen=True)
class Hardware:
    flops_per_gpu: float
    memory_per_gpu: float
    memory_bandwidth: float
    alpha_coll_g: float
    beta_coll_g: float
    alpha_coll_n: float
    beta_coll_n: float
    alpha_coll_r: float
    beta_coll_r: float
    alpha_p2p_g: float
    beta_p2p_g: float
    alpha_p2p_n: float
    beta_p2p_n: float
    alpha_p2p_r: float
    beta_p2p_r: float
    gemm_m_half: float = 5.0
    gemm_k_half: float = 0.0
    decode_bw_eff: float = 0.15
    non_gemm_constant: float = 0.0
    non_gemm_scaling: float = 0.0
    non_gemm_batch_cal: float = 64
    op_generation_scale: float = 1.0
    op_inference_scale: float = 1.0
    op_training_scale: float = 1.0
    activation_comm_overhead_s: float = 0.0
    weight_comm_scale: float = 1.0
    reshard_scale: float = 1.0

    def tier_coll(self, allocs: Tuple[Allocation, ...]) -> Tuple[float, float]:
        """(alpha, beta) of collectives for the bounding span of `allocs`."""
        racks, nodes = _span(allocs)
        if racks > 1:
            return self.alpha_coll_r, self.beta_coll_r
        if nodes > 1:
            return self.alpha_coll_n, self.beta_coll_n
        return self.alpha_coll_g, self.beta_coll_g

    def tier_p2p(self, allocs: Tuple[Allocation, ...]) -> Tuple[float, float]:
        """(alpha, beta) of point-to-point transfers for the bounding span of `allocs`."""
        racks, nodes = _span(allocs)
        if racks > 1:
            return self.alpha_p2p_r, self.beta_p2p_r
        if nodes > 1:
            return self.alpha_p2p_n, self.beta_p2p_n
        return self.alpha_p2p_g, self.beta_p2p_g

    def tier(self, allocs: Tuple[Allocation, ...]) -> Tuple[float, float]:
        return self.tier_p2p(allocs)
