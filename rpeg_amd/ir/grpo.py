"""GRPO step template (no critic): g_pi -> {i_ref, i_R} -> t_pi, publication t_pi->g_pi
(same graph as RPEG/ir/grpo.py:17-108)."""

from typing import Optional

from ..core.types import Model
from ._template import assemble, two_byte


def build_GRPO_RPEG(suite, workload, tau: Optional[dict] = None, verbose: bool = False):
    B, K, S, T = workload.B, workload.K, workload.S, workload.T
    c = two_byte(prompts=B * S, completions=B * K * (S + T), log_pi=B * K * T, log_ref=B * K * T,
                 rewards=B * K, W_pi=suite.n_params(Model.ACTOR),
                 W_ref=suite.n_params(Model.REFERENCE), W_R=suite.n_params(Model.REWARD))
    return assemble(
        c, listed=("completions", "log_pi", "log_ref", "rewards", "W_pi", "W_ref", "W_R"),
        inputs=("prompts", "W_ref", "W_R"),
        vertices=(("g_pi", Model.ACTOR, ("W_pi", "prompts"), ("completions", "log_pi")),
                  ("i_ref", Model.REFERENCE, ("W_ref", "completions"), ("log_ref",)),
                  ("i_R", Model.REWARD, ("W_R", "completions"), ("rewards",)),
                  ("t_pi", Model.ACTOR, ("W_pi", "completions", "log_pi", "log_ref", "rewards"), ("W_pi",))),
        data=(("g_pi", "i_ref", "completions"), ("g_pi", "i_R", "completions"),
              ("i_ref", "t_pi", "log_ref"), ("i_R", "t_pi", "rewards")),
        pubs=(("t_pi", "g_pi", "W_pi"),),
        trainable={Model.ACTOR}, tau=tau, verbose=verbose, title="GRPO")
