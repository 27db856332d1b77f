"""Actor-critic weight-sharing rewrite of the PPO template: one AC_SHARE model generates,
scores values and trains (same graph as RPEG/ir/ac_share.py:17-118)."""

from typing import Optional

from ..core.types import Model
from ._template import assemble, two_byte


def is_AC_share_applicable(rpeg) -> bool:
    """True iff the template trains both an actor and a critic."""
    return Model.ACTOR in rpeg.trainable and Model.CRITIC in rpeg.trainable


def build_AC_share_RPEG(suite, workload, tau: Optional[dict] = None, verbose: bool = False):
    B, K, S, T = workload.B, workload.K, workload.S, workload.T
    c = two_byte(prompts=B * S, completions=B * K * (S + T), log_ac=B * K * T, log_ref=B * K * T,
                 rewards=B * K, values=B * K * T, W_AC=suite.n_params(Model.AC_SHARE),
                 W_ref=suite.n_params(Model.REFERENCE), W_R=suite.n_params(Model.REWARD))
    return assemble(
        c, listed=("completions", "log_ac", "log_ref", "rewards", "values", "W_AC", "W_ref", "W_R"),
        inputs=("prompts", "W_ref", "W_R"),
        vertices=(("g_ac", Model.AC_SHARE, ("W_AC", "prompts"), ("completions", "log_ac")),
                  ("i_ref", Model.REFERENCE, ("W_ref", "completions"), ("log_ref",)),
                  ("i_R", Model.REWARD, ("W_R", "completions"), ("rewards",)),
                  ("i_ac", Model.AC_SHARE, ("W_AC", "completions"), ("values",)),
                  ("t_ac", Model.AC_SHARE, ("W_AC", "completions", "log_ac", "log_ref", "rewards", "values"), ("W_AC",))),
        data=(("g_ac", "i_ref", "completions"), ("g_ac", "i_R", "completions"), ("g_ac", "i_ac", "completions"),
              ("i_ref", "t_ac", "log_ref"), ("i_R", "t_ac", "rewards"), ("i_ac", "t_ac", "values")),
        pubs=(("t_ac", "g_ac", "W_AC"), ("t_ac", "i_ac", "W_AC")),
        trainable={Model.AC_SHARE}, tau=tau, verbose=verbose, title="AC-Share PPO")
