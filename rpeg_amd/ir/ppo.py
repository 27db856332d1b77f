"""PPO step template: g_pi -> {i_ref, i_R, i_V} -> {t_pi, t_V}, publications t_pi->g_pi and
t_V->i_V (same graph as RPEG/ir/ppo.py:17-114)."""

from typing import Optional

from ..core.types import Model
from ._template import assemble, two_byte


def build_PPO_RPEG(suite, workload, tau: Optional[dict] = None, verbose: bool = False):
    B, K, S, T = workload.B, workload.K, workload.S, workload.T
    c = two_byte(prompts=B * S, completions=B * K * (S + T), log_pi=B * K * T, log_ref=B * K * T,
                 rewards=B * K, values=B * K * T,
                 W_pi=suite.n_params(Model.ACTOR), W_V=suite.n_params(Model.CRITIC),
                 W_ref=suite.n_params(Model.REFERENCE), W_R=suite.n_params(Model.REWARD))
    return assemble(
        c, listed=("completions", "log_pi", "log_ref", "rewards", "values", "W_pi", "W_V", "W_ref", "W_R"),
        inputs=("prompts", "W_ref", "W_R"),
        vertices=(("g_pi", Model.ACTOR, ("W_pi", "prompts"), ("completions", "log_pi")),
                  ("i_ref", Model.REFERENCE, ("W_ref", "completions"), ("log_ref",)),
                  ("i_R", Model.REWARD, ("W_R", "completions"), ("rewards",)),
                  ("i_V", Model.CRITIC, ("W_V", "completions"), ("values",)),
                  ("t_pi", Model.ACTOR, ("W_pi", "completions", "log_pi", "log_ref", "rewards", "values"), ("W_pi",)),
                  ("t_V", Model.CRITIC, ("W_V", "completions", "log_ref", "rewards", "values"), ("W_V",))),
        data=(("g_pi", "i_ref", "completions"), ("g_pi", "i_R", "completions"), ("g_pi", "i_V", "completions"),
              ("i_ref", "t_pi", "log_ref"), ("i_ref", "t_V", "log_ref"), ("i_R", "t_pi", "rewards"),
              ("i_V", "t_pi", "values"), ("i_R", "t_V", "rewards"), ("i_V", "t_V", "values")),
        pubs=(("t_pi", "g_pi", "W_pi"), ("t_V", "i_V", "W_V")),
        trainable={Model.ACTOR, Model.CRITIC}, tau=tau, verbose=verbose, title="PPO")
