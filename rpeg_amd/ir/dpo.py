"""DPO step template (no generation): {i_pi, i_ref} -> t_pi, publication t_pi->i_pi.  Every
batch element is a preference pair, hence the factor 2 in the sequence containers (same
graph as RPEG/ir/dpo.py:63-166)."""

from typing import Optional

from ..core.types import Model
from ._template import assemble, two_byte


def build_DPO_RPEG(suite, workload, tau: Optional[dict] = None, verbose: bool = False):
    B, S, T = workload.B, workload.S, workload.T
    c = two_byte(X_pref=B * 2 * (S + T), log_pi=B * 2 * T, log_ref=B * 2 * T,
                 W_pi=suite.n_params(Model.ACTOR), W_ref=suite.n_params(Model.REFERENCE))
    return assemble(
        c, listed=("log_pi", "log_ref", "W_pi", "W_ref"), inputs=("X_pref", "W_ref"),
        vertices=(("i_pi", Model.ACTOR, ("W_pi", "X_pref"), ("log_pi",)),
                  ("i_ref", Model.REFERENCE, ("W_ref", "X_pref"), ("log_ref",)),
                  ("t_pi", Model.ACTOR, ("W_pi", "X_pref", "log_pi", "log_ref"), ("W_pi",))),
        data=(("i_pi", "t_pi", "log_pi"), ("i_ref", "t_pi", "log_ref")),
        pubs=(("t_pi", "i_pi", "W_pi"),),
        trainable={Model.ACTOR}, tau=tau, verbose=verbose, title="DPO")
