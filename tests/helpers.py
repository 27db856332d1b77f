"""Shared helpers for the test-suite: golden fixtures, oracle evaluation of seeded candidates."""

import json
import os
import zlib

from oracle import rpeg_oracle as oracle
from rpeg_amd import configs
from rpeg_amd.search import candidates

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_golden(c):
    with open(os.path.join(GOLDEN, f"ref_cfg{c}.json")) as f:
        return json.load(f)


def seeded_batch(c, n=None, start=0):
    cfg = configs.config(c)
    return cfg, candidates.generate(cfg.problem, n or cfg.n_plans, cfg.tau_choices, seed=42, tag=c, start=start)


def oracle_eval(problem, batch, i, **kw):
    rpeg, plan, wl = batch.configuration(problem, i)
    return oracle.evaluate_plan(rpeg, plan, problem.device_space, problem.suite, wl, problem.hw,
                                problem.K_eval, problem.memory_policy, check_stale=False, **kw)


def order_crc(order):
    return zlib.crc32(",".join(order).encode())
