"""Writes tests/golden/ref_inter_model.json: what the REFERENCE's Iter_inter_model_candidates
(RPEG/search/inter_model.py:68-121) yields, in order, for the three algorithms and a few T_cand.

Run in the development container only (it needs the read-only reference tree):

    python tests/golden/make_golden_inter_model.py [--ref /root/reference]

inter_model.py and the template builders it calls are imported unmodified (the import set-up is the one
of make_golden_sa.py).
"""

from __future__ import annotations

import argparse
import json
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

import make_golden_sa as SA   # noqa: E402

T_CANDS = {"default": None, "wide": {"Pi": [2, 0, 1], "V": [1, 0], "AC": [3, 0]}, "no_ac": {"Pi": [0], "V": [1], "AC": []}}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    args = ap.parse_args()
    mods, moves, Configuration, ct = SA.load_moves(args.ref)
    import search.inter_model as rim
    from rpeg_amd import configs
    problem = configs.config(1).problem
    _, suite, wl, _, _, _, _ = SA.ref_world(mods, problem, {"Pi": 0, "V": 0})
    doc = {}
    for name, cand in T_CANDS.items():
        t_cand = None if cand is None else {ct.Model(m): set(v) for m, v in cand.items()}
        for algorithm in ("ppo", "grpo", "dpo"):
            out = []
            for rpeg, cfg in rim.Iter_inter_model_candidates(suite, wl, t_cand, algorithm=algorithm):
                assert rpeg.tau == cfg.tau
                out.append(dict(vertices=[v.id for v in rpeg.vertices], tau=[[m.value, t] for m, t in cfg.tau.items()],
                                ac_share=cfg.ac_share, fused=cfg.intra_stage_fusion, algorithm=cfg.algorithm))
            doc[f"{name}/{algorithm}"] = out
            print(name, algorithm, len(out))
    doc["t_cands"] = T_CANDS
    path = os.path.join(HERE, "ref_inter_model.json")
    with open(path, "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
