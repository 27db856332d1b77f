"""Writes tests/golden/ref_full_cfg{1..4}.json: digests of the REFERENCE's evaluation of the WHOLE seeded
candidate sets (4,096 / 65,536 / 262,144 / 1,048,576 plans of configurations 1-4).

Run in the development container only (it needs the read-only reference tree; hours of CPU time for
configurations 3 and 4):

    python tests/golden/make_golden_full.py [--ref /root/reference] [--configs 1,2,3,4] [--workers 6]
    python tests/golden/make_golden_full.py --configs 5 --limit 16384      (ref_full_cfg5_first16384.json: the first
                                                  16,384 seeded plans of the annealing configuration, which has no fixed set)

Every plan of a set goes through the reference's own passes exactly as `make_golden.py` sends the first few
hundred (`unroll`, `lower`, `NodeCostModel`, `schedule`, `Trace.throughput`, `mem_worst_violation`,
`_device_peaks`; the score and penalty lines of the unparsable `search/evaluate.py` — :288, :372-374, :396-401
— are applied here), plus the reference's `stale_publication_layout_valid` from the part of that file that
does parse.  Stored per configuration:

  * per chunk of 4,096 consecutive plans the CRC-32 of the little-endian float64 arrays `makespan`, `peak`
    (largest device peak), `score` (as `_eval_worker` scores: no stale-layout gate) and `score_gated` (as
    `evaluate_cached` scores: 0 where that gate fails), of the byte array `flags` (bit 0 memory-feasible,
    bit 1 stale-layout ok) and of the int16 array `device` (the (r, n, g) that `mem_worst_violation` names,
    -1 -1 -1 where it returns None), so that a mismatch names its chunk;
  * the best plan (first maximum) and the 32 best plans in ranking order (score descending, index ascending)
    under both scores, the number of feasible plans and of plans that pass the stale-layout gate.

Only data is written; tests regenerate the inputs from the seed.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time
import zlib

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, HERE)

CHUNK = 4096
PIECE = 512          # plans per pool task
TOP = 32

_state = {}


def _setup(ref_root):
    import make_golden as mg
    import make_golden_validity as mv
    mods = mg.load_reference(ref_root)
    ev = mv.load_reference_evaluate(ref_root, mods)
    _state.update(mg=mg, mods=mods, ev=ev)


def _eval_piece(task):
    """Reference evaluation of plans [start, start + n) of configuration c."""
    c, start, n = task
    from rpeg_amd import configs
    from rpeg_amd.search import candidates
    mg, mods, ev = _state["mg"], _state["mods"], _state["ev"]
    cfg = configs.config(c)
    p = cfg.problem
    pol = p.memory_policy
    mem_mod = mods["model.memory"]
    batch = candidates.generate(p, n, cfg.tau_choices, seed=42, tag=c, start=start)
    makespan = np.empty(n)
    peak = np.empty(n)
    score = np.empty(n)
    gated = np.empty(n)
    flags = np.zeros(n, np.uint8)
    device = np.full((n, 3), -1, np.int16)
    for i in range(n):
        rpeg, plan, wl, suite, hw, space = mg.to_reference(mods, p, batch, i)
        unrolled = mods["passes.unroll"].unroll(rpeg, p.K_eval)
        lowered = mods["passes.lower"].lower(rpeg, unrolled, plan, suite, p.K_eval, workload=wl)
        cost = mods["model.cost"].NodeCostModel(hw, suite, wl, optimizer_stage=pol.optimizer_stage,
                                                activation_checkpointing=pol.activation_checkpointing)
        trace = mods["schedule.scheduler"].schedule(lowered, cost, space)
        raw = trace.throughput(W_step=wl.B * wl.K * (wl.S + wl.T), K=p.K_eval)
        mm = mem_mod.NodeMemoryModel.from_policy(
            hw, suite, wl, mem_mod.MemoryPolicy(**{k: getattr(pol, k) for k in pol.__dataclass_fields__}),
            trainable=frozenset(rpeg.trainable),
            shadow_models=frozenset(m for m in rpeg.trainable if rpeg.tau.get(m, 0) > 0))
        violation = mem_mod.mem_worst_violation(lowered, mm)
        if violation is None:
            s, feasible = raw, True
            pk = max(mem_mod._device_peaks(lowered, mm).values())
        else:
            dev, req, cap = violation
            s = raw * max(math.exp(-40.0 * max(0.0, req / cap - 1.0)), 1e-12)
            feasible, pk = False, req
            device[i] = dev
        stale_ok = bool(ev.stale_publication_layout_valid(ev.Configuration(rpeg, plan, space)))
        makespan[i] = trace.makespan()
        peak[i] = pk
        score[i] = s
        gated[i] = s if stale_ok else 0.0
        flags[i] = (1 if feasible else 0) | (2 if stale_ok else 0)
    return start, makespan, peak, score, gated, flags, device


def digest(makespan, peak, score, gated, flags, device):
    """The stored record of a whole set (also what the tests compute from the engine's outputs)."""
    n = len(score)
    chunks = []
    for a in range(0, n, CHUNK):
        b = min(n, a + CHUNK)
        chunks.append([zlib.crc32(np.ascontiguousarray(makespan[a:b], "<f8").tobytes()),
                       zlib.crc32(np.ascontiguousarray(peak[a:b], "<f8").tobytes()),
                       zlib.crc32(np.ascontiguousarray(score[a:b], "<f8").tobytes()),
                       zlib.crc32(np.ascontiguousarray(gated[a:b], "<f8").tobytes()),
                       zlib.crc32(np.ascontiguousarray(flags[a:b], np.uint8).tobytes()),
                       zlib.crc32(np.ascontiguousarray(device[a:b], "<i2").tobytes())])
    return dict(n=n, chunk=CHUNK, chunks=chunks,
                argmax=int(np.argmax(score)), argmax_gated=int(np.argmax(gated)),
                top=[int(i) for i in np.argsort(-score, kind="stable")[:TOP]],
                top_gated=[int(i) for i in np.argsort(-gated, kind="stable")[:TOP]],
                best=float(np.max(score)).hex(), best_gated=float(np.max(gated)).hex(),
                n_feasible=int(np.sum(flags & 1)), n_stale_ok=int(np.sum((flags >> 1) & 1)))


def main():
    import multiprocessing as mp
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    ap.add_argument("--configs", default="1,2,3,4")
    ap.add_argument("--workers", type=int, default=6)
    ap.add_argument("--limit", type=int, default=0, help="evaluate only the first LIMIT plans (a trial run)")
    args = ap.parse_args()
    _setup(args.ref)
    from rpeg_amd import configs
    ctx = mp.get_context("fork")
    for c in (int(x) for x in args.configs.split(",")):
        n = args.limit or configs.config(c).n_plans
        tasks = [(c, a, min(PIECE, n - a)) for a in range(0, n, PIECE)]
        out = dict(makespan=np.empty(n), peak=np.empty(n), score=np.empty(n), gated=np.empty(n),
                   flags=np.zeros(n, np.uint8), device=np.full((n, 3), -1, np.int16))
        t0, done = time.time(), 0
        with ctx.Pool(args.workers) as pool:
            for start, *arrays in pool.imap_unordered(_eval_piece, tasks):
                m = len(arrays[0])
                for key, arr in zip(("makespan", "peak", "score", "gated", "flags", "device"), arrays):
                    out[key][start:start + m] = arr
                done += m
                if done % (PIECE * 16) == 0 or done == n:
                    dt = time.time() - t0
                    print(f"cfg{c}: {done}/{n} plans, {dt:.0f} s, {done / dt:.0f}/s", flush=True)
        doc = dict(config=c, seed=42, tag=c, **digest(**out))
        path = os.path.join(HERE, f"ref_full_cfg{c}.json" if not args.limit else f"ref_full_cfg{c}_first{n}.json")
        with open(path, "w") as f:
            json.dump(doc, f, separators=(",", ":"))
        print(f"cfg{c}: wrote {path} ({os.path.getsize(path)} bytes), argmax {doc['argmax']}/{doc['argmax_gated']}, "
              f"{doc['n_feasible']} feasible, {doc['n_stale_ok']} stale-ok", flush=True)


if __name__ == "__main__":
    main()
