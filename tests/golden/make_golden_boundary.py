"""Writes tests/golden/ref_boundary.json: what the REFERENCE's own `unroll`, `lower`, `NodeCostModel.time`,
`schedule`, `_device_peaks` and `mem_worst_violation` return when they are called one after the other as the
reference's pipeline calls them (pipeline.py:1015-1017, 1422-1497; runtime/job_plan.py:174-213).

Run in the development container only (it needs the read-only reference tree):

    python tests/golden/make_golden_boundary.py [--ref /root/reference]

For seeded plans of all five configurations the script records digests of the unrolled graph, of the lowered graph
(every field of every node, every edge, in order), of `time(node)` for every node, of the trace in the order of its
dictionaries, of the device-peak dictionary in ITS order, and the tuple `mem_worst_violation` returns -- the violating
device included -- under the configuration's memory and under a quarter of it (so that most plans violate).
`summary()` below computes the same record from any implementation of those names; the tests call it on this
repository's drop-in modules.  Only data is written.
"""

from __future__ import annotations

import argparse
import dataclasses
import json
import os
import sys
import zlib

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

N_PLANS = 24
TIGHT = 0.25


def _crc(obj) -> int:
    return zlib.crc32(json.dumps(obj, separators=(",", ":")).encode())


def _val(x):
    return getattr(x, "value", x)


def _alloc(a):
    return [list(a.origin), list(a.extent)]


def summary(api, rpeg, plan, wl, suite, hw, space, K_eval, trainable, shadow):
    """The recorded digest, from the functions in `api` (a dict of the reference's names)."""
    unrolled = api["unroll"](rpeg, K_eval, verbose=False)
    lowered = api["lower"](rpeg, unrolled, plan, suite, K_eval, workload=wl, verbose=False)
    cost = api["NodeCostModel"](hw, suite, wl)
    out = {}
    out["unroll"] = [len(unrolled.nodes), len(unrolled.data_edges), len(unrolled.pub_edges),
                     _crc([[e.src.template_vertex.id, e.src.k, e.dst.template_vertex.id, e.dst.k, e.container.name,
                            _val(e.kind)] for e in unrolled.pub_edges + unrolled.data_edges])]
    rows = []
    for n in lowered.nodes:
        rows.append([n.id, _val(n.kind), [_alloc(a) for a in n.allocs],
                     None if n.op is None else [n.op.template_vertex.id, n.op.k],
                     None if n.model is None else _val(n.model), None if n.pi is None else list(n.pi), n.mb,
                     n.n_seqs, n.n_active, n.phase_steps, n.phase_t_start, bool(n.is_prefill_phase),
                     int(n.payload_in_bytes), n.label])
    out["n_nodes"], out["nodes_crc"], out["first_nodes"] = len(rows), _crc(rows), rows[:3] + rows[-2:]
    edges = [[e.src.id, e.dst.id] for e in lowered.edges]
    out["n_edges"], out["edges_crc"] = len(edges), _crc(edges)
    times = [float(cost.time(n)).hex() for n in lowered.nodes]
    out["times_crc"], out["first_times"] = _crc(times), times[:4] + times[-2:]
    trace = api["schedule"](executable=lowered, cost_model=cost, device_space=space)
    out["makespan"] = float(trace.makespan()).hex()
    out["trace_crc"] = _crc([[n.id, float(s).hex(), float(trace.finish[n]).hex()] for n, s in trace.start.items()])
    out["memory"] = []
    for scale in (1.0, TIGHT):
        hw_s = dataclasses.replace(hw, memory_per_gpu=hw.memory_per_gpu * scale)
        mm = api["NodeMemoryModel"](hw_s, suite, wl, trainable=frozenset(trainable), shadow_models=frozenset(shadow))
        peaks = api["_device_peaks"](lowered, mm)
        viol = api["mem_worst_violation"](lowered, mm)
        out["memory"].append(dict(
            n_devices=len(peaks), peaks_crc=_crc([[list(d), float(p).hex()] for d, p in peaks.items()]),
            first_device=list(next(iter(peaks))),
            violation=None if viol is None else [list(viol[0]), float(viol[1]).hex(), float(viol[2]).hex()]))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--ref", default="/root/reference")
    args = ap.parse_args()
    sys.path.insert(0, HERE)
    import make_golden as mg
    mods = mg.load_reference(args.ref)
    api = dict(unroll=mods["passes.unroll"].unroll, lower=mods["passes.lower"].lower,
               NodeCostModel=mods["model.cost"].NodeCostModel, schedule=mods["schedule.scheduler"].schedule,
               NodeMemoryModel=mods["model.memory"].NodeMemoryModel, _device_peaks=mods["model.memory"]._device_peaks,
               mem_worst_violation=mods["model.memory"].mem_worst_violation)
    from tests.helpers import seeded_batch
    doc = {"n_plans": N_PLANS, "tight": TIGHT, "configs": {}}
    for c in (1, 2, 3, 4, 5):
        cfg, batch = seeded_batch(c, N_PLANS)
        rows = []
        for i in range(N_PLANS):
            rpeg, plan, wl, suite, hw, space = mg.to_reference(mods, cfg.problem, batch, i)
            shadow = [m for m in rpeg.trainable if rpeg.tau.get(m, 0) > 0]
            rows.append(summary(api, rpeg, plan, wl, suite, hw, space, cfg.problem.K_eval, rpeg.trainable, shadow))
        doc["configs"][str(c)] = rows
        nv = [sum(r["memory"][k]["violation"] is not None for r in rows) for k in (0, 1)]
        print(f"config {c}: {len(rows)} plans, violations {nv[0]} / {nv[1]} (tight)", flush=True)
    path = os.path.join(HERE, "ref_boundary.json")
    with open(path, "w") as f:
        json.dump(doc, f, separators=(",", ":"))
    print(f"wrote {path} ({os.path.getsize(path)} bytes)")


if __name__ == "__main__":
    main()
