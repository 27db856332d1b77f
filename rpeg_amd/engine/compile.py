"""Problem compiler: evaluates everything that does not depend on the candidate plan once, on the
host, with exact Python integer/float semantics, and packs it into the C ABI's rpeg_problem_t.

What is folded here (reference file:line):
  * generation phases per split variant           RPEG/passes/lower.py:288-327
  * work FLOPs of every operator-node variant      RPEG/model/cost.py:481-535  (ints of up to 65 bits,
    converted to float exactly as Python's int -> float conversion rounds them)
  * prefill work of generation nodes               RPEG/model/cost.py:383
  * container payloads and per-phase sub payloads  RPEG/passes/lower.py:523, 562-563
  * template order facts: LIFO topological order, same-model consecutive pairs, data reachability,
    sorted-id tie-break index                      RPEG/passes/lower.py:135-220, scheduler.py:385-397
  * which vertex pairs decide the lowered topology (relation table of the class signature)
"""

from __future__ import annotations

from typing import Dict, List, Tuple

from ..model.models import transformer_parameter_count
from . import abi
from .problem import EvalProblem

_LIMIT = 1 << 53


def gen_phases(workload) -> List[Tuple[int, int, int, int, bool]]:
    """(n_active, n_seqs, steps, t_start, is_prefill) per quantile (lower.py:288-327)."""
    total = workload.B * workload.K
    out, prev_step, prev_done = [], 0, 0
    for q, (frac, tokens) in enumerate(workload.gen_quantiles):
        done = round(frac * total)
        step = tokens - 1
        out.append((total - prev_done, done - prev_done, max(step - prev_step, 0), prev_step, q == 0))
        prev_step, prev_done = step, done
    return out


def _work(role: str, model: str, spec, wl, ckpt: bool, n_seqs=None, phase=None):
    """_work_cost (cost.py:481-535): int for inference/training, float for generation."""
    B, K, S, T = wl.B, wl.K, wl.S, wl.T
    L, d, d_ff, V = spec.L, spec.d, spec.d_ff, spec.V
    if role == "GEN":
        if phase is not None:
            n, _, steps, t0, pf = phase
            avg_past = S + t0 + steps / 2
            dec = n * (2 * steps * L * (4 * d ** 2 + 2 * d * d_ff + avg_past * d) + 2 * steps * V * d)
            if pf:
                return n * ((S * 2 * L) * (4 * d ** 2 + 2 * d * d_ff + S * d) + 2 * V * d) + dec
            return dec
        pre = B * K * ((S * 2 * L) * (4 * d ** 2 + 2 * d * d_ff + S * d) + 2 * V * d)
        dec = B * K * (2 * (T - 1) * L * (4 * d ** 2 + 2 * d * d_ff + (S + (T / 2)) * d) + 2 * (T - 1) * V * d)
        return pre + dec
    core = 2 * L * (4 * d ** 2 + 2 * d * d_ff + (S + T) * d)
    if role == "INF":
        n = n_seqs if n_seqs is not None else B * K
        if model in ("Pi", "Ref"):
            return n * (S + T) * (core + 2 * V * d)
        if model in ("V", "AC"):
            return n * (S + T) * (core + 2 * d)
        if model == "R":
            return n * (S + T) * core + n * (2 * d)
    if role == "TRAIN":
        mult = 4 if ckpt else 3
        if model == "Pi":
            return mult * B * K * (S + T) * (core + 2 * V * d)
        if model == "V":
            return mult * B * K * (S + T) * (core + 2 * d)
        if model == "AC":
            return mult * B * K * (S + T) * (core + 2 * V * d + 2 * d)
    raise ValueError(f"_work_cost: unhandled (role={role}, model={model})")


def _opconst(oc, role, model, spec, wl, ckpt, phase=None):
    B, K, S, T = wl.B, wl.K, wl.S, wl.T
    oc.sub = 0 if phase is None else 1
    if role == "GEN":
        oc.W = float(_work("GEN", model, spec, wl, ckpt, phase=phase))
        if phase is None:
            oc.n_eff, oc.steps, oc.prefill, oc.avg_past = B * K, T - 1, 1, S + T / 2
        else:
            n_act, _, steps, t0, pf = phase
            oc.n_eff, oc.steps, oc.prefill, oc.avg_past = n_act, steps, int(pf), S + t0 + steps / 2
        n_pf = oc.n_eff
        L, d, d_ff, V = spec.L, spec.d, spec.d_ff, spec.V
        oc.W_prefill = float(n_pf * ((S * 2 * L) * (4 * d ** 2 + 2 * d * d_ff + S * d) + 2 * V * d)) if oc.prefill else 0.0
    else:
        n = B * K if phase is None else phase[1]
        oc.n_eff = n
        oc.W = float(_work(role, model, spec, wl, ckpt, n_seqs=None if phase is None else n))
        oc.W_prefill, oc.avg_past, oc.steps, oc.prefill = 0.0, 0.0, 0, 0


def _lifo_topo(vertices, data_edges):
    """Kahn with a LIFO work list (lower.py:135-167)."""
    indeg = {v: 0 for v in vertices}
    succ = {v: [] for v in vertices}
    for e in data_edges:
        succ[e.src].append(e.dst)
        indeg[e.dst] += 1
    work = [v for v in vertices if indeg[v] == 0]
    order = []
    while work:
        v = work.pop()
        order.append(v)
        for w in succ[v]:
            indeg[w] -= 1
            if indeg[w] == 0:
                work.append(w)
    if len(order) != len(vertices):
        raise ValueError("Template data edge graph has a cycle.")
    return order


def _reach(vertices, data_edges):
    succ = {v: [] for v in vertices}
    for e in data_edges:
        succ[e.src].append(e.dst)
    out = set()
    for s in vertices:
        seen, todo = set(), list(succ[s])
        while todo:
            v = todo.pop()
            if v not in seen:
                seen.add(v)
                out.add((s, v))
                todo.extend(succ[v])
    return out


def compile_problem(problem: EvalProblem, check_sizes: bool = True) -> abi.ProblemT:
    """`check_sizes=False` for tables that only the host lowering reads: no horizon bound, no message-size bound."""
    wl, hw, sp, pol = problem.workload, problem.hw, problem.device_space, problem.memory_policy
    P = abi.ProblemT()
    P.abi_version = abi.ABI_VERSION
    if len(problem.structures) > abi.MAX_STRUCT:
        raise ValueError("too many structures")
    P.n_struct, P.n_split, P.K_eval = len(problem.structures), problem.n_splits(), problem.K_eval
    if P.n_split > abi.MAX_SPLIT:
        raise ValueError(f"at most {abi.MAX_PH} generation quantiles are supported")
    if problem.K_eval < 1 or (check_sizes and problem.K_eval > 4095):
        # (what bounds the horizon is the size of a lowered graph: 4,095 nodes per class, reported by the engine
        # when a plan's class exceeds it -- a few hundred steps, depending on the template)
        raise ValueError("K_eval must be in 1..4095")
    P.R, P.N, P.G = sp.R, sp.N, sp.G
    P.B, P.K, P.S, P.T = wl.B, wl.K, wl.S, wl.T
    P.optimizer_stage, P.ckpt = pol.optimizer_stage, int(pol.activation_checkpointing)
    P.max_groups = pol.max_worker_groups_per_gpu
    tp = problem.transfer_resource_policy
    P.transfer_both = int(tp.weight == "both_endpoints") | int(tp.activation == "both_endpoints") << 1
    for i, name in enumerate(abi.HW_FIELDS):
        P.hw[i] = float(getattr(hw, name))
    for name in ("op_generation_scale", "op_inference_scale", "op_training_scale", "weight_comm_scale",
                 "reshard_scale"):
        v = float(getattr(hw, name))
        if not (v > 0.0 and v < float("inf")):
            raise ValueError(f"hardware.{name} must be finite and > 0")   # cost.py:52-61
    if not (0.0 <= float(hw.activation_comm_overhead_s) < float("inf")):
        raise ValueError("hardware.activation_comm_overhead_s must be finite and >= 0")
    P.cap = (1 - pol.runtime_overhead_fraction) * hw.memory_per_gpu
    P.group_overhead = pol.worker_overhead_bytes + pol.semantic_activation_cache_bytes
    P.score_num = float(problem.K_eval * (wl.B * wl.K * (wl.S + wl.T)))

    phases: Dict[int, list] = {0: []}
    for j in range(1, P.n_split):
        phases[j] = gen_phases(problem.workload_for(j))
        for q, ph in enumerate(phases[j]):
            rec = P.phase[j][q]
            rec.n_active, rec.n_seqs, rec.steps, rec.t_start, rec.prefill = ph[0], ph[1], ph[2], ph[3], int(ph[4])
    for j in range(P.n_split):
        P.n_phase[j] = len(phases[j])

    for m, spec in problem.suite.specs.items():
        rec = P.model[abi.MODEL[m.value]]
        rec.L, rec.d, rec.d_ff, rec.V, rec.sb, rec.kind = spec.L, spec.d, spec.d_ff, spec.V, spec.dtype_bytes, abi.MODEL[m.value]
        rec.w_layer = 4 * spec.d ** 2 + 2 * spec.d * spec.d_ff
        rec.params_formula = spec.L * rec.w_layer + spec.V * spec.d
        rec.n_params = transformer_parameter_count(spec, m)
        big = wl.B * wl.K * (wl.S + wl.T) * spec.d * spec.dtype_bytes
        if check_sizes and max(big, 12 * rec.n_params * 4, rec.n_params * spec.dtype_bytes * sp.num_devices()) >= _LIMIT:
            raise ValueError("workload too large for exact float64 message sizes")

    total = wl.B * wl.K
    for s, structure in enumerate(problem.structures):
        rpeg = problem.template(s)
        if len(rpeg.vertices) > abi.MAX_V or len(rpeg.data_edges) > abi.MAX_E or len(rpeg.pub_edges) > abi.MAX_PUB:
            raise ValueError("template too large")
        S_ = P.st[s]
        vidx = {v: i for i, v in enumerate(rpeg.vertices)}
        S_.n_vertex, S_.n_edge, S_.n_pub = len(rpeg.vertices), len(rpeg.data_edges), len(rpeg.pub_edges)
        S_.n_tau = len(structure.tau_models)
        tau_slot = {m: i for i, m in enumerate(structure.tau_models)}
        if set(tau_slot) != set(rpeg.trainable):
            raise ValueError("structure tau_models must list exactly the trainable models")
        for m in rpeg.trainable:
            S_.trainable[abi.MODEL[m.value]] = 1
        for m in (rpeg.trainable if structure.memory_trainable is None else structure.memory_trainable):
            S_.mem_trainable[abi.MODEL[m.value]] = 1
        sorted_ids = sorted(v.id for v in rpeg.vertices)
        for i, v in enumerate(rpeg.vertices):
            rec = S_.vertex[i]
            role, model = v.kind.role.value, v.kind.model.value
            spec = problem.suite.specs[v.kind.model]
            rec.role, rec.model, rec.topo_idx = abi.ROLE[role], abi.MODEL[model], sorted_ids.index(v.id)
            rec.tau_slot = tau_slot.get(v.kind.model, -1)
            _opconst(rec.unsplit, role, model, spec, wl, pol.activation_checkpointing)
            if role in ("GEN", "INF"):
                for j in range(1, P.n_split):
                    for q, ph in enumerate(phases[j]):
                        _opconst(rec.sub[j][q], role, model, spec, wl, pol.activation_checkpointing, phase=ph)
        reach = _reach(rpeg.vertices, rpeg.data_edges)
        for (a, b) in reach:
            S_.reach[vidx[a]][vidx[b]] = 1
        rel: Dict[Tuple[int, int], int] = {}

        def need(a, b, flag):
            if a == b:
                return
            key = (min(a, b), max(a, b))
            rel[key] = rel.get(key, 0) | flag

        for i, e in enumerate(rpeg.data_edges):
            rec = S_.edge[i]
            rec.src, rec.dst = vidx[e.src], vidx[e.dst]
            rec.is_weight = int(str(e.container.name or "").startswith("W_"))
            rec.gen_inf = int(e.src.kind.role.value == "GEN" and e.dst.kind.role.value == "INF")
            rec.full_bytes = e.container.bytes()
            for j in range(1, P.n_split):
                for q, ph in enumerate(phases[j]):
                    rec.sub_bytes[j][q] = max(1, int(rec.full_bytes * (ph[1] / total)))
            need(rec.src, rec.dst, abi.NEED_DISJ if rec.gen_inf else 0)
        for i, e in enumerate(rpeg.pub_edges):
            rec = S_.pub[i]
            rec.src, rec.dst = vidx[e.src], vidx[e.dst]
            rec.model, rec.tau_slot = abi.MODEL[e.src.kind.model.value], tau_slot[e.src.kind.model]
            need(rec.src, rec.dst, abi.NEED_PI)
        order = _lifo_topo(rpeg.vertices, rpeg.data_edges)
        last, pairs = {}, []
        for v in order:
            m = v.kind.model
            if m in rpeg.trainable:
                if m in last:
                    pairs.append((last[m], v, m))
                last[m] = v
        if len(pairs) > abi.MAX_PAIR:
            raise ValueError("too many same-model vertex pairs")
        S_.n_pair = len(pairs)
        for i, (u, v, m) in enumerate(pairs):
            rec = S_.pair[i]
            rec.u, rec.v, rec.model, rec.tau_slot = vidx[u], vidx[v], abi.MODEL[m.value], tau_slot[m]
            rec.reach = int((u, v) in reach)
            need(rec.u, rec.v, abi.NEED_PI | abi.NEED_DISJ)
        # lifetime barriers (lower.py:752-793) compare a serving producer that returns to training
        # with the serving consumer of another model's publication
        producers = [u for (u, v, _m) in pairs if u.kind.role.value != "TRAIN" and v.kind.role.value == "TRAIN"]
        consumers = [e.dst for e in rpeg.pub_edges] + [v for (u, v, _m) in pairs
                                                       if u.kind.role.value == "TRAIN" and v.kind.role.value != "TRAIN"]
        for a in producers:
            for b in consumers:
                if a.kind.model != b.kind.model:
                    need(vidx[a], vidx[b], abi.NEED_DISJ)
        if len(rel) > abi.MAX_REL:
            raise ValueError("too many relation pairs")
        S_.n_rel = len(rel)
        for i, ((a, b), flags) in enumerate(sorted(rel.items())):
            S_.rel[i].u, S_.rel[i].v, S_.rel[i].flags = a, b, flags
    return P
