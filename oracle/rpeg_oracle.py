"""CPU oracle for the RPEG plan-evaluation path.  TEST INFRASTRUCTURE ONLY.

This module restates, in plain Python, the algorithm the reference runs for one
call of ``search.evaluate._eval_worker``: unroll -> lower -> node cost ->
list scheduling -> makespan/score -> per-device memory peaks -> soft OOM
penalty.  It is the checker for the HIP engine; nothing in the shipped package
imports it.  It follows the reference's evaluation order exactly (dict
insertion order, heap tie counters, left-to-right float expressions) because
the bar is bit-exact scores.

Objects are duck-typed: any template graph / plan / suite / workload /
hardware object that carries the reference's attribute names works, so the
same code runs on this repository's host mirror classes and on the
reference's own classes.

Reference files followed (relative to the reference tree):
  RPEG/core/types.py            geometry
  RPEG/passes/unroll.py         unroll
  RPEG/passes/lower.py          lowering, generation phases
  RPEG/passes/transfer_resources.py   device reservations of transfers
  RPEG/model/cost.py            node durations
  RPEG/model/memory.py          per-device peaks
  RPEG/schedule/scheduler.py    list scheduler
  RPEG/schedule/trace.py        makespan / throughput
  RPEG/search/evaluate.py       validity, score, penalty

Pins (see tests/test_oracle_*.py): golden vectors written by the reference
itself (tests/golden/*.json), closed forms from the reference's README files,
brute-force schedulers and per-device memory enumeration.
"""

from __future__ import annotations

import heapq
import math
import re
from collections import defaultdict, deque

GEN, INF, TRAIN = "GEN", "INF", "TRAIN"
ACTOR, CRITIC, REFERENCE, REWARD, AC_SHARE = "Pi", "V", "Ref", "R", "AC"
OP, COMM, RESHARD = "op", "comm", "reshard"
OOM_BETA = 40.0  # RPEG/search/evaluate.py:296


def _role(v):
    return v.kind.role.value


def _model(v):
    return v.kind.model.value


# --------------------------------------------------------------------------- geometry
def packing_geometry(dp, pp, tp, G):
    """RPEG/core/types.py:16-57."""
    s = min(pp, G // tp)
    if s == 0 or pp % s != 0:
        return None
    per_rep = s * tp
    span = pp // s
    if span != 1:
        return (G, dp * span)
    fit = G // per_rep
    if dp <= fit:
        return (dp * per_rep, 1)
    if dp % fit == 0:
        return (G, dp // fit)
    return None


def rectangular_node_layouts(nodes_needed, R, N):
    """RPEG/core/types.py:60-85."""
    if nodes_needed <= 0 or R <= 0 or N <= 0:
        return ()
    out = []
    for r_ext in range(1, min(R, nodes_needed) + 1):
        if nodes_needed % r_ext == 0 and nodes_needed // r_ext <= N:
            out.append((r_ext, nodes_needed // r_ext))
    return tuple(out)


def is_compatible(alloc, pi, space):
    """RPEG/search/evaluate.py:50-94."""
    dp, pp, tp = pi
    if tp > space.G:
        return False
    geom = packing_geometry(dp, pp, tp, space.G)
    if geom is None:
        return False
    if alloc.extent[2] != geom[0]:
        return False
    if (alloc.extent[0], alloc.extent[1]) not in rectangular_node_layouts(geom[1], space.R, space.N):
        return False
    lim = (space.R, space.N, space.G)
    for ax in range(3):
        if alloc.origin[ax] < 0 or alloc.origin[ax] + alloc.extent[ax] > lim[ax]:
            return False
    return True


def allocs_disjoint(a, b):
    """RPEG/passes/lower.py:223-239."""
    for ax in range(3):
        if a.origin[ax] + a.extent[ax] <= b.origin[ax] or b.origin[ax] + b.extent[ax] <= a.origin[ax]:
            return True
    return False


def allocations_overlap(a, b):
    """RPEG/search/evaluate.py:97-112."""
    return all(
        a.origin[ax] < b.origin[ax] + b.extent[ax] and b.origin[ax] < a.origin[ax] + a.extent[ax]
        for ax in range(3)
    )


def alloc_overlap_size(a, b):
    """RPEG/passes/lower.py:242-262."""
    vol = 1
    for ax in range(3):
        lo = max(a.origin[ax], b.origin[ax])
        hi = min(a.origin[ax] + a.extent[ax], b.origin[ax] + b.extent[ax])
        if hi <= lo:
            return 0
        vol *= hi - lo
    return vol


def alloc_key(a):
    return (tuple(a.origin), tuple(a.extent))


def alloc_size(a):
    return a.extent[0] * a.extent[1] * a.extent[2]


def stale_publication_layout_valid(rpeg, plan):
    """RPEG/search/evaluate.py:115-140."""
    for e in rpeg.pub_edges:
        if int(rpeg.tau.get(e.src.kind.model, 0)) <= 0:
            continue
        if allocations_overlap(plan.sigma[e.src], plan.sigma[e.dst]):
            return False
    return True


def plan_structurally_valid(rpeg, plan, space, suite, workload):
    """Integer part of RPEG/search/evaluate.py:143-200 (coverage, divisibility,
    microbatch rule, packing/layout), without the stale-layout and memory gates."""
    for v in rpeg.vertices:
        if v not in plan.sigma or v not in plan.pi or v not in plan.mb:
            return False
        dp, pp, tp = plan.pi[v]
        mb = plan.mb[v]
        L = suite.specs[v.kind.model].L
        if workload.B % dp != 0 or space.G % tp != 0 or L % pp != 0:
            return False
        if pp == 1:
            if mb != 1:
                return False
        elif (workload.B // dp) % mb != 0:
            return False
        if not is_compatible(plan.sigma[v], (dp, pp, tp), space):
            return False
    return True


# --------------------------------------------------------------------------- unroll
def unroll(rpeg, K_eval):
    """RPEG/passes/unroll.py:85-152.  Returns (nodes, data_edges, pub_edges) with
    nodes = [(vertex, k)], edges = [((u,k),(v,k'), container)]."""
    if K_eval <= 0:
        raise ValueError("K_eval must be >= 1")
    nodes = [(v, k) for k in range(K_eval) for v in rpeg.vertices]
    data = [((e.src, k), (e.dst, k), e.container) for k in range(K_eval) for e in rpeg.data_edges]
    pubs = []
    for k in range(1, K_eval):
        for e in rpeg.pub_edges:
            t = rpeg.tau[e.src.kind.model]
            if k <= t:
                continue
            pubs.append(((e.src, max(0, k - (t + 1))), (e.dst, k), e.container))
    return nodes, data, pubs


# --------------------------------------------------------------------------- lowering
class XNode:
    """Executable-graph node (RPEG/passes/lower.py:30-81)."""

    __slots__ = ("id", "kind", "allocs", "tpl", "k", "model", "pi", "mb", "n_seqs", "n_active",
                 "phase_steps", "phase_t_start", "is_prefill_phase", "payload", "label")

    def __init__(self, id, kind, allocs, tpl=None, k=None, model=None, pi=None, mb=None,
                 n_seqs=None, n_active=None, phase_steps=None, phase_t_start=None,
                 is_prefill_phase=False, payload=0, label=None):
        self.id, self.kind, self.allocs = id, kind, allocs
        self.tpl, self.k, self.model, self.pi, self.mb = tpl, k, model, pi, mb
        self.n_seqs, self.n_active = n_seqs, n_active
        self.phase_steps, self.phase_t_start = phase_steps, phase_t_start
        self.is_prefill_phase = is_prefill_phase
        self.payload, self.label = payload, label

    def __repr__(self):
        return f"<{self.id}>"


def gen_phases(workload):
    """RPEG/passes/lower.py:288-327 -> [(n_active, n_seqs, steps, t_start, is_prefill)]."""
    total = workload.B * workload.K
    out = []
    prev_step = 0
    prev_done = 0
    for q, (frac, tokens) in enumerate(workload.gen_quantiles):
        done = round(frac * total)
        step = tokens - 1
        out.append((total - prev_done, done - prev_done, max(step - prev_step, 0), prev_step, q == 0))
        prev_step, prev_done = step, done
    return out


def template_topo_order(rpeg):
    """RPEG/passes/lower.py:135-167 (Kahn with a LIFO work list)."""
    indeg = {v: 0 for v in rpeg.vertices}
    succ = {v: [] for v in rpeg.vertices}
    for e in rpeg.data_edges:
        succ[e.src].append(e.dst)
        indeg[e.dst] += 1
    stack = [v for v in rpeg.vertices if indeg[v] == 0]
    order = []
    while stack:
        v = stack.pop()
        order.append(v)
        for w in succ[v]:
            indeg[w] -= 1
            if indeg[w] == 0:
                stack.append(w)
    if len(order) != len(rpeg.vertices):
        raise ValueError("template data edges form a cycle")
    return order


def data_reachable(rpeg):
    """RPEG/passes/lower.py:170-193."""
    succ = {v: [] for v in rpeg.vertices}
    for e in rpeg.data_edges:
        succ[e.src].append(e.dst)
    reach = set()
    for s in rpeg.vertices:
        seen = set()
        todo = list(succ[s])
        while todo:
            v = todo.pop()
            if v in seen:
                continue
            seen.add(v)
            reach.add((s, v))
            todo.extend(succ[v])
    return reach


def within_step_priors(order, trainable):
    """RPEG/passes/lower.py:196-220."""
    last = {}
    out = []
    for v in order:
        m = v.kind.model
        if m not in trainable:
            continue
        if m in last:
            out.append((last[m], v, m))
        last[m] = v
    return out


def lower(rpeg, plan, suite, K_eval, workload):
    """RPEG/passes/lower.py:330-851 with intra_stage_fusion=False.
    Returns (nodes, edges): nodes = list of XNode in dict-insertion order,
    edges = list of (src XNode, dst XNode) in append order."""
    unodes, udata, upubs = unroll(rpeg, K_eval)
    nodes = {}
    edges = []
    seen = set()

    def add_edge(a, b):
        key = (a.id, b.id)
        if key not in seen:
            seen.add(key)
            edges.append((a, b))

    def n_params(model):
        return transformer_parameter_count(suite.specs[model], model)

    phases = gen_phases(workload) if (workload is not None and workload.gen_quantiles) else None

    gen_first, gen_last, gen_subs, inf_first, inf_subs = {}, {}, {}, {}, {}

    split_gen = set()
    if phases:
        for (u, _k), (v, _k2), _c in udata:
            if _role(u) == GEN and _role(v) == INF and allocs_disjoint(plan.sigma[u], plan.sigma[v]):
                split_gen.add(u.id)

    # stage 1: operator nodes (lower.py:433-474)
    for (tpl, k) in unodes:
        nid = f"{tpl.id}@{k}"
        if phases and _role(tpl) == GEN and tpl.id in split_gen:
            ids = []
            for q, (n_act, n_seq, steps, t0, pf) in enumerate(phases):
                sid = f"{tpl.id}@{k}:g{q}"
                nodes[sid] = XNode(sid, OP, (plan.sigma[tpl],), tpl=tpl, k=k, model=tpl.kind.model,
                                   pi=plan.pi[tpl], mb=plan.mb.get(tpl), n_seqs=n_seq, n_active=n_act,
                                   phase_steps=steps, phase_t_start=t0, is_prefill_phase=pf)
                ids.append(sid)
            for q in range(1, len(ids)):
                add_edge(nodes[ids[q - 1]], nodes[ids[q]])
            gen_first[nid], gen_last[nid], gen_subs[nid] = ids[0], ids[-1], ids
        else:
            nodes[nid] = XNode(nid, OP, (plan.sigma[tpl],), tpl=tpl, k=k, model=tpl.kind.model,
                               pi=plan.pi[tpl], mb=plan.mb.get(tpl))

    # stage 2: data edges / COMM insertion (lower.py:476-597)
    ctr = {"comm": 0, "reshard": 0}

    def edge_or_comm(a, b, payload, label):
        if alloc_key(a.allocs[0]) == alloc_key(b.allocs[0]):
            add_edge(a, b)
            return
        ctr["comm"] += 1
        c = XNode(f"comm{ctr['comm']}", COMM, (a.allocs[0], b.allocs[0]), payload=payload, label=label)
        nodes[c.id] = c
        add_edge(a, c)
        add_edge(c, b)

    first_pass, second_pass = [], []
    for e in udata:
        (u, k), (v, _k2), _c = e
        if f"{u.id}@{k}" in gen_subs and _role(v) == INF:
            first_pass.append(e)
        else:
            second_pass.append(e)

    for (u, k), (v, k2), cont in first_pass + second_pass:
        s_id, d_id = f"{u.id}@{k}", f"{v.id}@{k2}"
        full = cont.count * cont.elem_size_bytes
        label = cont.name
        if s_id in gen_subs and _role(v) == INF:
            if allocs_disjoint(plan.sigma[u], plan.sigma[v]):
                total = workload.B * workload.K
                if d_id not in inf_subs:
                    nodes.pop(d_id, None)
                    ids = []
                    for q, ph in enumerate(phases):
                        sid = f"{v.id}@{k2}:i{q}"
                        nodes[sid] = XNode(sid, OP, (plan.sigma[v],), tpl=v, k=k2, model=v.kind.model,
                                           pi=plan.pi[v], mb=plan.mb.get(v), n_seqs=ph[1])
                        ids.append(sid)
                    for q in range(1, len(ids)):
                        add_edge(nodes[ids[q - 1]], nodes[ids[q]])
                    inf_first[d_id], inf_subs[d_id] = ids[0], ids
                for q in range(len(phases)):
                    frac = phases[q][1] / total
                    edge_or_comm(nodes[gen_subs[s_id][q]], nodes[inf_subs[d_id][q]],
                                 max(1, int(full * frac)), label)
            else:
                edge_or_comm(nodes[gen_last[s_id]], nodes[d_id], full, label)
        elif s_id in gen_subs:
            edge_or_comm(nodes[gen_last[s_id]], nodes[d_id], full, label)
        elif s_id in inf_subs:
            dst = nodes.get(d_id)
            if dst is None:
                raise KeyError(f"Destination node {d_id} not found")
            edge_or_comm(nodes[inf_subs[s_id][-1]], dst, full, label)
        else:
            edge_or_comm(nodes[s_id], nodes[d_id], full, label)

    # stage 3: within-step weight reshards (lower.py:626-681)
    pairs = within_step_priors(template_topo_order(rpeg), rpeg.trainable)
    reach = data_reachable(rpeg)
    resharded = set()

    def mk_reshard(a, b, model):
        ctr["reshard"] += 1
        return XNode(f"reshard{ctr['reshard']}", RESHARD, (a.allocs[0], b.allocs[0]), model=model,
                     payload=n_params(model) * suite.specs[model].dtype_bytes, label=f"W_{model.value}")

    for u_t, v_t, model in pairs:
        au, av = plan.sigma[u_t], plan.sigma[v_t]
        if rpeg.tau.get(model, 0) > 0 and allocs_disjoint(au, av):
            continue
        if (u_t, v_t) in reach and alloc_key(au) != alloc_key(av):
            continue
        for k in range(K_eval):
            ui, vi = f"{u_t.id}@{k}", f"{v_t.id}@{k}"
            if ui in gen_last:
                a = nodes[gen_last[ui]]
            elif ui in inf_subs:
                a = nodes[inf_subs[ui][-1]]
            else:
                a = nodes[ui]
            if vi in gen_first:
                b = nodes[gen_first[vi]]
            elif vi in inf_first:
                b = nodes[inf_first[vi]]
            else:
                b = nodes[vi]
            same_alloc = alloc_key(a.allocs[0]) == alloc_key(b.allocs[0])
            if same_alloc and tuple(a.pi) == tuple(b.pi):
                continue
            if not same_alloc:
                add_edge(a, b)
            else:
                r = mk_reshard(a, b, model)
                nodes[r.id] = r
                add_edge(a, r)
                add_edge(r, b)
                resharded.add(v_t)

    # stage 4a: publication edges (lower.py:683-728)
    for (u, ku), (v, kv), _cont in upubs:
        a = nodes[f"{u.id}@{ku}"]
        d_id = f"{v.id}@{kv}"
        if d_id in gen_first:
            b = nodes[gen_first[d_id]]
        elif d_id in inf_first:
            b = nodes[inf_first[d_id]]
        else:
            b = nodes[d_id]
        model = a.model
        if b.tpl in resharded:
            continue
        same_alloc = alloc_key(a.allocs[0]) == alloc_key(b.allocs[0])
        if same_alloc and tuple(a.pi) == tuple(b.pi):
            add_edge(a, b)
            continue
        if same_alloc:
            r = mk_reshard(a, b, model)
            nodes[r.id] = r
            add_edge(a, r)
            add_edge(r, b)
        else:
            ctr["comm"] += 1
            full = n_params(model) * suite.specs[model].dtype_bytes
            n_max = max(alloc_size(a.allocs[0]), alloc_size(b.allocs[0]))
            n_ov = alloc_overlap_size(a.allocs[0], b.allocs[0])
            payload = full * (n_max - n_ov) // n_max if n_max > 0 else full
            c = XNode(f"comm{ctr['comm']}", COMM, (a.allocs[0], b.allocs[0]), payload=payload,
                      label=f"W_{model.value}")
            nodes[c.id] = c
            add_edge(a, c)
            add_edge(c, b)

    # stage 4b: colocated trainable-layout lifetime barriers (lower.py:730-793)
    preds, succs = {}, {}
    for a, b in edges:
        preds.setdefault(b.id, []).append(nodes[a.id])
        succs.setdefault(a.id, []).append(nodes[b.id])
    back_to_train, to_serving = [], []
    for t in nodes.values():
        if t.kind != RESHARD:
            continue
        p_ops = [n for n in preds.get(t.id, ()) if n.kind == OP]
        s_ops = [n for n in succs.get(t.id, ()) if n.kind == OP]
        if len(p_ops) != 1 or len(s_ops) != 1:
            continue
        p, s = p_ops[0], s_ops[0]
        if p.model != s.model or p.model not in rpeg.trainable:
            continue
        if _role(p.tpl) != TRAIN and _role(s.tpl) == TRAIN:
            back_to_train.append((t, p, s))
        elif _role(p.tpl) == TRAIN and _role(s.tpl) != TRAIN:
            to_serving.append((t, p, s))
    for ret, producer, _c in back_to_train:
        for pub, _p, consumer in to_serving:
            if producer.model == consumer.model or producer.k != consumer.k:
                continue
            if allocs_disjoint(producer.allocs[0], consumer.allocs[0]):
                continue
            if (producer.tpl, consumer.tpl) not in reach:
                continue
            add_edge(ret, pub)

    return list(nodes.values()), edges


# --------------------------------------------------------------------------- parameters
def base_transformer_params(spec):
    """RPEG/model/models.py:38-48."""
    if getattr(spec, "parameter_count", None) is not None:
        return int(spec.parameter_count)
    return spec.L * (4 * spec.d ** 2 + 2 * spec.d * spec.d_ff) + spec.V * spec.d


def transformer_parameter_count(spec, model):
    """RPEG/model/models.py:51-63."""
    return base_transformer_params(spec) + (spec.d if model.value in (CRITIC, REWARD, AC_SHARE) else 0)


# --------------------------------------------------------------------------- cost model
class CostModel:
    """RPEG/model/cost.py:33-686 (NodeCostModel)."""

    def __init__(self, hw, suite, workload, optimizer_stage=2, activation_checkpointing=True):
        self.hw, self.suite, self.wl = hw, suite, workload
        self.stage, self.ckpt = optimizer_stage, activation_checkpointing

    # -- tiers (RPEG/model/hardware.py:70-110)
    @staticmethod
    def _span(allocs):
        r0 = min(a.origin[0] for a in allocs)
        r1 = max(a.origin[0] + a.extent[0] for a in allocs)
        n0 = min(a.origin[1] for a in allocs)
        n1 = max(a.origin[1] + a.extent[1] for a in allocs)
        return r1 - r0, n1 - n0

    def tier_coll(self, allocs):
        dr, dn = self._span(allocs)
        h = self.hw
        if dr > 1:
            return h.alpha_coll_r, h.beta_coll_r
        if dn > 1:
            return h.alpha_coll_n, h.beta_coll_n
        return h.alpha_coll_g, h.beta_coll_g

    def tier_p2p(self, allocs):
        dr, dn = self._span(allocs)
        h = self.hw
        if dr > 1:
            return h.alpha_p2p_r, h.beta_p2p_r
        if dn > 1:
            return h.alpha_p2p_n, h.beta_p2p_n
        return h.alpha_p2p_g, h.beta_p2p_g

    # -- entry (cost.py:66-88)
    def time(self, nd):
        if nd.kind == OP:
            return self.op_time(nd)
        if nd.kind == COMM:
            return self.comm_time(nd)
        if nd.kind == RESHARD:
            return self.reshard_time(nd)
        raise ValueError("unknown node kind")

    def eff_batch(self, nd):
        """cost.py:131-145."""
        if nd.n_active is not None:
            return nd.n_active
        if nd.n_seqs is not None:
            return nd.n_seqs
        return self.wl.B * self.wl.K

    def eff_mb(self, nd):
        """cost.py:147-159."""
        return max(1, min(nd.mb, int(self.eff_batch(nd)) // max(1, nd.pi[0])))

    def role_scale(self, role):
        """cost.py:195-210."""
        h = self.hw
        return {GEN: h.op_generation_scale, INF: h.op_inference_scale, TRAIN: h.op_training_scale}.get(role, 1.0)

    def op_time(self, nd):
        """cost.py:161-193."""
        role = _role(nd.tpl)
        pd, pp, pt = nd.pi
        m = self.eff_mb(nd)
        bubble = (m + pp - 1) / m
        F = self.effective_flops(nd)
        t = (self.work_cost(nd) / (F * pd * pp * pt)) * bubble + self.intra_comm(nd)
        t += self.non_gemm(nd)
        if role == TRAIN:
            sp = self.suite.specs[nd.model]
            params = sp.L * (4 * sp.d ** 2 + 2 * sp.d * sp.d_ff) + sp.V * sp.d
            odp = pd if self.stage >= 1 else 1
            per_rank = params / (odp * pp * pt)
            t += (per_rank * 18) / self.hw.memory_bandwidth
        return t * self.role_scale(role)

    def breakdown(self, nd):
        """cost.py:90-128 (fields sum to op_time up to rounding)."""
        role = _role(nd.tpl)
        pd, pp, pt = nd.pi
        m = self.eff_mb(nd)
        F = self.effective_flops(nd)
        gemm = self.work_cost(nd) / (F * pd * pp * pt)
        parts = [gemm, gemm * (pp - 1) / m, self.intra_comm(nd), self.non_gemm(nd), 0.0]
        if role == TRAIN:
            sp = self.suite.specs[nd.model]
            params = sp.L * (4 * sp.d ** 2 + 2 * sp.d * sp.d_ff) + sp.V * sp.d
            odp = pd if self.stage >= 1 else 1
            parts[4] = ((params / (odp * pp * pt)) * 18) / self.hw.memory_bandwidth
        sc = self.role_scale(role)
        return tuple(p * sc for p in parts)

    def non_gemm(self, nd):
        """cost.py:212-269."""
        h = self.hw
        if h.non_gemm_constant == 0.0 and h.non_gemm_scaling == 0.0:
            return 0.0
        role = _role(nd.tpl)
        if role == GEN:
            return 0.0
        pd, pp, pt = nd.pi
        Lpp = self.suite.specs[nd.model].L / pp
        m = self.eff_mb(nd)
        b_local = self.eff_batch(nd) / (pd * m)
        B_cal = h.non_gemm_batch_cal
        scale = b_local / B_cal if B_cal > 0 else 1.0
        at_tp = Lpp * (h.non_gemm_constant + h.non_gemm_scaling / pt)
        at_tp1 = Lpp * (h.non_gemm_constant + h.non_gemm_scaling) / pt
        extra = (at_tp - at_tp1) * scale
        if role == TRAIN:
            extra *= 4 if self.ckpt else 3
        return max(0.0, extra)

    def effective_flops(self, nd):
        """cost.py:271-289."""
        if _role(nd.tpl) == GEN:
            return self.effective_flops_generation(nd)
        I = self.intensity(nd)
        eta = self.gemm_efficiency(nd)
        h = self.hw
        if I >= h.flops_per_gpu / h.memory_bandwidth:
            return h.flops_per_gpu * eta
        return I * h.memory_bandwidth

    def gemm_efficiency(self, nd):
        """cost.py:291-328."""
        h = self.hw
        M_half = h.gemm_m_half
        K_half = getattr(h, "gemm_k_half", 0.0)
        pd, pp, pt = nd.pi
        m = self.eff_mb(nd)
        b_local = self.eff_batch(nd) / (pd * m)
        M_eff = b_local * (self.wl.S + self.wl.T)
        eta_b = M_eff / (M_eff + M_half) if M_half > 0 else 1.0
        if pt > 1 and K_half > 0:
            sp = self.suite.specs[nd.model]
            K_min = min(sp.d // pt, sp.d_ff // pt)
            eta_t = K_min / (K_min + K_half)
        else:
            eta_t = 1.0
        return eta_b * eta_t

    def effective_flops_generation(self, nd):
        """cost.py:330-404."""
        h = self.hw
        pd, pp, pt = nd.pi
        P = pd * pp * pt
        S, T = self.wl.S, self.wl.T
        sp = self.suite.specs[nd.model]
        L, d, d_ff, V, sb = sp.L, sp.d, sp.d_ff, sp.V, sp.dtype_bytes
        Lpp = L / pp
        m = self.eff_mb(nd)
        b_local = self.eff_batch(nd) / (pd * m)
        if nd.phase_steps is not None:
            steps = nd.phase_steps
            avg_past = S + nd.phase_t_start + steps / 2
            prefill = nd.is_prefill_phase
        else:
            steps = T - 1
            avg_past = S + T / 2
            prefill = True
        omega_W = (Lpp / pt) * (4 * d ** 2 + 2 * d * d_ff) * sb
        M_half = h.gemm_m_half
        I_star = h.flops_per_gpu / h.memory_bandwidth
        EFF_W = h.decode_bw_eff
        EFF_KV = min(1.0, h.decode_bw_eff * 3.5)
        W_total = self.work_cost(nd)
        total = 0.0
        W_prefill = None
        if prefill:
            eta = (b_local * S) / (b_local * S + M_half) if M_half > 0 else 1.0
            fl = b_local * S * (2 * Lpp / pt) * (4 * d ** 2 + 2 * d * d_ff + S * d)
            omega_A = 2 * b_local * S * d * Lpp * sb
            I = fl / (omega_W + omega_A) if (omega_W + omega_A) > 0 else float("inf")
            F = h.flops_per_gpu * eta if I >= I_star else I * h.memory_bandwidth
            n_pf = self.eff_batch(nd)
            W_prefill = n_pf * ((S * 2 * L) * (4 * d ** 2 + 2 * d * d_ff + S * d) + 2 * V * d)
            total += W_prefill / (P * F) if F > 0 else 0
        if steps > 0:
            eta = b_local / (b_local + M_half) if M_half > 0 else 1.0
            fl = b_local * (2 * Lpp / pt) * (4 * d ** 2 + 2 * d * d_ff + avg_past * d)
            omega_A = 2 * b_local * d * Lpp * sb
            omega_KV = 2 * avg_past * (d / pt) * sb * b_local * Lpp
            omega = omega_W + omega_A + omega_KV
            eff = (omega_W * EFF_W + omega_KV * EFF_KV + omega_A * 1.0) / omega if omega > 0 else EFF_W
            bw = h.memory_bandwidth * eff
            I = fl / omega if omega > 0 else float("inf")
            F = h.flops_per_gpu * eta if I >= I_star else I * bw
            W_decode = W_total - W_prefill if prefill else W_total
            total += W_decode / (P * F) if F > 0 else 0
        if total > 0:
            return W_total / (P * total)
        return h.flops_per_gpu

    def intensity(self, nd):
        """cost.py:406-444."""
        pd, pp, pt = nd.pi
        sp = self.suite.specs[nd.model]
        L, d, d_ff, sb = sp.L, sp.d, sp.d_ff, sp.dtype_bytes
        Lpp = L / pp
        seq = self.wl.S + self.wl.T
        m = self.eff_mb(nd)
        b_local = self.eff_batch(nd) / (pd * m)
        fl = b_local * seq * (2 * Lpp / pt) * (4 * d ** 2 + 2 * d * d_ff + seq * d)
        omega_W = (Lpp / pt) * (4 * d ** 2 + 2 * d * d_ff) * sb
        omega_A = 2 * b_local * seq * d * Lpp * sb
        tot = omega_W + omega_A
        if tot <= 0:
            return float("inf")
        return fl / tot

    def comm_time(self, nd):
        """cost.py:446-462."""
        alpha, beta = self.tier_p2p(nd.allocs)
        p_min = min(alloc_size(nd.allocs[0]), alloc_size(nd.allocs[1]))
        t = alpha + (nd.payload / p_min) * beta
        if str(nd.label or "").startswith("W_"):
            return t * self.hw.weight_comm_scale
        return t + self.hw.activation_comm_overhead_s

    def reshard_time(self, nd):
        """cost.py:464-479."""
        P = alloc_size(nd.allocs[0])
        return self.hw.reshard_scale * self.collective("a2a", nd.payload / P, nd.allocs, P)

    def work_cost(self, nd):
        """cost.py:481-535."""
        role, model = _role(nd.tpl), nd.model.value
        B, K, S, T = self.wl.B, self.wl.K, self.wl.S, self.wl.T
        sp = self.suite.specs[nd.model]
        L, d, d_ff, V = sp.L, sp.d, sp.d_ff, sp.V
        if role == GEN:
            if nd.n_active is not None:
                n, steps = nd.n_active, nd.phase_steps
                avg_past = S + nd.phase_t_start + steps / 2
                dec = n * (2 * steps * L * (4 * d ** 2 + 2 * d * d_ff + avg_past * d) + 2 * steps * V * d)
                if nd.is_prefill_phase:
                    pre = n * ((S * 2 * L) * (4 * d ** 2 + 2 * d * d_ff + S * d) + 2 * V * d)
                    return pre + dec
                return dec
            pre = B * K * ((S * 2 * L) * (4 * d ** 2 + 2 * d * d_ff + S * d) + 2 * V * d)
            dec = B * K * (2 * (T - 1) * L * (4 * d ** 2 + 2 * d * d_ff + (S + (T / 2)) * d) + 2 * (T - 1) * V * d)
            return pre + dec
        if role == INF:
            n = nd.n_seqs if nd.n_seqs is not None else B * K
            if model in (ACTOR, REFERENCE):
                return n * (S + T) * (2 * L * (4 * d ** 2 + 2 * d * d_ff + (S + T) * d) + 2 * V * d)
            if model in (CRITIC, AC_SHARE):
                return n * (S + T) * (2 * L * (4 * d ** 2 + 2 * d * d_ff + (S + T) * d) + 2 * d)
            if model == REWARD:
                return n * (S + T) * (2 * L * (4 * d ** 2 + 2 * d * d_ff + (S + T) * d)) + n * (2 * d)
        if role == TRAIN:
            mult = 4 if self.ckpt else 3
            if model == ACTOR:
                return mult * B * K * (S + T) * (2 * L * (4 * d ** 2 + 2 * d * d_ff + (S + T) * d) + 2 * V * d)
            if model == CRITIC:
                return mult * B * K * (S + T) * (2 * L * (4 * d ** 2 + 2 * d * d_ff + (S + T) * d) + 2 * d)
            if model == AC_SHARE:
                return mult * B * K * (S + T) * (2 * L * (4 * d ** 2 + 2 * d * d_ff + (S + T) * d) + 2 * V * d + 2 * d)
        raise ValueError(f"work_cost: unhandled (role={role}, model={model})")

    def intra_comm(self, nd):
        """cost.py:538-652."""
        h = self.hw
        role, model = _role(nd.tpl), nd.model.value
        B, K, S, T = self.wl.B, self.wl.K, self.wl.S, self.wl.T
        sp = self.suite.specs[nd.model]
        L, d, d_ff, V, sb = sp.L, sp.d, sp.d_ff, sp.V, sp.dtype_bytes
        pd, pp, pt = nd.pi
        m = self.eff_mb(nd)
        a_tp, b_tp = h.alpha_coll_g, h.beta_coll_g

        def tp_ar(M, p):
            return 2 * (p - 1) * a_tp + 2 * (p - 1) / p * M * b_tp

        r_ext, n_ext, g_node = nd.allocs[0].extent
        s = g_node // pt
        per_rep = math.ceil(pp / s) if s > 0 else pp
        e_total = pp - 1
        e_inter = per_rep - 1
        e_intra = e_total - e_inter
        if r_ext > 1:
            a_x, b_x = h.alpha_p2p_r, h.beta_p2p_r
        elif n_ext > 1:
            a_x, b_x = h.alpha_p2p_n, h.beta_p2p_n
        else:
            a_x, b_x = h.alpha_p2p_g, h.beta_p2p_g
        a_i, b_i = h.alpha_p2p_g, h.beta_p2p_g

        def pp_p2p(M, n_steps):
            if e_total == 0 or n_steps == 0:
                return 0.0
            c_in = (e_intra / e_total) * n_steps * (a_i + M * b_i)
            c_x = (e_inter / e_total) * n_steps * (a_x + M * b_x)
            return c_in + c_x

        Lpp = L / pp
        if role == GEN:
            if nd.n_active is not None:
                n, steps = nd.n_active, nd.phase_steps
                cost = 0.0
                if nd.is_prefill_phase:
                    cost += pp_p2p((n * S * d * sb) / (pd * m), m + pp - 2)
                    cost += 2 * Lpp * m * tp_ar((n * S * d * sb) / (pd * m), pt)
                cost += pp_p2p((n * d * sb) / (pd * m), steps * (m + pp - 2))
                cost += 2 * steps * Lpp * m * tp_ar((n * d * sb) / (pd * m), pt)
                return cost
            return (pp_p2p((B * K * S * d * sb) / (pd * m), m + pp - 2)
                    + pp_p2p((B * K * d * sb) / (pd * m), (T - 1) * (m + pp - 2))
                    + 2 * Lpp * m * tp_ar((B * K * S * d * sb) / (pd * m), pt)
                    + 2 * (T - 1) * Lpp * m * tp_ar((B * K * d * sb) / (pd * m), pt))
        if role == INF:
            n = nd.n_seqs if nd.n_seqs is not None else B * K
            return (pp_p2p((n * (S + T) * d * sb) / (pd * m), m + pp - 2)
                    + 2 * Lpp * m * tp_ar((n * (S + T) * d * sb) / (pd * m), pt))
        if role == TRAIN:
            params = L * (4 * d ** 2 + 2 * d * d_ff) + V * d + (d if model in (CRITIC, AC_SHARE) else 0)
            g_msg = (params * sb) / (pp * pt)
            w_msg = (params * sb) / (pp * pt)
            if self.stage == 0:
                dp_comm = self.collective("ar", g_msg, nd.allocs, pd)
            elif self.stage == 1:
                dp_comm = self.collective("ar", g_msg, nd.allocs, pd) + self.collective("ag", w_msg, nd.allocs, pd)
            else:
                dp_comm = self.collective("rs", g_msg, nd.allocs, pd) + self.collective("ag", w_msg, nd.allocs, pd)
            n_tp = 6 if self.ckpt else 4
            return (dp_comm
                    + pp_p2p((B * K * (S + T) * d * sb) / (pd * m), m + 2 * pp - 3)
                    + n_tp * Lpp * m * tp_ar((B * K * (S + T) * d * sb) / (pd * m), pt))
        raise ValueError(f"intra_comm: unhandled (role={role}, model={model})")

    def collective(self, coll, M, allocs, p):
        """cost.py:655-686."""
        if coll in ("ag", "rs", "ar", "a2a"):
            alpha, beta = self.tier_coll(allocs)
        else:
            alpha, beta = self.tier_p2p(allocs)
        if coll in ("ag", "rs"):
            return (p - 1) * alpha + (p - 1) / p * M * beta
        if coll == "ar":
            return 2 * (p - 1) * alpha + 2 * (p - 1) / p * M * beta
        if coll == "a2a":
            return (p - 1) * alpha + M * beta
        return alpha + M * beta


# --------------------------------------------------------------------------- memory model
class MemModel:
    """RPEG/model/memory.py:188-575 (NodeMemoryModel), policy fields as in MemoryPolicy."""

    def __init__(self, hw, suite, workload, trainable, eps_rt=0.0, optimizer_stage=2,
                 worker_overhead_bytes=0.0, semantic_activation_cache_bytes=0.0,
                 max_worker_groups_per_gpu=0, activation_checkpointing=True):
        self.hw, self.suite, self.wl = hw, suite, workload
        self.trainable = frozenset(trainable)
        self.eps_rt, self.stage, self.ckpt = eps_rt, optimizer_stage, activation_checkpointing
        self.worker_overhead = worker_overhead_bytes
        self.act_cache = semantic_activation_cache_bytes
        self.max_groups = max_worker_groups_per_gpu
        self._cache = {}

    def capacity(self):
        """memory.py:291-298."""
        return (1 - self.eps_rt) * self.hw.memory_per_gpu

    def w_layer(self, model):
        sp = self.suite.specs[model]
        return 4 * sp.d ** 2 + 2 * sp.d * sp.d_ff

    def w_stage(self, model, p, pp):
        """memory.py:312-343."""
        sp = self.suite.specs[model]
        emb, head = sp.V * sp.d, sp.d
        split = math.ceil(sp.L / pp) * self.w_layer(model)
        mv = model.value
        if mv in (ACTOR, REFERENCE):
            rest = (emb if p == 1 else 0) + (emb if p == pp else 0)
        elif mv in (CRITIC, REWARD):
            rest = (emb if p == 1 else 0) + (head if p == pp else 0)
        elif mv == AC_SHARE:
            rest = (emb if p == 1 else 0) + (emb if p == pp else 0) + (head if p == pp else 0)
        else:
            raise ValueError
        return split, rest

    def w_stage_max(self, model, pp):
        """memory.py:345-365: first stage with the largest total."""
        key = (model, pp)
        if key not in self._cache:
            stages = [self.w_stage(model, p, pp) for p in range(1, pp + 1)]
            self._cache[key] = max(stages, key=lambda s: s[0] + s[1])
        return self._cache[key]

    def w_shard(self, nd):
        """memory.py:367-387."""
        split, rest = self.w_stage_max(nd.model, nd.pi[1])
        return math.ceil(split / nd.pi[2]) + rest

    def mem_weights(self, nd):
        return self.w_shard(nd) * self.suite.specs[nd.model].dtype_bytes

    def mem_optimizer(self, nd):
        dp = nd.pi[0] if self.stage >= 1 else 1
        return 12 * self.w_shard(nd) / dp

    def mem_gradients(self, nd):
        dp = nd.pi[0] if self.stage >= 2 else 1
        return self.suite.specs[nd.model].dtype_bytes * self.w_shard(nd) / dp

    def act_per_microbatch(self, nd):
        """memory.py:23-65."""
        sp = self.suite.specs[nd.model]
        L, d, d_ff, sb = sp.L, sp.d, sp.d_ff, sp.dtype_bytes
        B, K, S, T = self.wl.B, self.wl.K, self.wl.S, self.wl.T
        dp, pp, tp = nd.pi
        b_local = B * K / (dp * nd.mb)
        L_pp = math.ceil(L / pp)
        layer_peak = max(2 * d + 6 * d / tp, 2 * d + 2 * d_ff / tp)
        if self.ckpt:
            c = max(1, math.isqrt(L_pp))
            n_ckpt = math.ceil(L_pp / c)
            per_token = n_ckpt * d + c * layer_peak
        else:
            per_token = L_pp * layer_peak
        return sb * b_local * (S + T) * per_token

    def mem_activations(self, nd):
        """memory.py:432-458."""
        return min(nd.mb, nd.pi[1]) * self.act_per_microbatch(nd)

    def mem_act_inference(self, nd):
        """memory.py:460-522."""
        sp = self.suite.specs[nd.model]
        d, d_ff, V, sb = sp.d, sp.d_ff, sp.V, sp.dtype_bytes
        B, K, S, T = self.wl.B, self.wl.K, self.wl.S, self.wl.T
        dp, _, tp = nd.pi
        mb = nd.mb if nd.mb is not None else 1
        b_local = B * K / (dp * mb)
        seq = S + T if _role(nd.tpl) != GEN else S
        per_token = max(2 * d + 6 * d / tp, 2 * d + 2 * d_ff / tp, d + V)
        return sb * b_local * seq * per_token

    def mem_kv(self, nd):
        """memory.py:524-537."""
        sp = self.suite.specs[nd.model]
        B, K, S, T = self.wl.B, self.wl.K, self.wl.S, self.wl.T
        dp, pp, tp = nd.pi
        return 2 * sp.dtype_bytes * (B / dp) * K * (S + T) * (sp.L / pp) * (sp.d / tp)

    def role_extra(self, nd):
        role = _role(nd.tpl)
        if role == TRAIN:
            return self.mem_gradients(nd) + self.mem_activations(nd)
        if role == GEN:
            return self.mem_kv(nd) + self.mem_act_inference(nd)
        return self.mem_act_inference(nd)

    def peak_bytes(self, nd):
        """memory.py:273-288."""
        role = _role(nd.tpl)
        w = self.mem_weights(nd)
        if role == TRAIN:
            return w + self.mem_optimizer(nd) + self.mem_gradients(nd) + self.mem_activations(nd)
        if role == GEN:
            return w + self.mem_kv(nd) + self.mem_act_inference(nd)
        return w + self.mem_act_inference(nd)


def alloc_devices(a):
    return [(r, n, g)
            for r in range(a.origin[0], a.origin[0] + a.extent[0])
            for n in range(a.origin[1], a.origin[1] + a.extent[1])
            for g in range(a.origin[2], a.origin[2] + a.extent[2])]


def device_peaks(nodes, mm):
    """RPEG/model/memory.py:608-841 without fusion groups: the worker-liveness model, or -- for a memory model
    without trainable models -- the co-resident sum model (:706-742).  Returns {device: peak bytes} in first-touch
    order."""
    per_dev = defaultdict(list)
    ops = []
    for nd in nodes:
        if nd.kind != OP:
            continue
        ops.append(nd)
        for a in nd.allocs:
            for dev in set(alloc_devices(a)):
                per_dev[dev].append(nd)
    ws = {id(n): mm.w_shard(n) for n in ops}
    mw = {id(n): mm.mem_weights(n) for n in ops}
    extra = {id(n): mm.role_extra(n) for n in ops}
    peaks = {}
    for dev, here in per_dev.items():
        keys = {(n.model, alloc_key(n.allocs[0])) for n in here}
        overhead = len(keys) * (mm.worker_overhead + mm.act_cache)
        if mm.max_groups > 0 and len(keys) > mm.max_groups:
            peaks[dev] = math.inf
            continue
        if not mm.trainable:
            # every model present keeps its static footprint (the largest shard among its nodes; optimizer state
            # and gradients too where a training node of the model is present, at that node's dp), the nodes
            # share the room for their transients
            info = {}
            for n in here:
                trained = _role(n.tpl) == TRAIN
                if n.model not in info:
                    info[n.model] = [ws[id(n)], trained, n.pi[0]]
                else:
                    rec = info[n.model]
                    rec[0] = max(rec[0], ws[id(n)])
                    if trained:
                        rec[1], rec[2] = True, n.pi[0]
            static = 0
            for m, (w, trained, dp) in info.items():
                sb = mm.suite.specs[m].dtype_bytes
                if trained:
                    static = static + (sb * w + 12 * w / (dp if mm.stage >= 1 else 1) + sb * w / (dp if mm.stage >= 2 else 1))
                else:
                    static = static + sb * w
            transient = 0.0
            for n in here:
                transient = max(transient, extra[id(n)])
            peaks[dev] = overhead + static + transient
            continue
        opt = {}
        train_keys = defaultdict(set)
        for n in here:
            if n.model in mm.trainable and _role(n.tpl) == TRAIN:
                train_keys[n.model].add((n.model, alloc_key(n.allocs[0])))
        serving = {}
        frozen = {}
        for n in here:
            m = n.model
            w = ws[id(n)]
            if m in mm.trainable:
                if _role(n.tpl) == TRAIN:
                    if m not in opt or w > opt[m][0]:
                        opt[m] = (w, n.pi[0])
                else:
                    key = (m, alloc_key(n.allocs[0]))
                    if key not in train_keys[m]:
                        serving[key] = max(serving.get(key, 0), w)
            else:
                frozen[m] = max(frozen.get(m, 0.0), mw[id(n)])
        persistent = 0.0
        for m, (w, dp) in opt.items():
            persistent += 12 * w / (dp if mm.stage >= 1 else 1)
        for key, w in serving.items():
            persistent += mm.suite.specs[key[0]].dtype_bytes * w
        for m, wb in frozen.items():
            persistent += wb
        top = 0.0
        for n in here:
            key = (n.model, alloc_key(n.allocs[0]))
            if key in serving or n.model in frozen:
                c = extra[id(n)]
            else:
                c = mw[id(n)] + extra[id(n)]
            top = max(top, c)
        peaks[dev] = overhead + persistent + top
    return peaks


def mem_worst_violation(nodes, mm):
    """RPEG/model/memory.py:864-887 -> None | (device, peak, cap)."""
    cap = mm.capacity()
    worst, worst_peak = None, 0.0
    for dev, peak in device_peaks(nodes, mm).items():
        if peak > cap and peak > worst_peak:
            worst, worst_peak = dev, peak
    if worst is None:
        return None
    return worst, worst_peak, cap


# --------------------------------------------------------------------------- scheduler
_SUB = re.compile(r"^(.+@\d+):[gi](\d+)$")


def reserved_allocations(nd, preds, succs, by_id, policy=("destination_only", "destination_only")):
    """RPEG/passes/transfer_resources.py:18-148.  policy = (weight, activation)."""
    dest_only = False
    if nd.kind in (COMM, RESHARD) and len(nd.allocs) >= 2:
        is_w = str(nd.label or "").startswith("W_")
        if (policy[0] if is_w else policy[1]) == "destination_only":
            if is_w:
                dest_only = True
            else:
                ends = []
                for ids in (preds[nd.id], succs[nd.id]):
                    op = next((by_id[i] for i in sorted(ids)
                               if i in by_id and by_id[i].kind == OP and by_id[i].pi is not None), None)
                    ends.append(op)
                dest_only = (None not in ends) and int(ends[0].pi[0]) == int(ends[1].pi[0])
    sel = nd.allocs[-1:] if dest_only else nd.allocs
    out, seen = [], set()
    for a in sel:
        if alloc_key(a) not in seen:
            seen.add(alloc_key(a))
            out.append(a)
    return tuple(out)


def node_ranks(nodes, edges, dur):
    """RPEG/schedule/scheduler.py:28-100 + chain inheritance :367-378."""
    indeg = {n.id: 0 for n in nodes}
    adj = defaultdict(list)
    for a, b in edges:
        indeg[b.id] += 1
        adj[a.id].append(b)
    q = deque(n for n in nodes if indeg[n.id] == 0)
    topo = []
    while q:
        u = q.popleft()
        for w in adj[u.id]:
            indeg[w.id] -= 1
            if indeg[w.id] == 0:
                q.append(w)
        topo.append(u)
    rank = {}
    for v in reversed(topo):
        rank[v.id] = dur[v.id] + max((rank[w.id] for w in adj[v.id]), default=0)
    groups = defaultdict(list)
    for v in nodes:
        mt = _SUB.match(v.id)
        if mt:
            groups[mt.group(1)].append(v)
    for members in groups.values():
        top = max(rank[v.id] for v in members)
        for v in members:
            rank[v.id] = top
    return rank


def schedule(nodes, edges, cost, space, policy=("destination_only", "destination_only")):
    """RPEG/schedule/scheduler.py:270-552 without fusion groups.
    Returns (start, finish, order): dicts keyed by node id, and the dispatch order."""
    avail = {(r, n, g): 0.0 for r in range(space.R) for n in range(space.N) for g in range(space.G)}
    indeg = {n.id: 0 for n in nodes}
    adj = defaultdict(list)
    preds = {n.id: set() for n in nodes}
    succs = {n.id: set() for n in nodes}
    for a, b in edges:
        indeg[b.id] += 1
        adj[a.id].append(b)
        preds[b.id].add(a.id)
        succs[a.id].add(b.id)
    by_id = {n.id: n for n in nodes}
    blocked = {}
    for n in nodes:
        devs = set()
        for a in reserved_allocations(n, preds, succs, by_id, policy):
            devs.update(alloc_devices(a))
        blocked[n.id] = devs
    dur = {n.id: cost.time(n) for n in nodes}
    rank = node_ranks(nodes, edges, dur)
    tpl_ids = sorted({n.tpl.id for n in nodes if n.kind == OP})
    tpl_pos = {t: i for i, t in enumerate(tpl_ids)}
    tidx = {n.id: (tpl_pos[n.tpl.id] if n.kind == OP else len(tpl_ids)) for n in nodes}
    prio = {n.id: (1 if n.kind == OP else 0) for n in nodes}
    pf = defaultdict(list)

    def est(n):
        return max(max(pf[n.id]), max(avail[dv] for dv in blocked[n.id]))

    heap, tie = [], 0
    ready = set()
    start, finish, order = {}, {}, []
    for n in nodes:
        if indeg[n.id] == 0:
            pf[n.id].append(0.0)
            heapq.heappush(heap, (est(n), prio[n.id], tidx[n.id], -rank[n.id], tie, n.id))
            tie += 1
            ready.add(n.id)
    while heap:
        e_h, cp, ti, nr, _, nid = heapq.heappop(heap)
        if nid not in ready:
            continue
        n = by_id[nid]
        e_now = est(n)
        if e_now > e_h:
            heapq.heappush(heap, (e_now, cp, ti, nr, tie, nid))
            tie += 1
            continue
        ready.discard(nid)
        start[nid] = e_now
        finish[nid] = e_now + dur[nid]
        order.append(nid)
        for dv in blocked[nid]:
            avail[dv] = finish[nid]
        for w in adj[nid]:
            indeg[w.id] -= 1
            pf[w.id].append(finish[nid])
            if indeg[w.id] == 0:
                heapq.heappush(heap, (est(w), prio[w.id], tidx[w.id], -rank[w.id], tie, w.id))
                tie += 1
                ready.add(w.id)
    if len(start) != len(nodes):
        raise ValueError("cycle in executable graph")
    return start, finish, order


def reserved_by_node(nodes, edges, policy=("destination_only", "destination_only")):
    """node id -> tuple of the allocations the scheduler reserves for it (scheduler.py:334-343)."""
    preds = {n.id: set() for n in nodes}
    succs = {n.id: set() for n in nodes}
    for a, b in edges:
        preds[b.id].add(a.id)
        succs[a.id].add(b.id)
    by_id = {n.id: n for n in nodes}
    return {n.id: reserved_allocations(n, preds, succs, by_id, policy) for n in nodes}


def utilization(start, finish, order, reserved):
    """Trace.utilization (RPEG/schedule/trace.py:53-101): per device the merged busy intervals of the nodes
    that reserve it, divided by the makespan, averaged over the devices any node reserves.  `order` is the
    dispatch order (the insertion order of Trace.start), which fixes the order of the devices in the
    reference's dict and hence of its float sum."""
    ms = max(finish.values())
    if ms <= 0:
        return 0.0
    intervals = {}
    for nid in order:
        for a in reserved[nid]:
            for dv in alloc_devices(a):
                intervals.setdefault(dv, []).append((start[nid], finish[nid]))
    if not intervals:
        return 0.0
    total = 0.0
    for spans in intervals.values():
        merged = 0.0
        cs = ce = None
        for s, e in sorted(spans):
            if ce is None or s > ce:
                if ce is not None:
                    merged += ce - cs
                cs, ce = s, e
            else:
                ce = max(ce, e)
        if ce is not None:
            merged += ce - cs
        total += merged / ms    # the builtin sum of this interpreter (3.10) is a plain left fold
    return total / len(intervals)


def n_active(nodes):
    """Trace.n_active (trace.py:103-118): devices inside any allocation of any node."""
    devices = set()
    for n in nodes:
        for a in n.allocs:
            devices.update(alloc_devices(a))
    return len(devices)


# --------------------------------------------------------------------------- evaluate
def make_mem_model(rpeg, suite, workload, hw, policy):
    return MemModel(
        hw, suite, workload, trainable=rpeg.trainable,
        eps_rt=policy.runtime_overhead_fraction, optimizer_stage=policy.optimizer_stage,
        worker_overhead_bytes=policy.worker_overhead_bytes,
        semantic_activation_cache_bytes=policy.semantic_activation_cache_bytes,
        max_worker_groups_per_gpu=policy.max_worker_groups_per_gpu,
        activation_checkpointing=policy.activation_checkpointing)


class DefaultPolicy:
    """MemoryPolicy defaults (RPEG/model/memory.py:138-148)."""
    optimizer_stage = 2
    activation_checkpointing = True
    runtime_overhead_fraction = 0.0
    worker_overhead_bytes = 0.0
    semantic_activation_cache_bytes = 0.0
    max_worker_groups_per_gpu = 0


def evaluate_plan(rpeg, plan, space, suite, workload, hw, K_eval, policy=None, check_stale=True,
                  want_trace=False, transfer_policy=("destination_only", "destination_only")):
    """One evaluation as `evaluate_cached` computes it on a miss
    (RPEG/search/evaluate.py:235-290, 364-403).  With check_stale=False it is
    `_eval_worker` (:406-442), which omits the stale-layout gate.

    Returns a dict: makespan, raw (K_eval*B*K*(S+T)/makespan), peak (worst
    violating device peak, or the max device peak when feasible), cap,
    feasible, stale_ok, score.  transfer_policy = (weight, activation) is what the scheduler is given
    as `transfer_resource_policy` (evaluate.py:280-287)."""
    policy = policy or DefaultPolicy()
    nodes, edges = lower(rpeg, plan, suite, K_eval, workload)
    cost = CostModel(hw, suite, workload, policy.optimizer_stage, policy.activation_checkpointing)
    start, finish, order = schedule(nodes, edges, cost, space, transfer_policy)
    makespan = max(finish.values())
    raw = K_eval * (workload.B * workload.K * (workload.S + workload.T)) / makespan
    mm = make_mem_model(rpeg, suite, workload, hw, policy)
    peaks = device_peaks(nodes, mm)
    cap = mm.capacity()
    max_peak = max(peaks.values())
    stale_ok = stale_publication_layout_valid(rpeg, plan)
    feasible = not (max_peak > cap)
    if feasible:
        score = raw
    else:
        over = max(0.0, max_peak / cap - 1.0)
        score = raw * max(math.exp(-OOM_BETA * over), 1e-12)
    if check_stale and not stale_ok:
        score, feasible = 0.0, False
    out = dict(makespan=makespan, raw=raw, peak=max_peak, cap=cap, feasible=feasible,
               stale_ok=stale_ok, score=score)
    if want_trace:
        out.update(nodes=nodes, edges=edges, start=start, finish=finish, order=order)
    return out
