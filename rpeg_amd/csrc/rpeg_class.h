// rpeg_class.h - lowering classes: the plan-dependent DAG topology, factored out of the plans.
//
// The reference lowers every plan into its own executable graph (RPEG/passes/lower.py:330-851).
// The topology of that graph depends on the plan only through a handful of predicates on pairs of
// template vertices (allocations equal / overlapping / disjoint, equal (dp,pp,tp), equal dp), the
// staleness budgets and the generation-split variant.  Those predicates are packed into a 64-bit
// SIGNATURE per plan; all plans with one signature share one CLASS: node list, edge lists, duration
// slots, tie-break keys and device-reservation masks, in exactly the reference's insertion order.
// A class is lowered once (rpeg_lower.h, host) and then drives the numeric kernel for every plan
// that maps to it.
#ifndef RPEG_CLASS_H
#define RPEG_CLASS_H

#include "rpeg_core.h"

namespace rpeg {

// ------------------------------------------------------------------------------------- signature
// bits 0-1 structure, 2-4 split, 5-6 tau slot 0, 7-8 tau slot 1, then 4 bits per relation pair:
// relation (0 equal, 1 different but not known/needed to be disjoint, 2 disjoint) and pi-equal.
// Equality of dp across an activation transfer only changes which endpoints the transfer reserves
// (transfer_resources.py:30-62), not the graph, so it stays a per-plan bit (dp_differs) instead of
// splitting classes.
constexpr int SIG_REL_SHIFT = 9;
constexpr uint64_t SIG_INVALID = ~0ull;

// `a[v]` yields the plan fields of vertex v (an array of VPlan, or an accessor returning VPlan by value).
template <class PLANS>
RPEG_HD uint64_t plan_signature(const rpeg_problem_t& P, int s, int split, int tau0, int tau1, const PLANS& a) {
  const rpeg_struct_t& st = P.st[s];
  uint64_t sig = (uint64_t)s | ((uint64_t)split << 2) | ((uint64_t)tau0 << 5) | ((uint64_t)tau1 << 7);
  for (int r = 0; r < st.n_rel; ++r) {
    const VPlan& x = a[st.rel[r].u];
    const VPlan& y = a[st.rel[r].v];
    const int flags = st.rel[r].flags;
    unsigned rel = alloc_equal(x, y) ? 0u : (alloc_disjoint(x, y) ? 2u : 1u);
    if (rel == 2u && !(flags & RPEG_NEED_DISJ)) rel = 1u;
    unsigned pi = ((flags & RPEG_NEED_PI) && rel == 0u && x.dp == y.dp && x.pp == y.pp && x.tp == y.tp) ? 1u : 0u;
    sig |= (uint64_t)(rel | (pi << 2)) << (SIG_REL_SHIFT + 4 * r);
  }
  return sig;
}

// ------------------------------------------------------------------------------------- class blob
enum SlotType : uint8_t {
  SLOT_OP_UNSPLIT = 0,  // a = vertex
  SLOT_OP_SUB = 1,      // a = vertex, q = phase
  SLOT_COMM_DATA = 2,   // a = data edge, q = phase or 0xFF for the full container
  SLOT_COMM_PUB = 3,    // a = publication edge
  SLOT_RESHARD = 4      // a = vertex whose allocation hosts the reshard, b = model
};

struct SlotDesc { uint8_t type, a, b, q; };

struct NodeRec {
  uint16_t succ_begin;  // into the class successor array, in the reference's adjacency order
  uint8_t n_succ;
  uint8_t slot;         // duration slot
  uint8_t ptkey;        // comm_prio * 8 + topo_idx: second and third heap-key fields (scheduler.py:427)
  uint8_t blocked;      // bit set of vertices whose allocations the node always reserves
  uint8_t indeg;
  uint8_t cond;         // activation transfer src->dst: 1 + src*8 + dst; the source allocation is reserved
                        // too when dp differs across the transfer.  0 otherwise.
};

// dpne: bit (u*8 + v) set when dp of vertex u differs from dp of vertex v (PlanMasks::dpne)
RPEG_HD unsigned blocked_mask(const NodeRec& r, uint64_t dpne) {
  unsigned b = r.blocked;
  if (r.cond) {
    const unsigned c = r.cond - 1u;
    b |= (unsigned)((dpne >> c) & 1ull) << (c >> 3);
  }
  return b;
}

struct GroupRec { uint16_t begin, count; };  // sub-node chains that share the chain's top rank

struct ClassHdr {
  uint32_t n_nodes, n_slots, n_succ, n_init, n_groups, n_gmembers;
  uint32_t off_node, off_succ, off_init, off_topo, off_slot, off_group, off_gmember;  // byte offsets in the blob
  uint32_t off_pbeg, off_pred;       // predecessor lists in edge order: pred[pbeg[v] .. pbeg[v+1])
  uint32_t off_umap;                 // per slot: its index in the structure's slot universe (slot_universe)
  uint32_t bytes;
  uint32_t structure, split, error;  // error != 0: the reference would raise for this class
  uint32_t id;                       // index of the class in the tables of the engine that holds it (0 elsewhere)
  uint8_t vorder[8];                 // vertices by first appearance among the lowered operator nodes
};

struct ClassView {
  const ClassHdr* h;
  const NodeRec* node;
  const uint16_t* succ;
  const uint16_t* init;
  const uint16_t* topo;
  const SlotDesc* slot;
  const GroupRec* group;
  const uint16_t* gmember;
  const uint16_t* pbeg;
  const uint16_t* pred;
  const uint8_t* umap;
};

RPEG_HD ClassView class_view(const uint8_t* blob) {
  ClassView v;
  v.h = (const ClassHdr*)blob;
  v.node = (const NodeRec*)(blob + v.h->off_node);
  v.succ = (const uint16_t*)(blob + v.h->off_succ);
  v.init = (const uint16_t*)(blob + v.h->off_init);
  v.topo = (const uint16_t*)(blob + v.h->off_topo);
  v.slot = (const SlotDesc*)(blob + v.h->off_slot);
  v.group = (const GroupRec*)(blob + v.h->off_group);
  v.gmember = (const uint16_t*)(blob + v.h->off_gmember);
  v.pbeg = (const uint16_t*)(blob + v.h->off_pbeg);
  v.pred = (const uint16_t*)(blob + v.h->off_pred);
  v.umap = blob + v.h->off_umap;
  return v;
}

// duration of one slot for one plan (NodeCostModel.time of every node that uses the slot)
RPEG_HD double slot_duration(const rpeg_problem_t& P, const rpeg_struct_t& st, int split, const SlotDesc& sd,
                             const VPlan* a, bool* zero_div) {
  switch (sd.type) {
    case SLOT_OP_UNSPLIT:
      return op_time(P, st.vertex[sd.a], st.vertex[sd.a].unsplit, a[sd.a], zero_div);
    case SLOT_OP_SUB:
      return op_time(P, st.vertex[sd.a], st.vertex[sd.a].sub[split][sd.q], a[sd.a], zero_div);
    case SLOT_COMM_DATA: {
      const rpeg_edge_t& e = st.edge[sd.a];
      int64_t payload = sd.q == 0xFF ? e.full_bytes : e.sub_bytes[split][sd.q];
      return comm_time(P, a[e.src], a[e.dst], payload, e.is_weight != 0);
    }
    case SLOT_COMM_PUB: {
      const rpeg_pub_t& p = st.pub[sd.a];
      return comm_time(P, a[p.src], a[p.dst], pub_payload(P, a[p.src], a[p.dst], p.model), true);
    }
    default:
      return reshard_time(P, a[sd.a], sd.b);
  }
}

// ------------------------------------------------------------------------------------- slot universe
// Every duration slot a class of structure `st` can have, whatever the plan: the operator of every vertex unsplit and
// by quantile phase, the transfer of every data edge whole and (generation -> inference edges) by phase, every
// publication transfer, and the reshards lowering can place (between the vertices of a same-model pair, at the
// source of a publication).  Durations depend on the plan only through the plan fields, so a launch of its own can
// evaluate the whole universe for every plan before the classes of a batch are even known; a class's slot s is entry
// ClassView::umap[s].  Entries by phase carry the phase in q: for a plan of split variant j only those with
// q < P.n_phase[j] exist.  At most RPEG_MAX_UNIVERSE entries; returns their number.
constexpr int RPEG_MAX_UNIVERSE = 96;
RPEG_HD int slot_universe(const rpeg_problem_t& P, const rpeg_struct_t& st, SlotDesc* out) {
  int n = 0, max_ph = 0;
  for (int j = 1; j < P.n_split; ++j) max_ph = P.n_phase[j] > max_ph ? P.n_phase[j] : max_ph;
  auto put = [&](uint8_t type, int a, int b, int q) {
    for (int i = 0; i < n; ++i)
      if (out[i].type == type && out[i].a == a && out[i].b == b && out[i].q == q) return;
    if (n < RPEG_MAX_UNIVERSE) out[n] = SlotDesc{type, (uint8_t)a, (uint8_t)b, (uint8_t)q};
    ++n;
  };
  for (int v = 0; v < st.n_vertex; ++v) put(SLOT_OP_UNSPLIT, v, 0, 0);
  for (int v = 0; v < st.n_vertex; ++v)
    if (st.vertex[v].role != RPEG_ROLE_TRAIN)
      for (int q = 0; q < max_ph; ++q) put(SLOT_OP_SUB, v, 0, q);
  for (int e = 0; e < st.n_edge; ++e) put(SLOT_COMM_DATA, e, 0, 0xFF);
  for (int e = 0; e < st.n_edge; ++e)
    if (st.edge[e].gen_inf)
      for (int q = 0; q < max_ph; ++q) put(SLOT_COMM_DATA, e, 0, q);
  for (int p = 0; p < st.n_pub; ++p) put(SLOT_COMM_PUB, p, 0, 0);
  for (int p = 0; p < st.n_pair; ++p) put(SLOT_RESHARD, st.pair[p].u, st.pair[p].model, 0);
  for (int p = 0; p < st.n_pub; ++p) put(SLOT_RESHARD, st.pub[p].src, st.pub[p].model, 0);
  return n;
}
RPEG_HD bool slot_in_split(const rpeg_problem_t& P, int split, const SlotDesc& sd) {
  const int nph = split > 0 ? P.n_phase[split] : 0;
  if (sd.type == SLOT_OP_SUB) return sd.q < nph;
  if (sd.type == SLOT_COMM_DATA && sd.q != 0xFF) return sd.q < nph;
  return true;
}

// The order in which the template vertices first appear among a plan's lowered operator nodes (ClassHdr::vorder),
// from the plan itself: template order, except that an inference vertex whose node is split into quantile phases
// (its generation producer is split -- some inference consumer of it sits on disjoint devices -- and so is it:
// lower.py:425-431, 528-558) is taken out and appended again, in the order of the data edges that split them.
template <class PLANS>
RPEG_HD void plan_vorder(const rpeg_problem_t& P, const rpeg_struct_t& st, int split, const PLANS& a, uint8_t* order) {
  const int nv = st.n_vertex, nph = split > 0 ? P.n_phase[split] : 0;
  unsigned gen_split = 0, moved = 0;
  int n_tail = 0;
  uint8_t tail[RPEG_MAX_V];
  if (nph > 0) {
    for (int e = 0; e < st.n_edge; ++e)
      if (st.edge[e].gen_inf && alloc_disjoint(a[st.edge[e].src], a[st.edge[e].dst])) gen_split |= 1u << st.edge[e].src;
    for (int e = 0; e < st.n_edge; ++e) {
      const int u = st.edge[e].src, v = st.edge[e].dst;
      if (!((gen_split >> u) & 1u) || st.vertex[v].role != RPEG_ROLE_INF || ((moved >> v) & 1u)) continue;
      if (alloc_disjoint(a[u], a[v])) { moved |= 1u << v; tail[n_tail++] = (uint8_t)v; }
    }
  }
  int c = 0;
  for (int v = 0; v < nv; ++v)
    if (!((moved >> v) & 1u)) order[c++] = (uint8_t)v;
  for (int j = 0; j < n_tail; ++j) order[c++] = tail[j];
}

// ------------------------------------------------------------------------------------- scheduler
// List scheduler of RPEG/schedule/scheduler.py:270-552, restated without a heap and without
// per-device state:
//  * Heap entries are (est, comm_prio, topo_idx, -rank, tie).  A node has at most one live entry,
//    and `tie` grows with every push, so a list kept in push order with "first strictly smaller
//    (est, ptkey, -rank) wins" pops exactly the heap's minimum.  A stale pop (the recomputed est is
//    larger) moves the node to the list's end with the new est, as the re-push with a fresh tie does.
//  * avail[d] only ever grows, and every node reserves the union of at most two vertex allocations,
//    so max(avail[d] for d in blocked(v)) equals the maximum of last_fin[x] over the vertices x in
//    blocked(v), where last_fin[x] is the largest finish time of any scheduled node whose reserved
//    set intersects the allocation of x.  ovl[x] is the bit set of vertices intersecting x.
//
// MEM provides time(i), rank(i) (double&), indeg(i) (uint8_t&), dur(slot) (double), the ready list
// rd_node(j) (uint16_t&) of capacity ready_cap, and on_schedule(node, start, finish).
template <class MEM>
RPEG_HD double list_schedule(const ClassView& c, MEM& mem, const uint8_t* ovl, uint64_t dpne, int nv, int ready_cap,
                             bool* error) {
  const int n = (int)c.h->n_nodes;
  // ranks: reverse topological pass, then chain inheritance (scheduler.py:71-100, 367-378)
  for (int i = n - 1; i >= 0; --i) {
    const int v = c.topo[i];
    const NodeRec nr = c.node[v];
    double best = 0.0;
    for (int j = 0; j < nr.n_succ; ++j) {
      double r = mem.rank(c.succ[nr.succ_begin + j]);
      if (r > best) best = r;
    }
    mem.rank(v) = mem.dur(nr.slot) + best;
  }
  for (unsigned g = 0; g < c.h->n_groups; ++g) {
    const GroupRec gr = c.group[g];
    double top = mem.rank(c.gmember[gr.begin]);
    for (int j = 1; j < gr.count; ++j) {
      double r = mem.rank(c.gmember[gr.begin + j]);
      if (r > top) top = r;
    }
    for (int j = 0; j < gr.count; ++j) mem.rank(c.gmember[gr.begin + j]) = top;
  }
  for (int v = 0; v < n; ++v) {
    mem.indeg(v) = c.node[v].indeg;
    mem.time(v) = 0.0;
  }
  double last_fin[RPEG_MAX_V];
  for (int x = 0; x < RPEG_MAX_V; ++x) last_fin[x] = 0.0;
  int n_ready = 0;
  for (unsigned i = 0; i < c.h->n_init; ++i) {
    if (n_ready >= ready_cap) { *error = true; return 0.0; }
    mem.rd_node(n_ready++) = c.init[i];
  }
  double makespan = 0.0;
  int done = 0;
  // every iteration either schedules a node or raises one node's key; the bound guards a broken class
  for (long guard = 0; done < n && guard < (long)n * n + 64; ++guard) {
    if (n_ready == 0) { *error = true; return 0.0; }  // cycle (scheduler.py:548-550)
    int bj = 0;
    int bv = mem.rd_node(0);
    double bt = mem.time(bv);
    for (int j = 1; j < n_ready; ++j) {
      const int v = mem.rd_node(j);
      const double t = mem.time(v);
      bool better = t < bt;
      if (t == bt) {
        const int ka = c.node[v].ptkey, kb = c.node[bv].ptkey;
        better = ka < kb || (ka == kb && mem.rank(v) > mem.rank(bv));
      }
      if (better) { bj = j; bv = v; bt = t; }
    }
    const NodeRec nr = c.node[bv];
    const unsigned blocked = blocked_mask(nr, dpne);
    double dev = 0.0;
    for (int x = 0; x < nv; ++x)
      if ((blocked >> x) & 1) dev = dmax(dev, last_fin[x]);
    const double est = dmax(bt, dev);
    for (int j = bj; j + 1 < n_ready; ++j) mem.rd_node(j) = mem.rd_node(j + 1);
    if (est > bt) {  // stale key: re-push with the corrected est and a fresh tie
      mem.time(bv) = est;
      mem.rd_node(n_ready - 1) = (uint16_t)bv;
      continue;
    }
    --n_ready;
    const double fin = est + mem.dur(nr.slot);
    mem.on_schedule(bv, est, fin);
    if (fin > makespan) makespan = fin;
    ++done;
    unsigned touched = 0;
    for (int x = 0; x < nv; ++x)
      if ((blocked >> x) & 1) touched |= ovl[x];
    for (int x = 0; x < nv; ++x)
      if ((touched >> x) & 1) last_fin[x] = dmax(last_fin[x], fin);
    for (int j = 0; j < nr.n_succ; ++j) {
      const int w = c.succ[nr.succ_begin + j];
      double t = mem.time(w);
      if (fin > t) t = fin;
      const uint8_t left = (uint8_t)(mem.indeg(w) - 1);
      mem.indeg(w) = left;
      if (left == 0) {
        const unsigned blk = blocked_mask(c.node[w], dpne);
        double d2 = 0.0;
        for (int x = 0; x < nv; ++x)
          if ((blk >> x) & 1) d2 = dmax(d2, last_fin[x]);
        t = dmax(t, d2);
        if (n_ready >= ready_cap) { *error = true; return 0.0; }
        mem.rd_node(n_ready++) = (uint16_t)w;
      }
      mem.time(w) = t;
    }
  }
  if (done != n) *error = true;
  return makespan;
}

// Critical-chain mass per template vertex (RPEG/search/moves.py:590-642): from the first node of
// largest finish time follow, at every node, the first predecessor (in edge order) of largest finish
// time; a vertex's mass is the sum of finish - start over its operator nodes on that chain, added from
// the sink backwards.  fin(i) / start(i) give the times of node i.
template <class Fin, class Start>
RPEG_HD void critical_mass(const ClassView& c, Fin fin, Start start, double (&mass)[RPEG_MAX_V]) {
  for (int x = 0; x < RPEG_MAX_V; ++x) mass[x] = 0.0;
  const int n = (int)c.h->n_nodes;
  int cur = 0;
  double best = fin(0);
  for (int i = 1; i < n; ++i) {
    const double f = fin(i);
    if (f > best) { best = f; cur = i; }
  }
  for (int hops = 0; hops <= n; ++hops) {   // a chain visits a node at most once
    const SlotDesc sd = c.slot[c.node[cur].slot];
    if (sd.type <= SLOT_OP_SUB) {
      const double d = best - start(cur);
      for (int x = 0; x < RPEG_MAX_V; ++x)
        if (x == (int)sd.a) mass[x] += d;
    }
    const int pb = c.pbeg[cur], pe = c.pbeg[cur + 1];
    if (pb == pe) break;
    int nx = c.pred[pb];
    double bf = fin(nx);
    for (int j = pb + 1; j < pe; ++j) {
      const int q = c.pred[j];
      const double f = fin(q);
      if (f > bf) { bf = f; nx = q; }
    }
    cur = nx;
    best = bf;
  }
}

}  // namespace rpeg
#endif
