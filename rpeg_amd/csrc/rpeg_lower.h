// rpeg_lower.h - host-side lowering of one class signature into a class blob.
//
// Follows RPEG/passes/unroll.py:85-152 and RPEG/passes/lower.py:330-851 statement by statement on
// vertex indices instead of objects, answering every plan predicate from the signature bits
// (rpeg_class.h).  Node order is the insertion order of the reference's `nodes` dict (with the
// pop-and-reappend of split inference vertices), edge order the append order of its `edges` list:
// both decide scheduler ties.  Also derives what schedule() derives from the graph alone:
// reserved allocations (RPEG/passes/transfer_resources.py:18-148), tie-break keys and chain
// groups (RPEG/schedule/scheduler.py:367-397).
#ifndef RPEG_LOWER_H
#define RPEG_LOWER_H

#include <cstring>
#include <map>
#include <set>
#include <stdexcept>
#include <string>
#include <tuple>
#include <utility>
#include <vector>

#include "rpeg_class.h"

namespace rpeg {

struct SigView {
  const rpeg_struct_t* st;
  uint64_t sig;
  int structure() const { return (int)(sig & 3); }
  int split() const { return (int)((sig >> 2) & 7); }
  int tau(int slot) const { return slot < 0 ? 0 : (int)((sig >> (5 + 2 * slot)) & 3); }
  int rel_index(int u, int v) const {
    for (int r = 0; r < st->n_rel; ++r)
      if ((st->rel[r].u == u && st->rel[r].v == v) || (st->rel[r].u == v && st->rel[r].v == u)) return r;
    throw std::logic_error("lowering asked for a vertex pair outside the relation table");
  }
  unsigned bits(int u, int v) const { return (unsigned)((sig >> (SIG_REL_SHIFT + 4 * rel_index(u, v))) & 15); }
  bool eq(int u, int v) const { return u == v || (bits(u, v) & 3) == 0; }
  bool disjoint(int u, int v) const {
    if (u == v) return false;
    if (!(st->rel[rel_index(u, v)].flags & RPEG_NEED_DISJ))
      throw std::logic_error("disjointness queried for a pair that does not record it");
    return (bits(u, v) & 3) == 2;
  }
  bool pi_eq(int u, int v) const {
    if (u == v) return true;
    if (!(st->rel[rel_index(u, v)].flags & RPEG_NEED_PI)) throw std::logic_error("pi equality not recorded");
    return (bits(u, v) & 4) != 0;  // recorded only when the allocations are equal
  }
};

struct LoweredNode {
  int kind;     // 0 OP, 1 COMM, 2 RESHARD
  int vertex;   // OP: template vertex
  int step;     // OP: unroll step k
  int sub;      // OP: -1 unsplit, else phase index
  int a0, a1;   // COMM/RESHARD: source / destination vertex (allocations)
  int weight;   // COMM/RESHARD: label starts with "W_"
  int model;    // RESHARD: model
  int slot;
  bool alive;
};

struct LoweredClass {
  std::vector<LoweredNode> nodes;          // alive nodes, reference order
  std::vector<std::pair<int, int>> edges;  // indices into nodes, reference order
  std::vector<uint8_t> blob;
};

inline LoweredClass lower_class(const rpeg_problem_t& P, uint64_t sig_bits) {
  SigView sg{&P.st[sig_bits & 3], sig_bits};
  const rpeg_struct_t& st = *sg.st;
  const int nv = st.n_vertex, K = P.K_eval, split = sg.split();
  const int nph = split > 0 ? P.n_phase[split] : 0;

  std::vector<LoweredNode> nodes;
  std::vector<std::pair<int, int>> edges;
  std::set<std::pair<int, int>> seen;
  std::vector<SlotDesc> slots;
  std::map<std::tuple<int, int, int, int>, int> slot_of;
  auto slot = [&](SlotType t, int a, int b, int q) {
    auto key = std::make_tuple((int)t, a, b, q);
    auto it = slot_of.find(key);
    if (it != slot_of.end()) return it->second;
    if (slots.size() >= 255) throw std::runtime_error("too many duration slots");
    slots.push_back(SlotDesc{(uint8_t)t, (uint8_t)a, (uint8_t)b, (uint8_t)q});
    return slot_of[key] = (int)slots.size() - 1;
  };
  auto add_edge = [&](int a, int b) {
    if (seen.insert({a, b}).second) edges.push_back({a, b});
  };
  auto add_node = [&](const LoweredNode& n) { nodes.push_back(n); return (int)nodes.size() - 1; };

  // per (vertex, step): the unsplit node, generation sub-nodes, inference sub-nodes
  std::vector<std::vector<int>> base(nv, std::vector<int>(K, -1));
  std::vector<std::vector<std::vector<int>>> gsub(nv, std::vector<std::vector<int>>(K)), isub = gsub;

  // which generation vertices split: quantile phases exist and some inference consumer is disjoint
  std::vector<bool> gen_split(nv, false);
  if (nph > 0)
    for (int e = 0; e < st.n_edge; ++e) {
      const rpeg_edge_t& ed = st.edge[e];
      if (st.vertex[ed.src].role == RPEG_ROLE_GEN && st.vertex[ed.dst].role == RPEG_ROLE_INF &&
          sg.disjoint(ed.src, ed.dst))
        gen_split[ed.src] = true;
    }

  // 1) operator nodes, step-major in template order (unroll.py:103-110, lower.py:433-474)
  for (int k = 0; k < K; ++k)
    for (int v = 0; v < nv; ++v) {
      if (nph > 0 && st.vertex[v].role == RPEG_ROLE_GEN && gen_split[v]) {
        for (int q = 0; q < nph; ++q)
          gsub[v][k].push_back(add_node({0, v, k, q, v, v, 0, st.vertex[v].model, slot(SLOT_OP_SUB, v, 0, q), true}));
        for (int q = 1; q < nph; ++q) add_edge(gsub[v][k][q - 1], gsub[v][k][q]);
      } else {
        base[v][k] = add_node({0, v, k, -1, v, v, 0, st.vertex[v].model, slot(SLOT_OP_UNSPLIT, v, 0, 0), true});
      }
    }

  // 2) data edges, generation->inference edges of split generators first (lower.py:476-597)
  auto edge_or_comm = [&](int a, int b, int e, int q) {
    const int va = nodes[a].vertex, vb = nodes[b].vertex;
    if (sg.eq(va, vb)) { add_edge(a, b); return; }
    int c = add_node({1, -1, nodes[a].step, -1, va, vb, st.edge[e].is_weight, -1,
                      slot(SLOT_COMM_DATA, e, 0, q < 0 ? 0xFF : q), true});
    add_edge(a, c);
    add_edge(c, b);
  };
  std::vector<std::pair<int, int>> pass1, pass2;  // (step, edge)
  for (int k = 0; k < K; ++k)
    for (int e = 0; e < st.n_edge; ++e) {
      const rpeg_edge_t& ed = st.edge[e];
      if (!gsub[ed.src][k].empty() && st.vertex[ed.dst].role == RPEG_ROLE_INF) pass1.push_back({k, e});
      else pass2.push_back({k, e});
    }
  pass1.insert(pass1.end(), pass2.begin(), pass2.end());
  for (auto& ke : pass1) {
    const int k = ke.first, e = ke.second;
    const rpeg_edge_t& ed = st.edge[e];
    const int u = ed.src, v = ed.dst;
    const bool src_gen_split = !gsub[u][k].empty();
    if (src_gen_split && st.vertex[v].role == RPEG_ROLE_INF) {
      if (sg.disjoint(u, v)) {
        if (isub[v][k].empty()) {
          if (base[v][k] >= 0) { nodes[base[v][k]].alive = false; base[v][k] = -1; }
          for (int q = 0; q < nph; ++q)
            isub[v][k].push_back(add_node({0, v, k, q, v, v, 0, st.vertex[v].model, slot(SLOT_OP_SUB, v, 0, q), true}));
          for (int q = 1; q < nph; ++q) add_edge(isub[v][k][q - 1], isub[v][k][q]);
        }
        for (int q = 0; q < nph; ++q) edge_or_comm(gsub[u][k][q], isub[v][k][q], e, q);
      } else {
        edge_or_comm(gsub[u][k].back(), base[v][k], e, -1);
      }
    } else if (src_gen_split) {
      edge_or_comm(gsub[u][k].back(), base[v][k], e, -1);
    } else if (!isub[u][k].empty()) {
      if (base[v][k] < 0) throw std::runtime_error("destination node of a split inference edge not found");
      edge_or_comm(isub[u][k].back(), base[v][k], e, -1);
    } else {
      if (base[u][k] < 0 || base[v][k] < 0) throw std::runtime_error("edge endpoint missing");
      edge_or_comm(base[u][k], base[v][k], e, -1);
    }
  }

  // 3) within-step weight reshards between consecutive vertices of one trainable model (lower.py:626-681)
  auto last_of = [&](int v, int k) {
    if (!gsub[v][k].empty()) return gsub[v][k].back();
    if (!isub[v][k].empty()) return isub[v][k].back();
    return base[v][k];
  };
  auto first_of = [&](int v, int k) {
    if (!gsub[v][k].empty()) return gsub[v][k].front();
    if (!isub[v][k].empty()) return isub[v][k].front();
    return base[v][k];
  };
  std::vector<bool> resharded(nv, false);
  auto make_reshard = [&](int a, int b, int model) {
    return add_node({2, -1, nodes[a].step, -1, nodes[a].vertex, nodes[b].vertex, 1, model,
                     slot(SLOT_RESHARD, nodes[a].vertex, model, 0), true});
  };
  for (int p = 0; p < st.n_pair; ++p) {
    const rpeg_pair_t& pr = st.pair[p];
    if (sg.tau(pr.tau_slot) > 0 && sg.disjoint(pr.u, pr.v)) continue;  // shadow pair
    if (pr.reach && !sg.eq(pr.u, pr.v)) continue;
    for (int k = 0; k < K; ++k) {
      const int a = last_of(pr.u, k), b = first_of(pr.v, k);
      const bool same = sg.eq(pr.u, pr.v);
      if (same && sg.pi_eq(pr.u, pr.v)) continue;
      if (!same) { add_edge(a, b); continue; }
      int r = make_reshard(a, b, pr.model);
      add_edge(a, r);
      add_edge(r, b);
      resharded[pr.v] = true;
    }
  }

  // 4a) publication edges (unroll.py:121-135, lower.py:683-728)
  for (int k = 1; k < K; ++k)
    for (int p = 0; p < st.n_pub; ++p) {
      const rpeg_pub_t& pb = st.pub[p];
      const int t = sg.tau(pb.tau_slot);
      if (k <= t) continue;
      const int ks = k - (t + 1) > 0 ? k - (t + 1) : 0;
      const int a = base[pb.src][ks];
      const int b = first_of(pb.dst, k);
      if (a < 0 || b < 0) throw std::runtime_error("publication endpoint missing");
      if (resharded[pb.dst]) continue;
      const bool same = sg.eq(pb.src, pb.dst);
      if (same && sg.pi_eq(pb.src, pb.dst)) { add_edge(a, b); continue; }
      int c;
      if (same) c = make_reshard(a, b, pb.model);
      else c = add_node({1, -1, nodes[a].step, -1, pb.src, pb.dst, 1, pb.model, slot(SLOT_COMM_PUB, p, 0, 0), true});
      add_edge(a, c);
      add_edge(c, b);
    }

  // 4b) lifetime barriers between colocated trainable layouts (lower.py:730-793)
  {
    std::vector<std::vector<int>> preds(nodes.size()), succs(nodes.size());
    for (auto& ed : edges) { preds[ed.second].push_back(ed.first); succs[ed.first].push_back(ed.second); }
    struct Tr { int node, pred, succ; };
    std::vector<Tr> to_train, to_serving;
    for (int i = 0; i < (int)nodes.size(); ++i) {
      if (!nodes[i].alive || nodes[i].kind != 2) continue;
      std::vector<int> po, so;
      for (int x : preds[i]) if (nodes[x].kind == 0) po.push_back(x);
      for (int x : succs[i]) if (nodes[x].kind == 0) so.push_back(x);
      if (po.size() != 1 || so.size() != 1) continue;
      const LoweredNode &pn = nodes[po[0]], &sn = nodes[so[0]];
      if (pn.model != sn.model || !st.trainable[pn.model]) continue;
      const int pr = st.vertex[pn.vertex].role, sr = st.vertex[sn.vertex].role;
      if (pr != RPEG_ROLE_TRAIN && sr == RPEG_ROLE_TRAIN) to_train.push_back({i, po[0], so[0]});
      else if (pr == RPEG_ROLE_TRAIN && sr != RPEG_ROLE_TRAIN) to_serving.push_back({i, po[0], so[0]});
    }
    for (auto& rt : to_train)
      for (auto& pb : to_serving) {
        const LoweredNode &producer = nodes[rt.pred], &consumer = nodes[pb.succ];
        if (producer.model == consumer.model || producer.step != consumer.step) continue;
        if (sg.disjoint(producer.vertex, consumer.vertex)) continue;
        if (!st.reach[producer.vertex][consumer.vertex]) continue;
        add_edge(rt.node, pb.node);
      }
  }

  // compact to alive nodes, keep order
  std::vector<int> remap(nodes.size(), -1);
  LoweredClass out;
  for (int i = 0; i < (int)nodes.size(); ++i)
    if (nodes[i].alive) { remap[i] = (int)out.nodes.size(); out.nodes.push_back(nodes[i]); }
  for (auto& ed : edges) {
    if (remap[ed.first] < 0 || remap[ed.second] < 0) throw std::runtime_error("edge to a removed node");
    out.edges.push_back({remap[ed.first], remap[ed.second]});
  }
  const int n = (int)out.nodes.size();
  if (n > 65535) throw std::runtime_error("too many lowered nodes");

  // adjacency in edge order, in-degrees, Kahn order (scheduler.py:28-67)
  std::vector<std::vector<int>> adj(n);
  std::vector<int> indeg(n, 0);
  for (auto& ed : out.edges) { adj[ed.first].push_back(ed.second); ++indeg[ed.second]; }
  std::vector<int> topo, deg = indeg;
  for (int i = 0; i < n; ++i) if (deg[i] == 0) topo.push_back(i);
  for (size_t h = 0; h < topo.size(); ++h)
    for (int w : adj[topo[h]]) if (--deg[w] == 0) topo.push_back(w);
  const bool cycle = (int)topo.size() != n;

  // chain groups: quantile sub-nodes of one (vertex, step) (scheduler.py:369-378)
  std::map<std::pair<int, int>, std::vector<int>> chains;
  for (int i = 0; i < n; ++i)
    if (out.nodes[i].kind == 0 && out.nodes[i].sub >= 0) chains[{out.nodes[i].vertex, out.nodes[i].step}].push_back(i);

  // vertex order of first appearance among operator nodes (dict orders of memory.py:763-808)
  uint8_t vorder[8] = {0, 1, 2, 3, 4, 5, 6, 7};
  {
    std::vector<bool> seen_v(nv, false);
    int c = 0;
    for (int i = 0; i < n; ++i)
      if (out.nodes[i].kind == 0 && !seen_v[out.nodes[i].vertex]) { seen_v[out.nodes[i].vertex] = true; vorder[c++] = (uint8_t)out.nodes[i].vertex; }
    if (c != nv) throw std::runtime_error("a template vertex has no lowered operator node");
    // The memory launch derives this order from the plan alone (plan_vorder): hold the two to each other here,
    // from the signature's predicates, for every class that is ever lowered.
    unsigned gs = 0, moved = 0;
    std::vector<uint8_t> want, tail;
    if (nph > 0) {
      for (int e = 0; e < st.n_edge; ++e)
        if (st.edge[e].gen_inf && sg.disjoint(st.edge[e].src, st.edge[e].dst)) gs |= 1u << st.edge[e].src;
      for (int e = 0; e < st.n_edge; ++e) {
        const int u = st.edge[e].src, v = st.edge[e].dst;
        if (!((gs >> u) & 1u) || st.vertex[v].role != RPEG_ROLE_INF || ((moved >> v) & 1u)) continue;
        if (sg.disjoint(u, v)) { moved |= 1u << v; tail.push_back((uint8_t)v); }
      }
    }
    for (int v = 0; v < nv; ++v)
      if (!((moved >> v) & 1u)) want.push_back((uint8_t)v);
    want.insert(want.end(), tail.begin(), tail.end());
    for (int v = 0; v < nv; ++v)
      if (want[v] != vorder[v]) throw std::logic_error("vertex order of the lowered graph differs from the plan's own");
  }

  // blob
  std::vector<NodeRec> recs(n);
  std::vector<uint16_t> succ, init, topo16, gmember;
  std::vector<GroupRec> groups;
  for (int i = 0; i < n; ++i) {
    const LoweredNode& nd = out.nodes[i];
    NodeRec r{};
    r.succ_begin = (uint16_t)succ.size();
    if (adj[i].size() > 255 || indeg[i] > 255 || succ.size() + adj[i].size() > 65535)
      throw std::runtime_error("node degree out of range");
    r.n_succ = (uint8_t)adj[i].size();
    for (int w : adj[i]) succ.push_back((uint16_t)w);
    r.slot = (uint8_t)nd.slot;
    r.indeg = (uint8_t)indeg[i];
    if (nd.kind == 0) {
      r.ptkey = (uint8_t)(8 + st.vertex[nd.vertex].topo_idx);
      r.blocked = (uint8_t)(1u << nd.vertex);
    } else {
      r.ptkey = (uint8_t)nv;  // comm_prio 0, topo_idx = number of template ids (scheduler.py:391-397)
      // transfer_resources.py:73-148.  "destination_only": weights reserve the destination, activations
      // also the source unless both adjacent operators use the same dp (a per-plan bit).
      // "both_endpoints" for the payload class: source and destination, whatever dp is.  A reshard's
      // two allocations are one and the same.
      const bool both = nd.kind == 1 && (P.transfer_both >> (nd.weight ? 0 : 1) & 1);
      r.blocked = (uint8_t)(1u << nd.a1 | (both ? 1u << nd.a0 : 0u));
      // (with both endpoints reserved the condition adds nothing to `blocked`; it is kept as the record of which
      // endpoint is the source: the utilisation lists a transfer's source devices before its destination's)
      r.cond = nd.weight && !both ? 0 : (uint8_t)(1 + nd.a0 * 8 + nd.a1);
    }
    recs[i] = r;
    if (indeg[i] == 0) init.push_back((uint16_t)i);
  }
  for (int v : topo) topo16.push_back((uint16_t)v);
  topo16.resize(n, 0);
  for (auto& kv : chains) {
    groups.push_back(GroupRec{(uint16_t)gmember.size(), (uint16_t)kv.second.size()});
    for (int i : kv.second) gmember.push_back((uint16_t)i);
  }
  // every slot's place in the structure's slot universe
  std::vector<uint8_t> umap(slots.size(), 0);
  {
    SlotDesc uni[RPEG_MAX_UNIVERSE];
    const int nu = slot_universe(P, st, uni);
    if (nu > RPEG_MAX_UNIVERSE) throw std::runtime_error("slot universe too large");
    for (size_t k = 0; k < slots.size(); ++k) {
      int hit = -1;
      for (int u = 0; u < nu && hit < 0; ++u)
        if (uni[u].type == slots[k].type && uni[u].a == slots[k].a && uni[u].b == slots[k].b && uni[u].q == slots[k].q) hit = u;
      if (hit < 0) throw std::logic_error("a duration slot outside the slot universe");
      umap[k] = (uint8_t)hit;
    }
  }
  std::vector<uint16_t> pbeg(n + 1, 0), pred(out.edges.size(), 0);
  {
    for (auto& ed : out.edges) ++pbeg[ed.second + 1];
    for (int i = 0; i < n; ++i) pbeg[i + 1] = (uint16_t)(pbeg[i + 1] + pbeg[i]);
    std::vector<uint16_t> cur(pbeg.begin(), pbeg.end() - 1);
    for (auto& ed : out.edges) pred[cur[ed.second]++] = (uint16_t)ed.first;
  }
  ClassHdr h{};
  h.n_nodes = n; h.n_slots = (uint32_t)slots.size(); h.n_succ = (uint32_t)succ.size(); h.n_init = (uint32_t)init.size();
  h.n_groups = (uint32_t)groups.size(); h.n_gmembers = (uint32_t)gmember.size();
  h.structure = sg.structure(); h.split = split; h.error = cycle ? 1u : 0u;
  std::memcpy(h.vorder, vorder, 8);
  auto align8 = [](size_t x) { return (x + 7) & ~size_t(7); };
  size_t off = align8(sizeof(ClassHdr));
  h.off_node = (uint32_t)off; off = align8(off + recs.size() * sizeof(NodeRec));
  h.off_succ = (uint32_t)off; off = align8(off + succ.size() * 2);
  h.off_init = (uint32_t)off; off = align8(off + init.size() * 2);
  h.off_topo = (uint32_t)off; off = align8(off + topo16.size() * 2);
  h.off_slot = (uint32_t)off; off = align8(off + slots.size() * sizeof(SlotDesc));
  h.off_group = (uint32_t)off; off = align8(off + groups.size() * sizeof(GroupRec));
  h.off_gmember = (uint32_t)off; off = align8(off + gmember.size() * 2);
  h.off_pbeg = (uint32_t)off; off = align8(off + pbeg.size() * 2);
  h.off_pred = (uint32_t)off; off = align8(off + pred.size() * 2);
  h.off_umap = (uint32_t)off; off = align8(off + umap.size());
  h.bytes = (uint32_t)off;
  out.blob.assign(off, 0);
  std::memcpy(out.blob.data(), &h, sizeof h);
  if (!recs.empty()) std::memcpy(out.blob.data() + h.off_node, recs.data(), recs.size() * sizeof(NodeRec));
  if (!succ.empty()) std::memcpy(out.blob.data() + h.off_succ, succ.data(), succ.size() * 2);
  if (!init.empty()) std::memcpy(out.blob.data() + h.off_init, init.data(), init.size() * 2);
  if (!topo16.empty()) std::memcpy(out.blob.data() + h.off_topo, topo16.data(), topo16.size() * 2);
  if (!slots.empty()) std::memcpy(out.blob.data() + h.off_slot, slots.data(), slots.size() * sizeof(SlotDesc));
  if (!groups.empty()) std::memcpy(out.blob.data() + h.off_group, groups.data(), groups.size() * sizeof(GroupRec));
  if (!gmember.empty()) std::memcpy(out.blob.data() + h.off_gmember, gmember.data(), gmember.size() * 2);
  std::memcpy(out.blob.data() + h.off_pbeg, pbeg.data(), pbeg.size() * 2);
  if (!pred.empty()) std::memcpy(out.blob.data() + h.off_pred, pred.data(), pred.size() * 2);
  if (!umap.empty()) std::memcpy(out.blob.data() + h.off_umap, umap.data(), umap.size());
  return out;
}

}  // namespace rpeg
#endif
