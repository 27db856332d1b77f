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
#include <stdexcept>
#include <string>
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

  // (A class is lowered on the critical path of the first call that meets it: flat arrays and one small open-addressing
  // table instead of node-based containers; the orders -- of nodes, of edges, of slots -- are the reference's.)
  std::vector<LoweredNode> nodes;
  std::vector<std::pair<int, int>> edges;
  nodes.reserve(512);
  edges.reserve(1024);
  std::vector<uint64_t> seen(2048, ~0ull);   // the edges met so far, keyed by (from << 32 | to)
  size_t n_seen = 0;
  auto seen_insert = [&](uint64_t key) {   // true when the key is new
    if (2 * (n_seen + 1) > seen.size()) {
      std::vector<uint64_t> old(seen.size() * 2, ~0ull);
      old.swap(seen);
      for (uint64_t k : old)
        if (k != ~0ull) {
          size_t h = (size_t)((k * 0x9E3779B97F4A7C15ull) >> 20) & (seen.size() - 1);
          while (seen[h] != ~0ull) h = (h + 1) & (seen.size() - 1);
          seen[h] = k;
        }
    }
    size_t h = (size_t)((key * 0x9E3779B97F4A7C15ull) >> 20) & (seen.size() - 1);
    while (seen[h] != ~0ull) {
      if (seen[h] == key) return false;
      h = (h + 1) & (seen.size() - 1);
    }
    seen[h] = key;
    ++n_seen;
    return true;
  };
  std::vector<SlotDesc> slots;
  slots.reserve(64);
  auto slot = [&](SlotType t, int a, int b, int q) {
    const SlotDesc want{(uint8_t)t, (uint8_t)a, (uint8_t)b, (uint8_t)q};
    for (size_t k = 0; k < slots.size(); ++k)
      if (slots[k].type == want.type && slots[k].a == want.a && slots[k].b == want.b && slots[k].q == want.q) return (int)k;
    if (slots.size() >= 255) throw std::runtime_error("too many duration slots");
    slots.push_back(want);
    return (int)slots.size() - 1;
  };
  auto add_edge = [&](int a, int b) {
    if (seen_insert((uint64_t)(uint32_t)a << 32 | (uint32_t)b)) edges.push_back({a, b});
  };
  auto add_node = [&](const LoweredNode& n) { nodes.push_back(n); return (int)nodes.size() - 1; };

  // per (vertex, step): the unsplit node; the first of the generation / inference sub-nodes (they are created one
  // after the other, so sub-node q of a vertex and step is first + q; -1: none)
  std::vector<int> base((size_t)nv * K, -1), gfirst((size_t)nv * K, -1), ifirst((size_t)nv * K, -1);
  auto at = [&](int v, int k) { return (size_t)v * K + k; };

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
        for (int q = 0; q < nph; ++q) {
          const int id = add_node({0, v, k, q, v, v, 0, st.vertex[v].model, slot(SLOT_OP_SUB, v, 0, q), true});
          if (q == 0) gfirst[at(v, k)] = id;
        }
        for (int q = 1; q < nph; ++q) add_edge(gfirst[at(v, k)] + q - 1, gfirst[at(v, k)] + q);
      } else {
        base[at(v, k)] = add_node({0, v, k, -1, v, v, 0, st.vertex[v].model, slot(SLOT_OP_UNSPLIT, v, 0, 0), true});
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
      if (gfirst[at(ed.src, k)] >= 0 && st.vertex[ed.dst].role == RPEG_ROLE_INF) pass1.push_back({k, e});
      else pass2.push_back({k, e});
    }
  pass1.insert(pass1.end(), pass2.begin(), pass2.end());
  for (auto& ke : pass1) {
    const int k = ke.first, e = ke.second;
    const rpeg_edge_t& ed = st.edge[e];
    const int u = ed.src, v = ed.dst;
    const int gu = gfirst[at(u, k)];
    const bool src_gen_split = gu >= 0;
    if (src_gen_split && st.vertex[v].role == RPEG_ROLE_INF) {
      if (sg.disjoint(u, v)) {
        if (ifirst[at(v, k)] < 0) {
          if (base[at(v, k)] >= 0) { nodes[base[at(v, k)]].alive = false; base[at(v, k)] = -1; }
          for (int q = 0; q < nph; ++q) {
            const int id = add_node({0, v, k, q, v, v, 0, st.vertex[v].model, slot(SLOT_OP_SUB, v, 0, q), true});
            if (q == 0) ifirst[at(v, k)] = id;
          }
          for (int q = 1; q < nph; ++q) add_edge(ifirst[at(v, k)] + q - 1, ifirst[at(v, k)] + q);
        }
        for (int q = 0; q < nph; ++q) edge_or_comm(gu + q, ifirst[at(v, k)] + q, e, q);
      } else {
        edge_or_comm(gu + nph - 1, base[at(v, k)], e, -1);
      }
    } else if (src_gen_split) {
      edge_or_comm(gu + nph - 1, base[at(v, k)], e, -1);
    } else if (ifirst[at(u, k)] >= 0) {
      if (base[at(v, k)] < 0) throw std::runtime_error("destination node of a split inference edge not found");
      edge_or_comm(ifirst[at(u, k)] + nph - 1, base[at(v, k)], e, -1);
    } else {
      if (base[at(u, k)] < 0 || base[at(v, k)] < 0) throw std::runtime_error("edge endpoint missing");
      edge_or_comm(base[at(u, k)], base[at(v, k)], e, -1);
    }
  }

  // 3) within-step weight reshards between consecutive vertices of one trainable model (lower.py:626-681)
  auto last_of = [&](int v, int k) {
    if (gfirst[at(v, k)] >= 0) return gfirst[at(v, k)] + nph - 1;
    if (ifirst[at(v, k)] >= 0) return ifirst[at(v, k)] + nph - 1;
    return base[at(v, k)];
  };
  auto first_of = [&](int v, int k) {
    if (gfirst[at(v, k)] >= 0) return gfirst[at(v, k)];
    if (ifirst[at(v, k)] >= 0) return ifirst[at(v, k)];
    return base[at(v, k)];
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
      const int a = base[at(pb.src, ks)];
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
    // operator predecessors / successors of the reshard nodes: how many, and one of them
    std::vector<int> n_po(nodes.size(), 0), n_so(nodes.size(), 0), a_po(nodes.size(), -1), a_so(nodes.size(), -1);
    bool any_reshard = false;
    for (auto& nd : nodes) any_reshard = any_reshard || (nd.alive && nd.kind == 2);
    if (any_reshard)
      for (auto& ed : edges) {
        if (nodes[ed.second].kind == 2 && nodes[ed.first].kind == 0) { ++n_po[ed.second]; a_po[ed.second] = ed.first; }
        if (nodes[ed.first].kind == 2 && nodes[ed.second].kind == 0) { ++n_so[ed.first]; a_so[ed.first] = ed.second; }
      }
    struct Tr { int node, pred, succ; };
    std::vector<Tr> to_train, to_serving;
    for (int i = 0; any_reshard && i < (int)nodes.size(); ++i) {
      if (!nodes[i].alive || nodes[i].kind != 2) continue;
      if (n_po[i] != 1 || n_so[i] != 1) continue;
      const int po[1] = {a_po[i]}, so[1] = {a_so[i]};
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
  out.nodes.reserve(nodes.size());
  out.edges.reserve(edges.size());
  for (int i = 0; i < (int)nodes.size(); ++i)
    if (nodes[i].alive) { remap[i] = (int)out.nodes.size(); out.nodes.push_back(nodes[i]); }
  for (auto& ed : edges) {
    if (remap[ed.first] < 0 || remap[ed.second] < 0) throw std::runtime_error("edge to a removed node");
    out.edges.push_back({remap[ed.first], remap[ed.second]});
  }
  const int n = (int)out.nodes.size();
  if (n > 65535) throw std::runtime_error("too many lowered nodes");

  // adjacency in edge order, in-degrees, Kahn order (scheduler.py:28-67)
  std::vector<int> adj_beg(n + 1, 0), adj_to(out.edges.size(), 0);   // (successors of a node in the order of its edges)
  std::vector<int> indeg(n, 0);
  for (auto& ed : out.edges) { ++adj_beg[ed.first + 1]; ++indeg[ed.second]; }
  for (int i = 0; i < n; ++i) adj_beg[i + 1] += adj_beg[i];
  {
    std::vector<int> cur(adj_beg.begin(), adj_beg.end() - 1);
    for (auto& ed : out.edges) adj_to[cur[ed.first]++] = ed.second;
  }
  std::vector<int> topo, deg = indeg;
  topo.reserve(n);
  for (int i = 0; i < n; ++i) if (deg[i] == 0) topo.push_back(i);
  for (size_t h = 0; h < topo.size(); ++h)
    for (int j = adj_beg[topo[h]]; j < adj_beg[topo[h] + 1]; ++j) if (--deg[adj_to[j]] == 0) topo.push_back(adj_to[j]);
  const bool cycle = (int)topo.size() != n;

  // chain groups: quantile sub-nodes of one (vertex, step) (scheduler.py:369-378), the groups in the order of
  // (vertex, step), the members of a group in node order
  std::vector<int> chain_beg((size_t)nv * K + 1, 0), chain_of;
  for (int i = 0; i < n; ++i)
    if (out.nodes[i].kind == 0 && out.nodes[i].sub >= 0) ++chain_beg[at(out.nodes[i].vertex, out.nodes[i].step) + 1];
  for (size_t k = 0; k < (size_t)nv * K; ++k) chain_beg[k + 1] += chain_beg[k];
  chain_of.assign(chain_beg.back(), 0);
  {
    std::vector<int> cur(chain_beg.begin(), chain_beg.end() - 1);
    for (int i = 0; i < n; ++i)
      if (out.nodes[i].kind == 0 && out.nodes[i].sub >= 0) chain_of[cur[at(out.nodes[i].vertex, out.nodes[i].step)]++] = i;
  }

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
  succ.reserve(out.edges.size());
  topo16.reserve(n);
  for (int i = 0; i < n; ++i) {
    const LoweredNode& nd = out.nodes[i];
    NodeRec r{};
    r.succ_begin = (uint16_t)succ.size();
    const int n_adj = adj_beg[i + 1] - adj_beg[i];
    if (n_adj > 255 || indeg[i] > 255 || succ.size() + (size_t)n_adj > 65535)
      throw std::runtime_error("node degree out of range");
    r.n_succ = (uint8_t)n_adj;
    for (int j = adj_beg[i]; j < adj_beg[i + 1]; ++j) succ.push_back((uint16_t)adj_to[j]);
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
  for (size_t k = 0; k < (size_t)nv * K; ++k) {
    if (chain_beg[k + 1] == chain_beg[k]) continue;
    groups.push_back(GroupRec{(uint16_t)gmember.size(), (uint16_t)(chain_beg[k + 1] - chain_beg[k])});
    for (int j = chain_beg[k]; j < chain_beg[k + 1]; ++j) gmember.push_back((uint16_t)chain_of[j]);
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
