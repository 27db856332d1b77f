// rpeg_kernel_quad.h - four lanes per plan, sixteen plans per wavefront (device only).
//
// For the classes whose wavefronts would end last in the plan-per-lane kernel (rpeg_kernel_eval.h): dense graphs
// whose ready lists are long and whose keys go stale often.  There a scheduling step is a chain of dependent LDS
// round trips; here the ready set of a plan lives in the REGISTERS of its four lanes, eight entries each, unordered:
//
//   entry = key (est, 8 bytes) | order word: position << 20 | tie | meta: node | reserved vertices << 12
//
// `position` is the place of the node in the order (comm_prio*8+topo_idx ascending, rank descending) of the plan's
// nodes, equal for nodes that agree in both; `tie` counts pushes.  (est, position, tie) is the reference's heap key
// (est, comm_prio, topo_idx, -rank, tie) of scheduler.py:427, so the heap is taken literally: a pop is the minimum
// over the 32 entries (minima in each lane, two quad-permute steps across the lanes, no memory access), a stale
// entry is re-keyed in place with a fresh tie (scheduler.py:437-443), a dispatched entry is cleared in place.  The
// four lanes look at four successors at once; those that became ready are handed, in successor order, to the lanes
// that have a free slot (one each per round, the rounds repeated until all are filed).  A plan with more than 32
// entries ready at once, or more than 2^20 pushes, is not evaluated here: it is flagged (EvalLaunch::limit) and redone
// by the launch that ends the call, whose ready list is as long as the graph.
//
// Per-plan state (ready time, rank, position, in-degree per node, duration per slot) is in LDS, interleaved by plan.
// Before the scheduling loop the four lanes of a plan share the cost model (slots by lane), the per-vertex memory
// terms, the positions and the initialisation; the rank sweep runs in all four alike.
#ifndef RPEG_KERNEL_QUAD_H
#define RPEG_KERNEL_QUAD_H

#include "rpeg_kernel_eval.h"

namespace rpeg {

constexpr int KQ_LANES = 4;       // lanes per plan
constexpr int KQ_PLANS = 16;      // plans per wavefront
constexpr int KQ_ENTRIES = 32;    // ready entries per plan, spread over its lanes
constexpr uint32_t KQ_TIE_BITS = 20, KQ_TIE_MASK = (1u << KQ_TIE_BITS) - 1u;
constexpr uint32_t KQ_EMPTY = 0xFFFFFFFFu;

// LDS of one wavefront of `np` plans: class tables (node records, successor lists), the class's reverse order and its
// nodes grouped by tie-break class (uint16 each, first-node table of 17 words), plan fields, memory terms, then the
// per-plan state [row][plan]: time and rank (a double per node each; ONE array for both unless the critical-chain
// masses are asked for: a rank is not read again once the positions are known, a ready time not written before),
// duration (double per slot), position (uint16 per node), in-degree (byte per node).
__host__ __device__ inline size_t kq_tab_bytes(uint32_t nodes) { return ((size_t)nodes * 4 + 17 * 2 + 15) & ~size_t(15); }
__host__ __device__ inline size_t kq_dyn_bytes(uint32_t nv, uint32_t np) {
  (void)nv; (void)np;   // (plan fields and memory terms used to sit here: the prologue launch computes from them now)
  return 0;
}
__host__ __device__ inline size_t kq_lds_bytes(uint32_t cls_bytes, uint32_t nodes, uint32_t slots, uint32_t nv, uint32_t np, bool mass) {
  return cls_bytes + kq_tab_bytes(nodes) + kq_dyn_bytes(nv, np) +
         (size_t)np * (((mass ? 16ull : 8ull) * nodes + 8ull * slots + 3ull * nodes + 15) & ~15ull);
}

#if defined(__HIPCC__)

template <int CTRL>
__device__ inline uint32_t kq_dpp(uint32_t v) {
  return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, 0xF, 0xF, false);
}
template <int CTRL>
__device__ inline double kq_dpp(double v) {
  return __hiloint2double((int)kq_dpp<CTRL>((uint32_t)__double2hiint(v)), (int)kq_dpp<CTRL>((uint32_t)__double2loint(v)));
}
constexpr int KQ_XOR1 = 0xB1, KQ_XOR2 = 0x4E;   // quad_perm [1,0,3,2], [2,3,0,1]

// reductions over the four lanes of a plan (a quad)
__device__ inline uint32_t kq_or(uint32_t v) {
  v |= kq_dpp<KQ_XOR1>(v);
  v |= kq_dpp<KQ_XOR2>(v);
  return v;
}
__device__ inline uint32_t kq_min(uint32_t v) {
  uint32_t o = kq_dpp<KQ_XOR1>(v);
  v = o < v ? o : v;
  o = kq_dpp<KQ_XOR2>(v);
  v = o < v ? o : v;
  return v;
}
__device__ inline double kq_min(double v) {
  v = __builtin_fmin(v, kq_dpp<KQ_XOR1>(v));
  v = __builtin_fmin(v, kq_dpp<KQ_XOR2>(v));
  return v;
}

__device__ inline void kq_eval_wave(const EvalLaunch& L, uint64_t w, uint8_t* lds) {
  constexpr int QL = KQ_LANES, NP = KQ_PLANS;
  constexpr int SL = KQ_ENTRIES / QL;       // ready entries per lane
  constexpr int RW = NP;
  const int lane = threadIdx.x, p = lane / QL, q = lane % QL;
  int first_lane = 0;
  const rpeg_problem_t& P = *L.P;
  const ClassView cv = class_view(L.pool + (L.wave_cls[w] & ~KE_CLS_LDS));   // uniform
  const int n = (int)cv.h->n_nodes, n_slots = (int)cv.h->n_slots, n_succ_all = (int)cv.h->n_succ;

  // ---- LDS carve-up
  uint64_t* l_node = (uint64_t*)lds;                                  // NodeRec[n]
  uint16_t* l_succ = (uint16_t*)(lds + (size_t)n * 8);                // uint16[n_succ]
  uint16_t* l_topo = (uint16_t*)(lds + L.cls_bytes);                  // uint16[n]: the class's topological order
  uint16_t* l_bykey = l_topo + L.ws_nodes;                            // uint16[n]: nodes grouped by tie-break class
  uint16_t* l_kbeg = l_bykey + L.ws_nodes;                            // uint16[17]: first place of every tie-break class
  uint8_t* dyn = lds + L.cls_bytes + kq_tab_bytes(L.ws_nodes);
  uint8_t* sbase = dyn + kq_dyn_bytes(L.max_v, NP);
  const size_t tr_rows = (L.mass ? 2 : 1) * (size_t)L.ws_nodes;   // rows of the time and rank arrays together
  double* g_time = (double*)sbase + p;
  double* g_rank = L.mass ? g_time + (size_t)L.ws_nodes * RW : g_time;
  double* g_dur = (double*)sbase + tr_rows * RW + p;
  uint16_t* g_pos = (uint16_t*)((double*)sbase + (tr_rows + L.ws_slots) * RW) + p;
  uint8_t* g_deg = (uint8_t*)((uint16_t*)((double*)sbase + (tr_rows + L.ws_slots) * RW) + (size_t)L.ws_nodes * RW) + p;

  const uint64_t pi = (uint64_t)L.perm[w * KE_WAVE + p];
  __syncthreads();  // the previous task of this wavefront is done with LDS
  for (int i = lane; i < n; i += KE_WAVE) {
    l_node[i] = ((const uint64_t*)cv.node)[i];
    l_topo[i] = cv.topo[i];
  }
  for (int i = lane; i < n_succ_all; i += KE_WAVE) l_succ[i] = cv.succ[i];
  __syncthreads();
  auto node_at = [&](int v) { NodeRec r; const uint64_t b = l_node[v]; __builtin_memcpy(&r, &b, 8); return r; };
  // nodes grouped by tie-break class (comm_prio*8+topo_idx < 16), ascending: lane k counts and places class k
  if (lane < 16) {
    int cnt = 0;
    for (int v = 0; v < n; ++v) cnt += node_at(v).ptkey == lane ? 1 : 0;
    int beg = cnt;   // inclusive prefix over the 16 classes, then exclusive
    for (int d = 1; d < 16; d <<= 1) {
      const int o = __shfl_up(beg, d, 16);
      if (lane >= d) beg += o;
    }
    beg -= cnt;
    l_kbeg[lane] = (uint16_t)beg;
    if (lane == 15) l_kbeg[16] = (uint16_t)(beg + cnt);
    for (int v = 0; v < n; ++v)
      if (node_at(v).ptkey == lane) l_bykey[beg++] = (uint16_t)v;
  }
  __syncthreads();
  if (pi == KE_IDLE) return;   // all lanes of a plan leave together: the lane exchanges below stay within a plan
  first_lane = __builtin_ctzll(__ballot(1));
  KE_STAMP(0);

  const rpeg_struct_t& st = P.st[cv.h->structure];   // uniform (the class fixes the structure)
  (void)st;
  // pair relations, penalty factor and gate bits of this plan and the durations of its class's slots (out of the table
  // of the slot universe) come from the prologue launches, by plan index
  const uint64_t ovl = L.aux_ovl[pi], dpne = L.aux_dpne[pi];
  const double pen = L.aux_pen ? L.aux_pen[pi] : 1.0;
  const uint8_t gates = L.aux_mask ? L.aux_mask[pi] : (uint8_t)(RPEG_MASK_VALID | RPEG_MASK_STALE_OK | RPEG_MASK_MEM_OK);
  KE_STAMP(1);
  bool err = cv.h->error != 0;
  {   // a slot whose duration the reference could not compute (division by zero) is NaN; a share by each lane
    bool bad = false;
    for (int s = q; s < n_slots; s += QL) {
      const double d = L.dur[(size_t)cv.umap[s] * L.dur_stride + pi];
      g_dur[s * RW] = d;
      bad = bad || d != d;
    }
    err = err || kq_or(bad ? 1u : 0u) != 0u;
  }
  __syncthreads();
  KE_STAMP(2);
  const bool stale_ok = (gates & RPEG_MASK_STALE_OK) != 0, mem_ok = (gates & RPEG_MASK_MEM_OK) != 0;

  KE_STAMP(3);
  // ---- ranks: reverse topological pass, then chain inheritance (scheduler.py:71-100, 367-378); all lanes alike
  for (int i = n - 1; i >= 0; --i) {
    const int v = l_topo[i];
    const NodeRec nr = node_at(v);
    double best = 0.0;
    const double dv = g_dur[nr.slot * RW];
    int j = 0;
    for (; j + 2 <= nr.n_succ; j += 2) {   // two independent pairs of LDS reads in flight
      const int u0 = l_succ[nr.succ_begin + j], u1 = l_succ[nr.succ_begin + j + 1];
      const double r0 = g_rank[u0 * RW], r1 = g_rank[u1 * RW];
      best = r0 > best ? r0 : best;
      best = r1 > best ? r1 : best;
    }
    if (j < nr.n_succ) {
      const double r = g_rank[(int)l_succ[nr.succ_begin + j] * RW];
      best = r > best ? r : best;
    }
    g_rank[v * RW] = dv + best;
  }
  for (unsigned g = 0; g < cv.h->n_groups; ++g) {
    const GroupRec gr = cv.group[g];
    double top = g_rank[(int)cv.gmember[gr.begin] * RW];
    for (int j = 1; j < gr.count; ++j) {
      const double r = g_rank[(int)cv.gmember[gr.begin + j] * RW];
      top = r > top ? r : top;
    }
    for (int j = 0; j < gr.count; ++j) g_rank[(int)cv.gmember[gr.begin + j] * RW] = top;
  }
  __syncthreads();
#ifdef KE_FINE_PROF
  KE_STAMP(4);
#endif
  // ---- positions: nodes before v in (comm_prio*8+topo_idx ascending, rank descending) = the nodes of lower
  // tie-break classes and the nodes of its own class with a larger rank
  for (int i = q; i < n; i += QL) {
    const int v = l_bykey[i];
    const unsigned k = node_at(v).ptkey;
    const int b0 = l_kbeg[k], b1 = l_kbeg[k + 1];
    const double rv = g_rank[v * RW];
    int cnt = b0;
    int j = b0;
    for (; j + 4 <= b1; j += 4) {   // four independent pairs of LDS reads in flight
      const int u0 = l_bykey[j], u1 = l_bykey[j + 1], u2 = l_bykey[j + 2], u3 = l_bykey[j + 3];
      const double r0 = g_rank[u0 * RW], r1 = g_rank[u1 * RW], r2 = g_rank[u2 * RW], r3 = g_rank[u3 * RW];
      cnt += (r0 > rv ? 1 : 0) + (r1 > rv ? 1 : 0) + (r2 > rv ? 1 : 0) + (r3 > rv ? 1 : 0);
    }
    for (; j < b1; ++j) cnt += g_rank[(int)l_bykey[j] * RW] > rv ? 1 : 0;
    g_pos[v * RW] = (uint16_t)cnt;
  }
  __syncthreads();   // (the ranks are dead from here on: their array becomes the ready times)
  for (int v = q; v < n; v += QL) {
    g_deg[v * RW] = node_at(v).indeg;
    g_time[v * RW] = 0.0;
  }
  __syncthreads();

#ifndef KE_FINE_PROF
  KE_STAMP(4);
#endif
  // ---- list scheduling (scheduler.py:399-546)
  double lf[RPEG_MAX_V];
#pragma unroll
  for (int x = 0; x < RPEG_MAX_V; ++x) lf[x] = 0.0;
  const double inf = __builtin_inf();
  double ek[SL];
  uint32_t eo[SL], em[SL];
#pragma unroll
  for (int u = 0; u < SL; ++u) { ek[u] = inf; eo[u] = KQ_EMPTY; em[u] = 0u; }
  uint32_t tie = 0;
  bool ovf = false;
  const unsigned group_shift = (unsigned)(lane & ~(QL - 1));
  const uint32_t below = (1u << q) - 1u;   // the lanes of this plan before this one
  // Entry `j` of a round of new entries goes to the j-th lane of the plan that has a free slot.  free_rank: the
  // place of this lane among those lanes (QL if it has none); returns its first free slot in u_free.
  auto free_rank = [&](int& u_free) {
    uint32_t fm = 0;
#pragma unroll
    for (int u = 0; u < SL; ++u) fm |= eo[u] == KQ_EMPTY ? 1u << u : 0u;
    u_free = fm ? __builtin_ctz(fm) : SL;
    const uint32_t g = (uint32_t)(__ballot(fm != 0u) >> group_shift) & ((1u << QL) - 1u);
    return fm ? (int)__builtin_popcount(g & below) : QL;
  };
  auto file = [&](int u_free, double key, uint32_t ord, uint32_t node_blk) {
#pragma unroll
    for (int u = 0; u < SL; ++u)
      if (u_free == u) { ek[u] = key; eo[u] = ord; em[u] = node_blk; }
  };
  {
    const int n_init = (int)cv.h->n_init;
    if (n_init > KQ_ENTRIES) ovf = true;
    for (int i0 = 0; i0 < n_init && !ovf; i0 += QL) {   // (at most 32 entries: every lane has room in every round)
      int u_free;
      const int r = free_rank(u_free);
      const bool mine = r < QL && i0 + r < n_init;
      if (mine) {
        const int v = cv.init[i0 + r];
        file(u_free, 0.0, ((uint32_t)g_pos[v * RW] << KQ_TIE_BITS) | (uint32_t)(i0 + r), (uint32_t)v | (blocked_mask(node_at(v), dpne) << 12));
      }
    }
    tie = (uint32_t)n_init;
  }
  if (kq_or(ovf ? 1u : 0u)) { ovf = true; err = true; }
  double makespan = 0.0;
  int done = 0;
  uint32_t guard_total = 0;
  auto min_u32 = [](uint32_t x, uint32_t y) { return x < y ? x : y; };
  while (!err && done < n) {
    // The heap's pops up to the next dispatch.  A pop: the smallest key of the 32 slots (minima in each lane, then
    // across the lanes), the smallest order word among the slots of that key, the meta word of the slot that holds
    // it (order words are unique).  A stale entry is re-keyed in place with a fresh tie (scheduler.py:437-443): every
    // stale pop makes one entry current, so at most 32 follow one another.  An empty set pops an empty slot, never stale.
    double bk, est;
    uint32_t bo, bm;
    for (;;) {
      ++guard_total;
      bk = ek[0];
#pragma unroll
      for (int u = 1; u < SL; ++u) bk = __builtin_fmin(bk, ek[u]);
      bk = kq_min(bk);
      bo = KQ_EMPTY;
#pragma unroll
      for (int u = 0; u < SL; ++u) bo = min_u32(bo, ek[u] == bk ? eo[u] : KQ_EMPTY);
      bo = kq_min(bo);
      bm = 0;
#pragma unroll
      for (int u = 0; u < SL; ++u) bm |= eo[u] == bo ? em[u] : 0u;
      bm = kq_or(bm);
      const double dv = ke_dev_max((bm >> 12) & 0xFFu, lf);
      est = dv > bk ? dv : bk;
      if (!(est > bk)) break;
      const uint32_t no = (bo & ~KQ_TIE_MASK) | tie;
      ++tie;
#pragma unroll
      for (int u = 0; u < SL; ++u)
        if (eo[u] == bo) { ek[u] = est; eo[u] = no; }
    }
    if (bo == KQ_EMPTY) { err = true; break; }
#pragma unroll
    for (int u = 0; u < SL; ++u)   // the dispatched entry leaves its slot
      if (eo[u] == bo) { ek[u] = inf; eo[u] = KQ_EMPTY; }
    const int bv = (int)(bm & 0xFFFu);
    const unsigned blocked = (bm >> 12) & 0xFFu;
    const NodeRec nr = node_at(bv);
    const double fin = est + g_dur[nr.slot * RW];
    makespan = fin > makespan ? fin : makespan;
    ++done;
    if (L.mass && q == 0) {  // keep the trace: a dispatched node needs neither its ready time nor its rank again
      g_time[bv * RW] = fin;
      g_rank[bv * RW] = est;
    }
    unsigned touched = 0;
#pragma unroll
    for (int x = 0; x < RPEG_MAX_V; ++x)
      if ((blocked >> x) & 1u) touched |= mask_row(ovl, x);
#pragma unroll
    for (int x = 0; x < RPEG_MAX_V; ++x)
      if (((touched >> x) & 1u) && fin > lf[x]) lf[x] = fin;
    // successors, QL at a time: lane q looks at successor j0 + q; those that became ready are filed in successor
    // order (scheduler.py:540-546), the j-th of them by the j-th lane with a free slot
    const int ns = nr.n_succ;
    for (int j0 = 0; j0 < ns; j0 += QL) {
      const bool mine = j0 + q < ns;
      const int wn = mine ? (int)l_succ[nr.succ_begin + j0 + q] : 0;
      bool ready = false;
      double t = 0.0;
      if (mine) {
        const double t0 = g_time[wn * RW];
        const uint8_t left = (uint8_t)(g_deg[wn * RW] - 1);
        t = fin > t0 ? fin : t0;
        ready = left == 0;
        if (!ready) {
          g_time[wn * RW] = t;
          g_deg[wn * RW] = left;
        }
      }
      uint32_t ord = 0, node_blk = 0;
      if (ready) {
        const unsigned blk = blocked_mask(node_at(wn), dpne);
        const double d2 = ke_dev_max(blk, lf);
        t = d2 > t ? d2 : t;
        ord = (uint32_t)g_pos[wn * RW] << KQ_TIE_BITS;
        node_blk = (uint32_t)wn | (blk << 12);
      }
      // hand the ready ones over: the j-th ready successor (lane order = successor order) to the j-th lane with room
      const uint32_t rdy = (uint32_t)(__ballot(ready) >> group_shift) & ((1u << QL) - 1u);
      const int n_rdy = __builtin_popcount(rdy);
      if (n_rdy) {   // uniform within the plan
        // A round hands one entry to every lane that has room; the rounds repeat until every entry is filed, so that a
        // plan overflows only when fewer free slots than entries are left in all four lanes together.
        uint32_t rem = rdy;
        int filed = 0;
        while (rem) {
          int u_free;
          const int r = free_rank(u_free);
          const uint32_t room = (uint32_t)(__ballot(r < QL) >> group_shift) & ((1u << QL) - 1u);
          const int n_room = __builtin_popcount(room), n_rem = __builtin_popcount(rem);
          if (n_room == 0) { ovf = true; break; }
          // source lane of the r-th ready successor still to file
          uint32_t src_mask = rem;
          for (int k = 0; k < r && k < QL; ++k) src_mask &= src_mask - 1u;
          const bool take = r < n_rem;
          const int src = (int)group_shift + (take ? __builtin_ctz(src_mask) : 0);
          const double tk = __hiloint2double(__builtin_amdgcn_ds_bpermute(src << 2, __double2hiint(t)),
                                             __builtin_amdgcn_ds_bpermute(src << 2, __double2loint(t)));
          const uint32_t to = (uint32_t)__builtin_amdgcn_ds_bpermute(src << 2, (int)ord);
          const uint32_t tm = (uint32_t)__builtin_amdgcn_ds_bpermute(src << 2, (int)node_blk);
          file(take ? u_free : SL, tk, to | (tie + (uint32_t)(filed + r)), tm);
          const int k_done = n_room < n_rem ? n_room : n_rem;
          for (int k = 0; k < k_done; ++k) rem &= rem - 1u;
          filed += k_done;
        }
        tie += (uint32_t)n_rdy;
      }
    }
    if (kq_or(ovf ? 1u : 0u) || tie >= KQ_TIE_MASK - 64u) { ovf = true; err = true; }
  }
  if (done != n) err = true;
  if (ovf && q == 0) ke_flag_limit(L, pi, L.wave_cls[w] & ~KE_CLS_LDS);
  KE_STAMP(5);
  if (L.prof && q == 0) atomicMax(&L.prof[w * 8 + 7], ((unsigned long long)n << 32) | (unsigned long long)guard_total);

  // ---- outputs
  uint8_t mask = RPEG_MASK_VALID;
  if (stale_ok) mask |= RPEG_MASK_STALE_OK;
  if (mem_ok) mask |= RPEG_MASK_MEM_OK;
  double out_makespan, out_score;
  if (err || makespan == 0.0) {
    out_makespan = out_score = __builtin_nan("");
    mask |= RPEG_MASK_ERROR;
    if (ovf) mask |= RPEG_MASK_LIMIT;
  } else {
    double score = P.score_num / makespan;
    if (!mem_ok) score = score * pen;
    if ((L.flags & RPEG_GATE_STALE) && !stale_ok) score = 0.0;
    out_makespan = makespan;
    out_score = score;
  }
  if (q == 0) {
    if (L.makespan) L.makespan[pi] = out_makespan;   // (the peak is the prologue launch's output)
    if (L.score) L.score[pi] = out_score;
    if (L.mask) L.mask[pi] = mask;
    if (L.mass) {
      double m[RPEG_MAX_V];
      if (err) {
#pragma unroll
        for (int x = 0; x < RPEG_MAX_V; ++x) m[x] = __builtin_nan("");
      } else {
        critical_mass(cv, [&](int i) { return g_time[i * RW]; }, [&](int i) { return g_rank[i * RW]; }, m);
      }
#pragma unroll
      for (int x = 0; x < RPEG_MAX_V; ++x) L.mass[pi * RPEG_MAX_V + x] = m[x];
    }
  }
  KE_STAMP(6);
}

#endif  // __HIPCC__

}  // namespace rpeg
#endif
