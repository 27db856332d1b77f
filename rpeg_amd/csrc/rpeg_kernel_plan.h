// rpeg_kernel_plan.h - the evaluation kernel for batches too small to fill the chip with one plan per
// lane (device only): ONE PLAN PER WAVEFRONT.
//
// The lanes share the plan's work instead of each carrying a plan of its own:
//   cost model      lane = duration slot of the class (NodeCostModel.time of one node variant each)
//   memory model    lane = template vertex, then lane = vertex subset (candidate device class)
//   ranks           lane = lowered node; Jacobi rounds of rank = duration + max(rank of successors) until
//                   nothing changes (the fixed point is the reverse topological pass of scheduler.py:71-100)
//   list scheduler  lane = lowered node (NS nodes per lane).  Every node keeps its heap key, its tie-break
//                   word, the latest finish of its predecessors and the availability of the devices it
//                   reserves in registers.  The heap's pop is a minimum over the wavefront (row shifts and
//                   broadcasts, no memory); all control flow is uniform, so the loop runs on the scalar unit
//                   and the successors of the dispatched node are read from the winner lane's registers.
//
// The heap key of the reference is (est, comm_prio, topo_idx, -rank, tie).  (comm_prio, topo_idx, -rank) is
// fixed once the ranks are known, so it is replaced by the node's position in that order (equal triples get
// equal positions), packed above the tie counter in one 32-bit word: a pop is the minimum of a double and,
// among equals, of that word.
//
// Device availability: a node waits for max(avail[d]) over the devices it reserves, i.e. for the largest
// finish time of any dispatched node whose reserved vertices intersect its own.  Every lane keeps that
// maximum for its nodes and raises it at each dispatch (max is exact, so the order does not matter).
#ifndef RPEG_KERNEL_PLAN_H
#define RPEG_KERNEL_PLAN_H

#include "rpeg_kernel_eval.h"

namespace rpeg {

constexpr int KP_MAX_NS = 6;                    // nodes per lane: classes of up to 384 nodes
constexpr uint32_t KP_TIE_BITS = 23u, KP_TIE_MASK = (1u << KP_TIE_BITS) - 1u;
constexpr uint32_t KP_SKIP = 0xFFFFFFFFu;        // task -> class blob offset of a task that is skipped (offsets stay below 2^31)
constexpr int KP_PLAN_I16 = 80;                 // plan fields in LDS (60 used; pair tests may read past them)

// LDS of one wavefront: plan fields, per-vertex memory terms, durations per slot, rank / finish and start
// per node (plus one neutral element each), tie-break class per node; busy-time table and dispatch order.
__host__ __device__ inline size_t kp_lds_bytes(uint32_t nodes, uint32_t slots) {
  const size_t base = ((size_t)KP_PLAN_I16 * 2 + (size_t)RPEG_MAX_V * 4 * 8 + 8ull * slots + 16ull * (nodes + 1) + nodes + 7) & ~size_t(7);
  // then, for the utilisation: busy time by allocation set (64 doubles) and the dispatch order (2 bytes per node);
  // for the critical chain: the predecessor it follows at every node (2 bytes per node)
  return (base + 64 * 8 + 2ull * nodes + 2ull * nodes + 15) & ~size_t(15);
}

#if defined(__HIPCC__)

template <int CTRL, int ROWS>
__device__ inline int kp_dpp(int v) { return __builtin_amdgcn_update_dpp(v, v, CTRL, ROWS, 0xF, false); }

struct KpMin { __device__ double operator()(double a, double b) const { return __builtin_fmin(a, b); } };
struct KpMax { __device__ double operator()(double a, double b) const { return __builtin_fmax(a, b); } };

template <int CTRL, int ROWS, class OP>
__device__ inline double kp_step(double v, OP op) {
  const int lo = kp_dpp<CTRL, ROWS>(__double2loint(v)), hi = kp_dpp<CTRL, ROWS>(__double2hiint(v));
  return op(v, __hiloint2double(hi, lo));
}
// reduction over the 64 lanes (all must be active); the result is uniform
template <class OP>
__device__ inline double kp_wave_reduce(double v, OP op) {
  v = kp_step<0xB1, 0xF>(v, op);    // lanes 1,0,3,2 of each quad
  v = kp_step<0x4E, 0xF>(v, op);    // lanes 2,3,0,1 of each quad
  v = kp_step<0x124, 0xF>(v, op);   // row rotated by 4
  v = kp_step<0x128, 0xF>(v, op);   // row rotated by 8: every lane holds its row's result
  v = kp_step<0x142, 0xA>(v, op);   // last lane of rows 0 and 2 into rows 1 and 3
  v = kp_step<0x143, 0xC>(v, op);   // last lane of row 1 into rows 2 and 3: row 3 holds the result
  return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), 63), __builtin_amdgcn_readlane(__double2loint(v), 63));
}
// minimum of an unsigned word over the 64 lanes; the neutral element fills the lanes a step does not
// write, so that each step is one instruction (the lane move folds into the minimum)
template <int CTRL, int ROWS>
__device__ inline uint32_t kp_ustep(uint32_t v) {
  const uint32_t o = (uint32_t)__builtin_amdgcn_update_dpp((int)0xFFFFFFFFu, (int)v, CTRL, ROWS, 0xF, false);
  return o < v ? o : v;
}
__device__ inline uint32_t kp_wave_umin(uint32_t v) {
  v = kp_ustep<0xB1, 0xF>(v);
  v = kp_ustep<0x4E, 0xF>(v);
  v = kp_ustep<0x124, 0xF>(v);
  v = kp_ustep<0x128, 0xF>(v);
  v = kp_ustep<0x142, 0xA>(v);
  v = kp_ustep<0x143, 0xC>(v);
  return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
__device__ inline double kp_readlane(double v, int l) {
  return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), l), __builtin_amdgcn_readlane(__double2loint(v), l));
}
__device__ inline bool kp_is_inf(double v) {   // on the bits, so that a uniform value stays on the scalar unit
  return __double2hiint(v) == 0x7FF00000 && __double2loint(v) == 0;
}

// Ranks, tie-break classes and the list scheduler for a class of at most 64 * NS nodes.  l_rank holds the
// ranks while they are computed and the finish times afterwards; nd is the index of the neutral element.
// Returns 0, 1 on a broken class (cycle), 2 when the push counter outgrew its field (a limit of this kernel).
template <int NS, bool keep_trace>
__device__ inline int kp_schedule(const ClassView& cv, const int n, const int lane, const uint64_t ovl,
                                   const uint64_t dpne, const int nd, const double* l_dur, double* l_rank,
                                   double* l_start, uint16_t* l_order, double* l_tab,
                                   double* out_makespan, long* out_pops, unsigned long long* stamp) {
  const double inf = __builtin_inf();
  double key[NS], tm[NS], dvc[NS], dur[NS], rk[NS];
  uint32_t ord[NS], info[NS], deg[NS], sxl[NS], sxh[NS], pt[NS];
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int v = s * 64 + lane;
    const bool ok = v < n;
    const uint64_t bits = ((const uint64_t*)cv.node)[ok ? v : 0];
    NodeRec nr;
    __builtin_memcpy(&nr, &bits, 8);
    info[s] = ok ? (blocked_mask(nr, dpne) | ((uint32_t)nr.n_succ << 8) | ((uint32_t)nr.succ_begin << 16)) : 0u;
    deg[s] = ok ? (uint32_t)nr.indeg : 0xFFFFu;
    dur[s] = ok ? l_dur[nr.slot] : 0.0;
    pt[s] = nr.ptkey;
    uint32_t q[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = (ok && j < nr.n_succ) ? (uint32_t)cv.succ[nr.succ_begin + j] : (uint32_t)nd;
    sxl[s] = q[0] | (q[1] << 16);
    sxh[s] = q[2] | (q[3] << 16);
    rk[s] = dur[s];
    key[s] = inf;
    tm[s] = 0.0;
    dvc[s] = 0.0;
    if (ok) l_rank[v] = rk[s];
  }
  if (lane == 0) l_rank[nd] = l_start[nd] = 0.0;
  __syncthreads();

  // ---- ranks (scheduler.py:71-100): rounds until no rank changes, at most one per node.  A round reads the ranks of
  // the round before from one array and writes its own into the other (l_start is free until the trace is written),
  // so that one barrier per round is enough.
  {
    double* cur = l_rank;
    double* nxt = l_start;
    for (int round = 0; round <= n; ++round) {
      bool changed = false;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const double r0 = cur[sxl[s] & 0xFFFFu], r1 = cur[sxl[s] >> 16], r2 = cur[sxh[s] & 0xFFFFu], r3 = cur[sxh[s] >> 16];
        double best = 0.0;
        best = r0 > best ? r0 : best;
        best = r1 > best ? r1 : best;
        best = r2 > best ? r2 : best;
        best = r3 > best ? r3 : best;
        const int ns = (int)((info[s] >> 8) & 0xFFu), sb = (int)(info[s] >> 16);
        for (int j = 4; j < ns; ++j) {
          const double r = cur[cv.succ[sb + j]];
          best = r > best ? r : best;
        }
        const double nr_ = dur[s] + best;
        changed = changed || nr_ != rk[s];
        rk[s] = nr_;
      }
#pragma unroll
      for (int s = 0; s < NS; ++s)
        if (s * 64 + lane < n) nxt[s * 64 + lane] = rk[s];
      __syncthreads();
      double* const t = cur; cur = nxt; nxt = t;
      if (!__ballot(changed)) break;
    }
    if (cur != l_rank) {   // the fixed point, in l_rank for what follows
#pragma unroll
      for (int s = 0; s < NS; ++s)
        if (s * 64 + lane < n) l_rank[s * 64 + lane] = rk[s];
      __syncthreads();
    }
  }
  // chain inheritance (scheduler.py:367-378): the sub-nodes of one split vertex share the chain's top rank
  for (unsigned g = lane; g < cv.h->n_groups; g += KE_WAVE) {
    const GroupRec gr = cv.group[g];
    double top = l_rank[cv.gmember[gr.begin]];
    for (int j = 1; j < gr.count; ++j) {
      const double r = l_rank[cv.gmember[gr.begin + j]];
      top = r > top ? r : top;
    }
    for (int j = 0; j < gr.count; ++j) l_rank[cv.gmember[gr.begin + j]] = top;
  }
  __syncthreads();
#pragma unroll
  for (int s = 0; s < NS; ++s) rk[s] = l_rank[s * 64 + lane < n ? s * 64 + lane : nd];

  if (stamp) stamp[3] = wall_clock64();
  // ---- position of every node in the order (comm_prio * 8 + topo_idx ascending, rank descending); `shared`
  // marks the nodes whose position another node has too: only among those does a tie counter ever decide
  bool shared[NS];
  {
    // Only nodes of one tie-break class (comm_prio * 8 + topo_idx, below 16) compare ranks: the ranks are laid out
    // class by class (l_start is free until the trace is written), and every node counts within its class's stretch.
    uint32_t* l_cnt = (uint32_t*)l_tab;   // [16] members of every class, then [17] first place of every class
    uint32_t* l_beg = l_cnt + 16;
    uint32_t place[NS], eq[NS];
    if (lane < 16) l_cnt[lane] = 0u;
    __syncthreads();
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      place[s] = 0u;
      if (s * 64 + lane < n) place[s] = atomicAdd(&l_cnt[pt[s] & 15u], 1u);
    }
    __syncthreads();
    if (lane < 16) {
      const uint32_t cnt = l_cnt[lane];
      uint32_t beg = cnt;   // inclusive prefix over the 16 classes, then exclusive
      for (int d = 1; d < 16; d <<= 1) {
        const uint32_t o = (uint32_t)__shfl_up((int)beg, d, 16);
        if (lane >= d) beg += o;
      }
      beg -= cnt;
      l_beg[lane] = beg;
      if (lane == 15) l_beg[16] = beg + cnt;
    }
    __syncthreads();
#pragma unroll
    for (int s = 0; s < NS; ++s)
      if (s * 64 + lane < n) l_start[l_beg[pt[s] & 15u] + place[s]] = rk[s];
    __syncthreads();
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const bool ok = s * 64 + lane < n;
      const uint32_t b0 = ok ? l_beg[pt[s] & 15u] : 0u, b1 = ok ? l_beg[(pt[s] & 15u) + 1u] : 0u;
      uint32_t before = 0u, same = 0u;
      uint32_t j = b0;
      for (; j + 4u <= b1; j += 4u) {   // four independent LDS reads in flight
        const double r0 = l_start[j], r1 = l_start[j + 1], r2 = l_start[j + 2], r3 = l_start[j + 3];
        before += (r0 > rk[s] ? 1u : 0u) + (r1 > rk[s] ? 1u : 0u) + (r2 > rk[s] ? 1u : 0u) + (r3 > rk[s] ? 1u : 0u);
        same += (r0 == rk[s] ? 1u : 0u) + (r1 == rk[s] ? 1u : 0u) + (r2 == rk[s] ? 1u : 0u) + (r3 == rk[s] ? 1u : 0u);
      }
      for (; j < b1; ++j) {
        const double ru = l_start[j];
        before += ru > rk[s] ? 1u : 0u;
        same += ru == rk[s] ? 1u : 0u;
      }
      ord[s] = b0 + before;
      eq[s] = same;
    }
    __syncthreads();   // (l_start is the trace's from here on)
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      ord[s] <<= KP_TIE_BITS;
      shared[s] = eq[s] > 1u;
      // pt[s] from here on: the vertices whose allocations overlap one this node reserves.  The overlap relation
      // is symmetric, so a dispatched node D delays node s exactly when D's reserved set meets this mask.
      uint32_t touch = 0u;
#pragma unroll
      for (int x = 0; x < RPEG_MAX_V; ++x)
        if ((info[s] >> x) & 1u) touch |= mask_row(ovl, x);
      pt[s] = touch;
    }
  }
  __syncthreads();   // l_rank is reused for the finish times from here on
  if (stamp) stamp[4] = wall_clock64();

  // ---- list scheduling (scheduler.py:399-546)
  uint32_t ctr = 0;
  for (unsigned i = 0; i < cv.h->n_init; ++i) {
    const int v = __builtin_amdgcn_readfirstlane((int)cv.init[i]);
#pragma unroll
    for (int s = 0; s < NS; ++s)
      if (s == (v >> 6) && lane == (v & 63)) {
        key[s] = 0.0;
        ord[s] |= ctr;
      }
    ++ctr;
  }
  double makespan = 0.0;
  int done = 0;
  bool ok = true;
  // the trace (start and finish of every node) stays in registers while the loop runs where there is room for it
  constexpr bool trace_regs = keep_trace && NS <= 4;
  double t_fin[trace_regs ? NS : 1], t_start[trace_regs ? NS : 1];
  uint32_t pops = 0, slow_decisions = 0;
  const uint32_t guard_max = (uint32_t)n * (uint32_t)n + 64u;   // (at most 384 nodes)
  uint32_t guard = 0;
  for (;;) {
    if (done >= n) break;
    if (guard >= guard_max) break;
    ++guard;
    ++pops;
    // ---- One decision of the heap: the pops up to the next dispatch.  The heap pops stale entries (key below
    // the true start time, because the node's devices are busy) in key order and pushes each back with its
    // true time and a fresh tie, until the minimum is current.  That entry D is the minimum of (true time,
    // position, tie); the entries pushed back on the way are exactly the stale ones whose old key is below
    // D's final key.  When D is alone with its (true time, position) and no other waiting entry has its
    // position, no tie counter decides which entry D is and the whole decision is taken at once; otherwise
    // the pops are replayed one by one.
    int wl, ws;
    double gk;
    bool slow;
    {
      double e[NS];
#pragma unroll
      for (int s = 0; s < NS; ++s) e[s] = dvc[s] > key[s] ? dvc[s] : key[s];
      double be = e[0];
      uint32_t bo = ord[0] >> KP_TIE_BITS;
      int bs = 0;
#pragma unroll
      for (int s = 1; s < NS; ++s) {
        const uint32_t o = ord[s] >> KP_TIE_BITS;
        const bool lt = (e[s] < be) | ((e[s] == be) & (o < bo));
        be = lt ? e[s] : be;
        bo = lt ? o : bo;
        bs = lt ? s : bs;
      }
      const uint32_t ehi = (uint32_t)__double2hiint(be), elo = (uint32_t)__double2loint(be);
      const uint32_t ghi = kp_wave_umin(ehi);
      if (ghi >= 0x7FF00000u) { ok = false; break; }   // nothing is ready: cycle (scheduler.py:548-550)
      bool cand = ehi == ghi;
      unsigned long long m = __ballot(cand);
      if (__builtin_popcountll(m) > 1) {
        // Lanes that agree in the high word nearly always hold the same time exactly (nodes released by one
        // finish, or waiting for one device): then the low words need no reduction of their own.
        const uint32_t lo0 = (uint32_t)__builtin_amdgcn_readlane((int)elo, __builtin_ctzll(m));
        // (ballots of single comparisons, combined on the scalar unit: every lane is active here)
        if ((m & __ballot(elo != lo0)) != 0ull) {
          const uint32_t glo = kp_wave_umin(cand ? elo : 0xFFFFFFFFu);
          cand = cand && elo == glo;
          m &= __ballot(elo == glo);
        }
        if (__builtin_popcountll(m) > 1) {
          const uint32_t go_ = kp_wave_umin(cand ? bo : 0xFFFFFFFFu);
          m &= __ballot(bo == go_);
        }
      }
      wl = __builtin_ctzll(m);
      ws = __builtin_amdgcn_readlane(bs, wl);
      gk = __hiloint2double((int)ghi, __builtin_amdgcn_readlane((int)elo, wl));
      const uint32_t go = (uint32_t)__builtin_amdgcn_readlane((int)bo, wl);
      bool other = false, in_r[NS];
      uint32_t n_shared = 0;
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const uint32_t o = ord[s] >> KP_TIE_BITS;
        const bool is_d = (lane == wl) & (s == ws);
        other = other | ((key[s] < inf) & (o == go) & !is_d);
        in_r[s] = (dvc[s] > key[s]) & ((key[s] < gk) | ((key[s] == gk) & (o < go)));
        n_shared += (in_r[s] & shared[s]) ? 1u : 0u;
      }
      slow = __builtin_popcountll(m) > 1 || __ballot(other) != 0ull;
      if (!slow) {
        // Fresh ties of the entries pushed back: the heap hands them out in pop order, i.e. in the order of
        // the old keys.  Entries that share their position with no other node never compare ties and take
        // any fresh value; two or more entries with shared positions are ranked among themselves first.
        uint32_t rank[NS], total = 1u;
#pragma unroll
        for (int s = 0; s < NS; ++s) rank[s] = 0u;
        const unsigned long long ms = __ballot(n_shared > 0u);
        if (__builtin_popcountll(ms) > 1 || __ballot(n_shared > 1u) != 0ull) {
          total = 0u;
#pragma unroll
          for (int s = 0; s < NS; ++s) {
            unsigned long long members = __ballot(in_r[s] & shared[s]);
            total += (uint32_t)__builtin_popcountll(members);
            while (members) {
              const int j = __builtin_ctzll(members);
              members &= members - 1ull;
              const double kj = kp_readlane(key[s], j);
              const uint32_t oj = (uint32_t)__builtin_amdgcn_readlane((int)ord[s], j);
#pragma unroll
              for (int t = 0; t < NS; ++t) rank[t] += ((kj < key[t]) | ((kj == key[t]) & (oj < ord[t]))) ? 1u : 0u;
            }
          }
        }
#pragma unroll
        for (int s = 0; s < NS; ++s)
          if (in_r[s]) {
            key[s] = dvc[s];
            ord[s] = (ord[s] & ~KP_TIE_MASK) | (ctr + rank[s]);
          }
        ctr += total;
      }
    }
    if (slow) {
      ++slow_decisions;
      for (;;) {
        // the heap's minimum: smallest key, among equals the smallest tie-break word.  Keys are non-negative
        // doubles or +inf, so they order like their bit patterns: the minimum is taken on the high words,
        // then (only if lanes still tie) on the low words, then on the tie-break words.
        double bk = key[0];
        uint32_t bo = ord[0];
        int bs = 0;
#pragma unroll
        for (int s = 1; s < NS; ++s) {
          const bool lt = (key[s] < bk) | ((key[s] == bk) & (ord[s] < bo));
          bk = lt ? key[s] : bk;
          bo = lt ? ord[s] : bo;
          bs = lt ? s : bs;
        }
        const uint32_t khi = (uint32_t)__double2hiint(bk), klo = (uint32_t)__double2loint(bk);
        const uint32_t ghi = kp_wave_umin(khi);
        bool cand = khi == ghi;
        unsigned long long m = __ballot(cand);
        if (__builtin_popcountll(m) > 1) {
          const uint32_t glo = kp_wave_umin(cand ? klo : 0xFFFFFFFFu);
          cand = cand && klo == glo;
          m = __ballot(cand);
          if (__builtin_popcountll(m) > 1) {
            const uint32_t go_ = kp_wave_umin(cand ? bo : 0xFFFFFFFFu);
            m = __ballot(cand && bo == go_);
          }
        }
        wl = __builtin_ctzll(m);
        gk = __hiloint2double((int)ghi, __builtin_amdgcn_readlane((int)klo, wl));
        ws = __builtin_amdgcn_readlane(bs, wl);
        // stale: push back with the true time and a fresh tie (scheduler.py:437-443)
        double wdv = dvc[0];
#pragma unroll
        for (int s = 1; s < NS; ++s) wdv = s == ws ? dvc[s] : wdv;
        if (!__ballot(lane == wl && wdv > gk)) break;
#pragma unroll
        for (int s = 0; s < NS; ++s)
          if (lane == wl && s == ws) {
            key[s] = dvc[s];
            ord[s] = (ord[s] & ~KP_TIE_MASK) | ctr;
          }
        ++ctr;
        ++pops;
        if (++guard >= guard_max) break;
      }
      if (guard >= guard_max) break;
    }
    const bool mine = lane == wl;
    // ---- dispatch node ws * 64 + wl at gk
    double wdur = dur[0];
    uint32_t winfo = info[0], wsl = sxl[0], wsh = sxh[0];
#pragma unroll
    for (int s = 1; s < NS; ++s) {
      wdur = s == ws ? dur[s] : wdur;
      winfo = s == ws ? info[s] : winfo;
      wsl = s == ws ? sxl[s] : wsl;
      wsh = s == ws ? sxh[s] : wsh;
    }
    const double d = kp_readlane(wdur, wl);
    const uint32_t binfo = (uint32_t)__builtin_amdgcn_readlane((int)winfo, wl);
    const uint32_t s01 = (uint32_t)__builtin_amdgcn_readlane((int)wsl, wl), s23 = (uint32_t)__builtin_amdgcn_readlane((int)wsh, wl);
    const double fin = gk + d;
    makespan = fin > makespan ? fin : makespan;
    ++done;
    const uint32_t reserved = binfo & 0xFFu;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const bool hit = (pt[s] & reserved) != 0u;
      dvc[s] = hit && fin > dvc[s] ? fin : dvc[s];
      if (mine && s == ws) key[s] = inf;
    }
    if (trace_regs) {
#pragma unroll
      for (int s = 0; s < NS; ++s) {
        const bool here = mine && s == ws;
        t_fin[trace_regs ? s : 0] = here ? fin : t_fin[trace_regs ? s : 0];
        t_start[trace_regs ? s : 0] = here ? gk : t_start[trace_regs ? s : 0];
      }
      if (l_order && mine) l_order[done - 1] = (uint16_t)(ws * 64 + wl);
    } else if (keep_trace && mine) {
      l_rank[ws * 64 + wl] = fin;
      l_start[ws * 64 + wl] = gk;
      if (l_order) l_order[done - 1] = (uint16_t)(ws * 64 + wl);
    }
    // successors in adjacency order; a node whose last predecessor this was becomes ready
    const int ns = (int)((binfo >> 8) & 0xFFu), sb = (int)(binfo >> 16);
    for (int j = 0; j < ns; ++j) {
      int wn;
      if (j < 4) wn = (int)(((j < 2 ? s01 : s23) >> ((j & 1) * 16)) & 0xFFFFu);
      else wn = __builtin_amdgcn_readfirstlane((int)cv.succ[sb + j]);
      const bool me = lane == (wn & 63);
#pragma unroll
      for (int s = 0; s < NS; ++s)
        if (me && (NS == 1 || s == (wn >> 6))) {   // (a successor is a node of the class: below 64 when NS is 1)
          tm[s] = fin > tm[s] ? fin : tm[s];
          deg[s] -= 1u;
          if (deg[s] == 0u) {
            key[s] = dvc[s] > tm[s] ? dvc[s] : tm[s];
            ord[s] |= ctr;
          }
        }
      ++ctr;
    }
  }
  if (done != n) ok = false;
  if (trace_regs && ok) {
#pragma unroll
    for (int s = 0; s < NS; ++s)
      if (s * 64 + lane < n) {
        l_rank[s * 64 + lane] = t_fin[trace_regs ? s : 0];
        l_start[s * 64 + lane] = t_start[trace_regs ? s : 0];
      }
  }
  *out_makespan = makespan;
  *out_pops = ((long)slow_decisions << 20) | (long)pops;
  if (ctr > KP_TIE_MASK) return 2;   // the push counter outgrew its field of the packed order: a limit of this kernel
  return ok ? 0 : 1;
}

// Critical-chain mass per template vertex (critical_mass of rpeg_class.h; moves.py:590-642) for one plan per
// wavefront.  What the walk needs at a node -- the predecessor it goes on to (the first one, in edge order, of largest
// finish time) and the vertex the node counts for -- is found for all nodes at once, a node per lane, and left in
// LDS; the walk itself, one hop after the other from the first node of largest finish time, then reads LDS only.
// Lane x < RPEG_MAX_V returns the mass of vertex x, summed in the order of the walk.
__device__ inline double kp_critical_mass(const ClassView& cv, const int n, const int lane, const double* l_fin,
                                          const double* l_start, uint16_t* l_next, uint8_t* l_vx) {
  double bf = -1.0;
  uint32_t bi = 0xFFFFFFFFu;
  for (int v = lane; v < n; v += KE_WAVE) {
    const double f = l_fin[v];
    if (f > bf) { bf = f; bi = (uint32_t)v; }
    const int pb = cv.pbeg[v], pe = cv.pbeg[v + 1];
    uint32_t nx = 0xFFFFu;
    if (pb != pe) {
      nx = cv.pred[pb];
      double b = l_fin[nx];
      for (int j = pb + 1; j < pe; ++j) {
        const uint32_t q = cv.pred[j];
        const double fq = l_fin[q];
        if (fq > b) { b = fq; nx = q; }
      }
    }
    l_next[v] = (uint16_t)nx;
    const SlotDesc sd = cv.slot[cv.node[v].slot];
    l_vx[v] = sd.type <= SLOT_OP_SUB ? sd.a : (uint8_t)0xFF;
  }
  __syncthreads();
  const double top = kp_wave_reduce(bf, KpMax());
  int cur = (int)kp_wave_umin(bf == top ? bi : 0xFFFFFFFFu);
  double m = 0.0;
  for (int hops = 0; hops <= n; ++hops) {   // a chain visits a node at most once
    const int vx = l_vx[cur];
    const double d = l_fin[cur] - l_start[cur];
    const int nx = __builtin_amdgcn_readfirstlane((int)l_next[cur]);
    if (lane == vx) m += d;
    if (nx == 0xFFFF) break;
    cur = nx;
  }
  return m;
}

// Pair relations and vertex sets of one plan by POSITION in the order of first appearance (bit 8i+j of a
// 64-bit word: positions i and j; bit i of a 32-bit word: position i).
struct KpOrdered {
  unsigned long long ovl, eq, same_model, train_same;
  unsigned train, trainable;
  bool coresident;
};
__device__ inline unsigned kp_row(unsigned long long m, int i) { return (unsigned)(m >> (8 * i)) & 0xFFu; }

__device__ inline bool kp_maximal_clique(int nv, unsigned long long ovl, unsigned M) {
  bool clique = true, maximal = true;
#pragma unroll
  for (int i = 0; i < RPEG_MAX_V; ++i) {
    if (i >= nv) break;
    const bool in = (M >> i) & 1u;
    const bool fits = (M & ~kp_row(ovl, i)) == 0;
    clique = clique && !(in && !fits);
    maximal = maximal && !(!in && fits);
  }
  return clique && maximal;
}

// device_class_peak of rpeg_core.h on position-indexed masks; vm[i * 4 + f] holds w_shard, mem_w, opt and
// extra of the vertex at position i.  M is uniform, so is the control flow; every loop runs over the
// compile-time bound and nothing is indexed dynamically.
__device__ inline double kp_class_peak(const rpeg_problem_t& P, const rpeg_struct_t& st, const uint8_t* order, int nv,
                                       const KpOrdered& om, const double* vm, unsigned M) {
  double persistent = 0.0;
  int groups = 0;
#pragma unroll
  for (int i = 0; i < RPEG_MAX_V; ++i) {   // distinct (model, allocation) worker keys
    if (!((M >> i) & 1u)) continue;
    if ((kp_row(om.eq, i) & M & kp_row(om.same_model, i) & ((1u << i) - 1u)) == 0) ++groups;
  }
  if (om.coresident) {   // the co-resident sum model, as in device_class_peak (vm[i * 4 + 2] carries dp)
    double stat = 0.0, transient = 0.0;
#pragma unroll
    for (int i = 0; i < RPEG_MAX_V; ++i) {
      if (!((M >> i) & 1u)) continue;
      transient = dmax(transient, vm[i * 4 + 3]);
      const unsigned same = M & kp_row(om.same_model, i);
      if (same & ((1u << i) - 1u)) continue;
      double wmax = 0.0, dp = vm[i * 4 + 2];
      bool trained = false;
#pragma unroll
      for (int q = 0; q < RPEG_MAX_V; ++q) {
        if (!((same >> q) & 1u)) continue;
        wmax = dmax(wmax, vm[q * 4 + 0]);
        if ((om.train >> q) & 1u) { trained = true; dp = vm[q * 4 + 2]; }
      }
      const double sbw = (double)P.model[st.vertex[order[i]].model].sb * wmax;
      double x = sbw;
      if (trained) x = (sbw + 12.0 * wmax / (P.optimizer_stage >= 1 ? dp : 1.0)) + sbw / (P.optimizer_stage >= 2 ? dp : 1.0);
      stat += x;
    }
    double peak = ((double)groups * P.group_overhead + stat) + transient;
    if (P.max_groups > 0 && groups > P.max_groups) peak = __builtin_inf();
    return peak;
  }
#pragma unroll
  for (int i = 0; i < RPEG_MAX_V; ++i)     // optimizer shards of the training vertices
    if (((M & om.train & om.trainable) >> i) & 1u) persistent += vm[i * 4 + 2];
  unsigned serving = 0;                    // serving shards: one per worker key that is not a training worker
#pragma unroll
  for (int i = 0; i < RPEG_MAX_V; ++i) {
    if (!(((M & om.trainable & ~om.train) >> i) & 1u)) continue;
    const unsigned same_key = kp_row(om.eq, i) & M & kp_row(om.same_model, i);
    if (same_key & kp_row(om.train_same, i)) continue;
    const bool first = (same_key & serving) == 0;
    serving |= 1u << i;
    if (!first) continue;
    double ws = 0.0;
#pragma unroll
    for (int q = 0; q < RPEG_MAX_V; ++q)
      if (((same_key & ~om.train) >> q) & 1u) ws = dmax(ws, vm[q * 4 + 0]);
    persistent += (double)P.model[st.vertex[order[i]].model].sb * ws;
  }
#pragma unroll
  for (int i = 0; i < RPEG_MAX_V; ++i) {   // frozen weights: one entry per model, its largest shard
    if (!(((M & ~om.trainable) >> i) & 1u)) continue;
    const unsigned same = M & kp_row(om.same_model, i);
    if (same & ((1u << i) - 1u)) continue;
    double wb = 0.0;
#pragma unroll
    for (int q = 0; q < RPEG_MAX_V; ++q)
      if ((same >> q) & 1u) wb = dmax(wb, vm[q * 4 + 1]);
    persistent += wb;
  }
  double top = 0.0;
#pragma unroll
  for (int i = 0; i < RPEG_MAX_V; ++i) {
    if (!((M >> i) & 1u)) continue;
    const bool resident = !((om.trainable >> i) & 1u) || (kp_row(om.eq, i) & serving & kp_row(om.same_model, i)) != 0;
    const double c = resident ? vm[i * 4 + 3] : vm[i * 4 + 1] + vm[i * 4 + 3];
    top = dmax(top, c);
  }
  double peak = (double)groups * P.group_overhead + persistent + top;
  if (P.max_groups > 0 && groups > P.max_groups) peak = __builtin_inf();   // memory.py:699-704
  (void)nv;
  return peak;
}

// Trace.utilization() (RPEG/schedule/trace.py:53-101) of the plan just scheduled: the mean over the devices that
// any node reserved of busy time / makespan, where a device's busy time is the measure of the union of the
// (start, finish) spans of the nodes whose reserved allocations hold it, merged in sorted order, and the mean is
// a running sum over the devices in the order in which the trace first met them (dispatch order of the nodes;
// within a node the source allocation before the destination; within an allocation rack-major) divided by
// their number.  The additions are done in exactly that order: the result equals the reference's bit for bit.
//
// All devices held by the same set of vertex allocations have the same spans, so the busy time is computed once
// per set (lane m takes the set with bit pattern m) over the nodes in dispatch order -- on one device that is
// the sorted order, because a node starts no earlier than the nodes dispatched before it on its devices ended.
// Then the vertices are taken in the order of their first reservation, and the devices of each allocation that
// no earlier one holds are added 64 at a time: the lanes find set and value of their device, one running sum
// takes the values in lane order.  l_start / l_fin: per node; l_order: node dispatched k-th; l_tab: 64 doubles.
__device__ inline double kp_utilization(const ClassView& cv, const int n, const int lane, const int nv, const int16_t* l_plan,
                                        const uint64_t dpne, const double* l_start, const double* l_fin,
                                        const uint16_t* l_order, double* l_tab, const double ms) {
  if (!(ms > 0.0) || n == 0) return 0.0;
  {
    const unsigned mine = (unsigned)lane;
    double merged = 0.0, cs = 0.0, ce = 0.0;
    bool open = false;
    for (int k = 0; k < n; ++k) {
      const int i = (int)l_order[k];
      const uint64_t bits = ((const uint64_t*)cv.node)[i];
      NodeRec nr;
      __builtin_memcpy(&nr, &bits, 8);
      const unsigned b = blocked_mask(nr, dpne);
      const double s = l_start[i], f = l_fin[i];
      if (b & mine) {
        if (!open || s > ce) {
          if (open) merged += ce - cs;
          cs = s;
          ce = f;
          open = true;
        } else {
          ce = f > ce ? f : ce;
        }
      }
    }
    if (open) merged += ce - cs;
    l_tab[lane] = merged / ms;
  }
  __syncthreads();
  // vertices by first reservation, four bits each
  uint32_t order = 0u;
  int n_ev = 0;
  {
    unsigned seen = 0u;
    for (int k = 0; k < n && n_ev < nv; ++k) {
      const int i = __builtin_amdgcn_readfirstlane((int)l_order[k]);
      const uint64_t bits = ((const uint64_t*)cv.node)[i];
      NodeRec nr;
      __builtin_memcpy(&nr, &bits, 8);
      unsigned b = blocked_mask(nr, dpne) & ~seen;
      if (nr.cond) {   // a transfer: source before destination
        const unsigned src = (nr.cond - 1u) >> 3;
        if ((b >> src) & 1u) {
          order |= src << (4 * n_ev);
          ++n_ev;
          seen |= 1u << src;
          b &= ~(1u << src);
        }
      }
      while (b) {
        const unsigned v = (unsigned)__builtin_ctz(b);
        b &= b - 1u;
        order |= v << (4 * n_ev);
        ++n_ev;
        seen |= 1u << v;
      }
    }
  }
  double total = 0.0;
  int count = 0;
  unsigned earlier = 0u;
  for (int e = 0; e < n_ev; ++e) {
    const int v = (int)((order >> (4 * e)) & 15u);
    const int16_t* bx = l_plan + v * RPEG_FIELDS;
    const int ro = bx[4], qo = bx[5], go = bx[6], re = bx[7], qe = bx[8], ge = bx[9];
    const uint32_t ng = (uint32_t)(qe * ge), cnt = (uint32_t)re * ng;
    const uint32_t m_ng = 0xFFFFFFFFu / ng + 1u, m_g = 0xFFFFFFFFu / (uint32_t)ge + 1u;   // exact quotients below 2^16
    for (uint32_t base = 0; base < cnt; base += 64u) {
      const uint32_t idx = base + (uint32_t)lane;
      const uint32_t r = ng == 1u ? idx : __umulhi(idx, m_ng);
      const uint32_t rem = idx - r * ng;
      const uint32_t q = ge == 1 ? rem : __umulhi(rem, m_g);
      const int R = ro + (int)r, Q = qo + (int)q, G = go + (int)(rem - q * (uint32_t)ge);
      unsigned M = 0u;
#pragma unroll
      for (int x = 0; x < RPEG_MAX_V; ++x) {
        const int16_t* p = l_plan + x * RPEG_FIELDS;
        const bool in = x < nv && R >= p[4] && R < p[4] + p[7] && Q >= p[5] && Q < p[5] + p[8] && G >= p[6] && G < p[6] + p[9];
        M |= in ? 1u << x : 0u;
      }
      const double val = l_tab[M & 63u];
      unsigned long long fresh = __ballot(idx < cnt && (M & earlier) == 0u);
      count += (int)__builtin_popcountll(fresh);
      while (fresh) {
        const int j = __builtin_ctzll(fresh);
        fresh &= fresh - 1ull;
        total += kp_readlane(val, j);
      }
    }
    earlier |= 1u << v;
  }
  return count ? total / (double)count : 0.0;
}

// One plan, evaluated by the whole wavefront.  pi: plan index (uniform).
__device__ inline void kp_eval_plan(const EvalLaunch& L, const uint64_t w, const uint64_t pi, const ClassView cv,
                                    uint8_t* lds) {
  const int lane = threadIdx.x;
  const rpeg_problem_t& P = *L.P;
  const int n = (int)cv.h->n_nodes, n_slots = (int)cv.h->n_slots;
  const int nd = (int)L.ws_nodes;
  int first_lane = 0;
  (void)first_lane;

  int16_t* l_plan = (int16_t*)lds;
  double* l_vm = (double*)(lds + KP_PLAN_I16 * 2);
  double* l_dur = l_vm + RPEG_MAX_V * 4;
  double* l_rank = l_dur + L.ws_slots;
  double* l_start = l_rank + (L.ws_nodes + 1);
  uint8_t* l_pt = (uint8_t*)(l_start + (L.ws_nodes + 1));
  double* l_tab = (double*)(((uintptr_t)(l_pt + L.ws_nodes) + 7) & ~(uintptr_t)7);
  uint16_t* l_ord = (uint16_t*)(l_tab + 64);
  uint16_t* l_next = l_ord + L.ws_nodes;

  __syncthreads();   // the previous plan of this wavefront is done with LDS
  KE_STAMP(0);
  const rpeg_struct_t& st = P.st[cv.h->structure];
  const int nv = st.n_vertex;
  PlanMasks pm;
  pm.ovl = pm.eq = pm.dpne = 0;
  bool err = cv.h->error != 0, limit = false, stale_ok = false, mem_ok = false;
  double peak = -1.0, pen = 1.0;
  if (L.dur) {
    // a task of a laid-out batch: the prologue launches have left the durations of the slot universe, the pair
    // relations, the penalty factor and the gate bits by plan index (and written the peak themselves)
    const uint64_t sp = pi;
    bool bad = false;
    for (int s = lane; s < n_slots; s += KE_WAVE) {
      const double d = L.dur[(size_t)cv.umap[s] * L.dur_stride + sp];
      l_dur[s] = d;
      bad = bad || d != d;
    }
    err = err || __ballot(bad) != 0ull;
    pm.ovl = L.aux_ovl[sp];
    pm.dpne = L.aux_dpne[sp];
    pen = L.aux_pen ? L.aux_pen[sp] : 1.0;
    const uint8_t gates = L.aux_mask ? L.aux_mask[sp] : (uint8_t)(RPEG_MASK_VALID | RPEG_MASK_STALE_OK | RPEG_MASK_MEM_OK);
    stale_ok = (gates & RPEG_MASK_STALE_OK) != 0;
    mem_ok = (gates & RPEG_MASK_MEM_OK) != 0;
    __syncthreads();
    KE_STAMP(1);
    KE_STAMP(2);
  } else {
    const PlanHead h = load_head(L.head, L.stride, pi);
    if (lane < KP_PLAN_I16) l_plan[lane] = lane < nv * RPEG_FIELDS ? L.vert[(uint64_t)lane * L.stride + pi] : (int16_t)1;
    __syncthreads();

    // ---- pair relations: lane 8u+v tests vertices u and v, the ballots are the masks
    {
      const int u = lane >> 3, v = lane & 7;
      const bool valid = u < nv && v < nv;
      const VPlan au = ke_vplan<1>(l_plan, valid ? u : 0), av = ke_vplan<1>(l_plan, valid ? v : 0);
      pm.ovl = __ballot(valid && !alloc_disjoint(au, av));
      pm.eq = 0;   // the memory model below works on position-indexed masks of its own
      pm.dpne = __ballot(valid && au.dp != av.dp);
    }
    KE_STAMP(1);

    // ---- durations of the class's slots, one slot per lane
    bool zero_div = false;
    const int split = (int)cv.h->split;
    for (int s = lane; s < n_slots; s += KE_WAVE) l_dur[s] = ke_slot_duration<1>(P, st, split, cv.slot[s], l_plan, &zero_div);
    err = err || __ballot(zero_div) != 0ull;
    KE_STAMP(2);

    // ---- memory model (memory.py:608-841), in the order of first appearance of the vertices among the
    // lowered operator nodes (position i = vertex vorder[i]): that order fixes the order of the float sums.
    // One vertex per lane, then one vertex subset per lane tests whether it is a device class (a maximal clique
    // of the overlap graph); the few that are get evaluated one after the other with uniform control flow.
    const uint8_t* order = cv.h->vorder;
    const bool coresident = struct_coresident(st);
    if (lane < nv) {
      const int v = order[lane];
      const VMem m = vertex_memory(P, st.vertex[v], ke_vplan<1>(l_plan, v), coresident);
      l_vm[lane * 4 + 0] = (double)m.w_shard;
      l_vm[lane * 4 + 1] = m.mem_w;
      l_vm[lane * 4 + 2] = m.opt;
      l_vm[lane * 4 + 3] = m.extra;
    }
    KpOrdered om;
    {
      const int i = lane >> 3, j = lane & 7;
      const bool valid = i < nv && j < nv;
      const int vi = order[valid ? i : 0], vj = order[valid ? j : 0];
      const VPlan ai = ke_vplan<1>(l_plan, vi), aj = ke_vplan<1>(l_plan, vj);
      const rpeg_vertex_t &xi = st.vertex[vi], &xj = st.vertex[vj];
      om.ovl = __ballot(valid && !alloc_disjoint(ai, aj));
      om.eq = __ballot(valid && alloc_equal(ai, aj));
      om.same_model = __ballot(valid && xi.model == xj.model);
      om.train_same = __ballot(valid && xi.model == xj.model && xj.role == RPEG_ROLE_TRAIN);
      const unsigned long long t = __ballot(valid && j == 0 && xi.role == RPEG_ROLE_TRAIN),
                               tr = __ballot(valid && j == 0 && st.mem_trainable[xi.model] != 0);   // bit 8i: position i
      om.train = om.trainable = 0u;
      om.coresident = coresident;
#pragma unroll
      for (int q = 0; q < RPEG_MAX_V; ++q) {
        om.train |= (unsigned)((t >> (8 * q)) & 1ull) << q;
        om.trainable |= (unsigned)((tr >> (8 * q)) & 1ull) << q;
      }
    }
    __syncthreads();
    {
      const unsigned M = (unsigned)lane + 1u;
      unsigned long long classes = __ballot(M < (1u << nv) && kp_maximal_clique(nv, om.ovl, M));
      while (classes) {
        const unsigned Mu = (unsigned)__builtin_ctzll(classes) + 1u;
        classes &= classes - 1ull;
        const double p = kp_class_peak(P, st, order, nv, om, l_vm, Mu);
        peak = p > peak ? p : peak;
      }
    }
    stale_ok = stale_layout_ok(st, h, pm.ovl);
    mem_ok = !(peak > P.cap);
    if (!mem_ok) pen = oom_penalty(peak, P.cap);
  }
  KE_STAMP(3);
  unsigned long long* stamp = L.prof && lane == 0 ? L.prof + w * 8 : nullptr;

  // ---- ranks and list scheduling
  double makespan = 0.0;
  long pops = 0;
  const bool keep = L.mass != nullptr || L.util != nullptr;
  uint16_t* const l_order = L.util ? l_ord : nullptr;
  if (!err) {
    int ok;
    // (the trace of start and finish times is compiled out where no output needs it: its flags and pointers would
    // otherwise be carried through the scheduling loop)
#define KP_SCHEDULE(NS) (keep ? kp_schedule<NS, true>(cv, n, lane, pm.ovl, pm.dpne, nd, l_dur, l_rank, l_start, l_order, l_tab, &makespan, &pops, stamp) \
                              : kp_schedule<NS, false>(cv, n, lane, pm.ovl, pm.dpne, nd, l_dur, l_rank, l_start, nullptr, l_tab, &makespan, &pops, stamp))
    if (n <= 64) ok = KP_SCHEDULE(1);
    else if (n <= 128) ok = KP_SCHEDULE(2);
    else if (n <= 192) ok = KP_SCHEDULE(3);
    else if (n <= 256) ok = KP_SCHEDULE(4);
    else if (n <= 320) ok = KP_SCHEDULE(5);
    else ok = KP_SCHEDULE(6);
#undef KP_SCHEDULE
    err = ok != 0;
    limit = ok == 2;
  }
  KE_STAMP(5);
  if (L.prof && lane == 0) L.prof[w * 8 + 7] = ((unsigned long long)n << 32) | (unsigned long long)pops;

  // ---- outputs
  uint8_t mask = RPEG_MASK_VALID;
  if (stale_ok) mask |= RPEG_MASK_STALE_OK;
  if (mem_ok) mask |= RPEG_MASK_MEM_OK;
  double out_makespan, out_score;
  if (err || makespan == 0.0) {
    out_makespan = out_score = __builtin_nan("");
    mask |= RPEG_MASK_ERROR;
    if (limit) mask |= RPEG_MASK_LIMIT;
  } else {
    double score = P.score_num / makespan;
    if (!mem_ok) score = score * pen;
    if ((L.flags & RPEG_GATE_STALE) && !stale_ok) score = 0.0;
    out_makespan = makespan;
    out_score = score;
  }
  double m = __builtin_nan("");   // lane x < RPEG_MAX_V: mass of vertex x
  if (L.mass) {
    __syncthreads();
    if (!err) m = kp_critical_mass(cv, n, lane, l_rank, l_start, l_next, l_pt);
  }
  double util = 0.0;
  if (L.util) {
    __syncthreads();
    util = err ? __builtin_nan("") : kp_utilization(cv, n, lane, nv, l_plan, pm.dpne, l_start, l_rank, l_ord, l_tab, makespan);
  }
  if (lane == 0) {
    if (L.util) L.util[pi] = util;
    if (L.makespan) L.makespan[pi] = out_makespan;
    if (L.peak && !L.dur) L.peak[pi] = peak;   // (with a prologue launch the peak is that launch's output)
    if (L.score) L.score[pi] = out_score;
    if (L.mask) L.mask[pi] = mask;
  }
  if (L.mass && lane < RPEG_MAX_V) L.mass[pi * RPEG_MAX_V + lane] = m;
  KE_STAMP(6);
}

#endif  // __HIPCC__

}  // namespace rpeg
#endif
