// rpeg_kernel_eval.h - the batch evaluation kernel (device only).
//
// One wavefront evaluates up to 64 plans of ONE lowering class, one plan per lane.
//
// Memory placement, chosen for the latency of the list scheduler's dependent accesses:
//   LDS   class tables (node records, successor lists): read with per-lane node indices
//         one area [row][lane] that holds, one after the other, the plan fields (int16, read by the cost
//         model), the per-vertex memory terms and the ready list: key (est) and a meta word (node, tie-break
//         class, reserved vertices) per entry.  The arg-min scan, the stale-key update and the removal never
//         leave LDS.
//   HBM   (LS = 0) per-plan arrays in a workspace, one block per wavefront, interleaved by lane
//         (array[row][lane]): ready time and rank per node, duration per slot, remaining in-degree per node.
//         The 64 plans of a wavefront belong to one class and mostly dispatch the same node at the same
//         moment, so their accesses fall into one 512-byte row (a contiguous block per lane made every
//         access touch 64 cache lines: 3.4 times the HBM traffic on GRPO graphs, 1.5 times the run time on
//         DPO graphs).  A scheduling step issues all of its loads (duration of the dispatched node; ready
//         time, in-degree and rank of up to four successors) before it waits.
//         With LS > 0 the same arrays sit in LDS, interleaved by lane.
#ifndef RPEG_KERNEL_EVAL_H
#define RPEG_KERNEL_EVAL_H

#include <type_traits>

#include "rpeg_plan.h"

namespace rpeg {

constexpr int KE_WAVE = 64;
constexpr uint32_t KE_IDLE = 0xFFFFFFFFu;
constexpr uint32_t KE_CLS_LDS = 0x80000000u;   // flag in EvalLaunch::wave_cls
constexpr int KE_FEW = 8;                      // plans of a wavefront so flagged

struct EvalLaunch {              // uniform launch parameters
  const rpeg_problem_t* P;
  const int16_t* vert;
  const uint8_t* head;
  uint64_t stride;
  const uint32_t* perm;          // lane -> plan index, KE_IDLE for padding lanes
  const uint32_t* wave_cls;      // wavefront -> class blob offset; KE_CLS_LDS set: few plans, state in LDS
  const uint8_t* pool;
  uint8_t* ws;
  uint64_t n_waves;
  uint32_t ws_nodes, ws_slots;   // workspace row counts (maxima over the engine's classes)
  uint32_t cls_bytes;            // LDS bytes reserved for class tables
  uint32_t rcap;                 // ready-list capacity per plan
  uint32_t max_v;                // largest vertex count of the problem's structures
  uint32_t flags;
  double* makespan;
  double* peak;
  double* score;
  uint8_t* mask;
  double* mass;                  // optional critical-chain mass, [plan][RPEG_MAX_V], or null
  double* util = nullptr;        // optional Trace.utilization() per plan (k_plan only), or null
  unsigned long long* prof;      // optional per-wavefront phase clocks (8 per wavefront), or null
  uint8_t* ovf;                  // per plan: its ready list outgrew rcap (set by a launch with a short list,
                                 // consumed by the KE_FIXUP launch with the full one), or null
  uint32_t* need;                // KE_NEED_SHARDS running maxima of the ready-list length, then one word that
                                 // counts the plans flagged in `ovf` and not yet redone; or null
  uint32_t* queue = nullptr;     // next wave task to take (zero at launch): the wavefronts of the grid take tasks as
                                 // they become free; null: block b takes tasks b, b + grid, ...
  uint32_t* cstat = nullptr;     // per class (ClassHdr::id), of its slowest 64-plan wavefront so far: microseconds
                                 // << 12 | heap pops per dispatch in sixteenths; or null
  // What the prologue launches (rpeg_kernel_prologue.h) computed for every plan of the call, indexed by plan.  All null
  // where a kernel computes these itself (the single-plan kernel without a layout).
  const double* dur = nullptr;         // [universe slot][plan], rows dur_stride apart; NaN where the reference would raise
  const uint64_t* aux_ovl = nullptr;   // PlanMasks::ovl
  const uint64_t* aux_dpne = nullptr;  // PlanMasks::dpne
  const double* aux_pen = nullptr;     // factor of the soft OOM penalty, 1.0 where the plan fits
  const uint8_t* aux_mask = nullptr;   // RPEG_MASK_VALID | _STALE_OK | _MEM_OK
                                       // (both null while `dur` is set: the kernel writes the score without penalty and
                                       // gate and sets both gate bits; k_finish puts the verdicts in afterwards)
  uint64_t dur_stride = 0;
  uint32_t* done = nullptr;      // k_plan only: done[w] = done_tag once the outputs of wave task w are written (a release
  uint32_t done_tag = 0;         // store at system scope, for a host that polls pinned memory instead of waiting for the
                                 // end of the launch); or null
  uint32_t* limit = nullptr;     // plans whose ready set outgrew what this kernel holds for good (no launch with a
                                 // longer list follows): limit[0] counts them, then (plan, class blob offset) pairs.
                                 // The launch that ends the call redoes them with a ready list as long as the
                                 // graph (the reference's heap has no capacity); or null
};

// Appends the plan of this lane to the list of plans to redo without a bound on the ready set.
__device__ inline void ke_flag_limit(const EvalLaunch& L, uint64_t pi, uint32_t cls_off) {
  if (!L.limit) return;
  const uint32_t k = atomicAdd(L.limit, 1u);
  L.limit[1 + 2 * (size_t)k] = (uint32_t)pi;
  L.limit[2 + 2 * (size_t)k] = cls_off;
}
constexpr uint32_t KE_FIXUP = 0x80000000u;   // EvalLaunch::flags: only the plans flagged in `ovf` are evaluated
constexpr int KE_NEED_SHARDS = 64;

__host__ __device__ inline size_t ke_ws_bytes(uint32_t nodes, uint32_t slots) {
  size_t lane = (16ull * nodes + 8ull * slots + nodes + 63) & ~size_t(63);
  return (size_t)KE_WAVE * lane;
}
// Dynamic LDS of one wavefront.  ls = 0: the per-plan state lives in the HBM workspace and all 64 lanes
// carry plans.  ls > 0: only the first `ls` lanes carry plans and their state (ready time, rank,
// in-degree per node) lives in LDS too, interleaved by lane.  The area holds the ready list (and, during the
// rank pass of the full-width kernel, a ring of ranks).
__host__ __device__ inline size_t ke_dyn_bytes(uint32_t rcap, uint32_t ls, uint32_t nv, uint32_t nodes = 0) {
  (void)nv;
  const size_t rw = ls ? ls : KE_WAVE;
  const size_t ready = (size_t)rcap * rw * 12;                 // key (8 bytes) and meta (4 bytes) per entry
  // (2 KB more for the full-width kernel: measured, not derived.  With 1-3 KB of slack behind the ready list the
  // steps of configs 2, 3 and 4 are 2-3 % shorter on the same machine; from 4 KB on config 3 loses a wavefront
  // per compute unit and from 6 KB on config 4 does.)
  const size_t bytes = ((ready + 15) & ~size_t(15)) + (ls ? 0 : 2048);
  // The rank pass of the full-width kernel keeps the ranks of the last nodes of the order in this area (a ring of a
  // power of two of rows of 64 doubles, and two bytes per node behind it); a successor further back is read from the
  // workspace, a round trip through the L2 right after the store.  With the unrolled steps of a graph of more than
  // 32 nodes the successors in the next step are 10-20 places on: 32 rows hold them, 16 do not.
  const size_t ring = !ls && nodes > 32 ? (size_t)32 * KE_WAVE * 8 + ((2 * (size_t)nodes + 15) & ~size_t(15)) : 0;
  return bytes > ring ? bytes : ring;
}
__host__ __device__ inline size_t ke_lds_bytes(uint32_t cls_bytes, uint32_t rcap, uint32_t ls, uint32_t nodes,
                                               uint32_t slots, uint32_t nv) {
  return cls_bytes + ke_dyn_bytes(rcap, ls, nv, nodes) + (size_t)ls * ((16ull * nodes + 8ull * slots + nodes + 15) & ~15ull);
}

#if defined(__HIPCC__)

template <int RW>
__device__ inline VPlan ke_vplan(const int16_t* pl, int v) {
  const int16_t* p = pl + v * RPEG_FIELDS * RW;
  VPlan a;
  a.dp = p[0 * RW]; a.pp = p[1 * RW]; a.tp = p[2 * RW]; a.mb = p[3 * RW];
  a.o[0] = p[4 * RW]; a.o[1] = p[5 * RW]; a.o[2] = p[6 * RW];
  a.e[0] = p[7 * RW]; a.e[1] = p[8 * RW]; a.e[2] = p[9 * RW];
  return a;
}

template <int RW>
__device__ inline double ke_slot_duration(const rpeg_problem_t& P, const rpeg_struct_t& st, int split,
                                          const SlotDesc sd, const int16_t* pl, bool* zero_div) {
  switch (sd.type) {
    case SLOT_OP_UNSPLIT:
      return op_time(P, st.vertex[sd.a], st.vertex[sd.a].unsplit, ke_vplan<RW>(pl, sd.a), zero_div);
    case SLOT_OP_SUB:
      return op_time(P, st.vertex[sd.a], st.vertex[sd.a].sub[split][sd.q], ke_vplan<RW>(pl, sd.a), zero_div);
    case SLOT_COMM_DATA: {
      const rpeg_edge_t& e = st.edge[sd.a];
      int64_t payload = sd.q == 0xFF ? e.full_bytes : e.sub_bytes[split][sd.q];
      return comm_time(P, ke_vplan<RW>(pl, e.src), ke_vplan<RW>(pl, e.dst), payload, e.is_weight != 0);
    }
    case SLOT_COMM_PUB: {
      const rpeg_pub_t& p = st.pub[sd.a];
      VPlan s = ke_vplan<RW>(pl, p.src), d = ke_vplan<RW>(pl, p.dst);
      return comm_time(P, s, d, pub_payload(P, s, d, p.model), true);
    }
    default:
      return reshard_time(P, ke_vplan<RW>(pl, sd.a), sd.b);
  }
}

template <int RW>
struct KeVMem {  // per-vertex memory quantities in LDS, [vertex*4 + field][lane]
  const double* p;
  __device__ double w_shard(int v) const { return p[(v * 4 + 0) * RW]; }
  __device__ double mem_w(int v) const { return p[(v * 4 + 1) * RW]; }
  __device__ double opt(int v) const { return p[(v * 4 + 2) * RW]; }
  __device__ double extra(int v) const { return p[(v * 4 + 3) * RW]; }
};

// max of last_fin over the vertices of a bit set
__device__ inline double ke_dev_max(unsigned m, const double (&lf)[RPEG_MAX_V]) {
  double d = 0.0;
#pragma unroll
  for (int x = 0; x < RPEG_MAX_V; ++x) d = ((m >> x) & 1u) && lf[x] > d ? lf[x] : d;
  return d;
}

#ifdef KE_FINE_PROF
#define KE_STAMP(k) do { if (L.prof && lane == first_lane && ((k) == 0 || (k) >= 5)) L.prof[w * 8 + (k)] = wall_clock64(); } while (0)
#else
#define KE_STAMP(k) do { if (L.prof && lane == first_lane) L.prof[w * 8 + (k)] = wall_clock64(); } while (0)
#endif

// LS = 0: 64 plans per wavefront, per-plan state in the HBM workspace.  LS > 0: LS plans per wavefront
// (lanes LS..63 only help to stage the class tables), per-plan state in LDS.
template <int LS>
__device__ inline void ke_eval_wave(const EvalLaunch& L, uint64_t w, uint8_t* lds) {
  constexpr int RW = LS ? LS : KE_WAVE;   // lane stride of the per-lane LDS arrays
  constexpr int SS = LS ? LS : KE_WAVE;   // element stride of the per-plan state arrays: interleaved by lane
  const int lane = threadIdx.x;
  int first_lane = 0;
  const rpeg_problem_t& P = *L.P;
  const ClassView cv = class_view(L.pool + (L.wave_cls[w] & ~KE_CLS_LDS));   // uniform
  const int n = (int)cv.h->n_nodes, n_slots = (int)cv.h->n_slots, n_succ_all = (int)cv.h->n_succ;

  // ---- LDS carve-up
  uint64_t* l_node = (uint64_t*)lds;                                  // NodeRec[n]
  uint16_t* l_succ = (uint16_t*)(lds + (size_t)n * 8);                // uint16[n_succ]
  uint8_t* dyn = lds + L.cls_bytes;
  double* r_key = (double*)dyn + lane;                                       // [rcap][RW]
  uint32_t* r_nt = (uint32_t*)(dyn + (size_t)L.rcap * RW * 8) + lane;        // [rcap][RW] meta, see below

  // which plan this lane carries; a fix-up launch only takes the plans whose list outgrew the short one
  uint64_t pi = (LS && lane >= LS) ? (uint64_t)KE_IDLE : (uint64_t)L.perm[w * KE_WAVE + lane];
  if (L.flags & KE_FIXUP) {
    if (pi != KE_IDLE && !L.ovf[pi]) pi = KE_IDLE;
    if (!__ballot(pi != KE_IDLE)) return;   // uniform: nothing to redo in this wavefront
  }
  __syncthreads();  // the previous task of this wavefront is done with LDS
  for (int i = lane; i < n; i += KE_WAVE) l_node[i] = ((const uint64_t*)cv.node)[i];
  for (int i = lane; i < n_succ_all; i += KE_WAVE) l_succ[i] = cv.succ[i];
  __syncthreads();

  if (pi == KE_IDLE) return;
  first_lane = __builtin_ctzll(__ballot(1));
  KE_STAMP(0);
  const unsigned long long t_begin = LS == 0 && L.cstat ? wall_clock64() : 0ull;   // (100 MHz)

  // ---- workspace rows of this lane
  double *g_time, *g_rank, *g_dur;
  uint8_t* g_deg;
  if (LS) {  // LDS, [row][lane]: time[nodes] rank[nodes] dur[slots] deg[nodes]
    uint8_t* sbase = dyn + ke_dyn_bytes(L.rcap, LS, L.max_v);
    g_time = (double*)sbase + lane;
    g_rank = g_time + (size_t)L.ws_nodes * LS;
    g_dur = g_rank + (size_t)L.ws_nodes * LS;
    g_deg = (uint8_t*)((double*)sbase + (2 * (size_t)L.ws_nodes + L.ws_slots) * LS) + lane;
  } else {   // HBM, the same arrays interleaved by lane: the plans of a wavefront share their class and mostly
             // work on the same node at the same time, so that their accesses fall into one row
    uint8_t* base = L.ws + (size_t)blockIdx.x * ke_ws_bytes(L.ws_nodes, L.ws_slots);
    g_time = (double*)base + lane;
    g_rank = g_time + (size_t)L.ws_nodes * KE_WAVE;
    g_dur = g_rank + (size_t)L.ws_nodes * KE_WAVE;
    g_deg = (uint8_t*)((double*)base + (2 * (size_t)L.ws_nodes + L.ws_slots) * KE_WAVE) + lane;
  }
  // Pair relations, penalty factor and gate bits of this lane's plan, and the durations of its class's slots out of
  // the table of the slot universe: the prologue launches left them by plan index (one gather each, all in flight at
  // once); the durations go into this lane's rows of the state, where the loops below read them coalesced.
  const uint64_t ovl = L.aux_ovl[pi], dpne = L.aux_dpne[pi];
  // (null: the memory-model launch runs beside this kernel, and the launch that ends the call applies its verdicts)
  const double pen = L.aux_pen ? L.aux_pen[pi] : 1.0;
  const uint8_t gates = L.aux_mask ? L.aux_mask[pi] : (uint8_t)(RPEG_MASK_VALID | RPEG_MASK_STALE_OK | RPEG_MASK_MEM_OK);
  KE_STAMP(1);
  bool err = cv.h->error != 0;
  {   // a slot whose duration the reference could not compute (division by zero) is NaN
    bool bad = false;
    const double* src = L.dur + pi;
    for (int s0 = 0; s0 < n_slots; s0 += 8) {
      double d[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) d[u] = s0 + u < n_slots ? src[(size_t)cv.umap[s0 + u] * L.dur_stride] : 0.0;
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (s0 + u < n_slots) { g_dur[(s0 + u) * SS] = d[u]; bad = bad || d[u] != d[u]; }
    }
    err = err || bad;
  }
  KE_STAMP(2);
  const bool stale_ok = (gates & RPEG_MASK_STALE_OK) != 0, mem_ok = (gates & RPEG_MASK_MEM_OK) != 0;

  KE_STAMP(3);
  // ---- ranks: reverse topological pass, then chain inheritance (scheduler.py:71-100, 367-378)
  if (LS == 0) {
    // Every rank is read back by the predecessors a few nodes further on, and a round trip through the
    // workspace per node made this pass a tenth of a long wavefront's time.  The LDS area (free between the
    // memory model and the ready list) holds the ranks of the last `win` nodes of the order, interleaved by
    // lane, and the place of every node in the order; a successor further back is read from the workspace.
    // All lanes carry plans of one class, so the control flow is uniform.
    const int dyn_bytes = (int)ke_dyn_bytes(L.rcap, 0, L.max_v, L.ws_nodes);
    int win = (dyn_bytes - ((2 * n + 15) & ~15)) / (KE_WAVE * 8);
    while (win & (win - 1)) win &= win - 1;   // a power of two: the place in the ring is a mask away
    uint16_t* l_pos = (uint16_t*)(dyn + (size_t)win * KE_WAVE * 8);
    double* ring = (double*)dyn + lane;
    __syncthreads();   // the memory terms in this area are dead
    if (lane == first_lane)
      for (int i = 0; i < n; ++i) l_pos[cv.topo[i]] = (uint16_t)i;
    __syncthreads();
    // node records and successor lists come from their LDS copies, the order itself one node ahead: the
    // chain from one rank to the next is LDS reads only
    auto node_at = [&](int v) { NodeRec r; const uint64_t b = l_node[v]; __builtin_memcpy(&r, &b, 8); return r; };
    int v_next = n > 0 ? cv.topo[n - 1] : 0;
    double d_next = n > 0 ? g_dur[(node_at(v_next).slot) * SS] : 0.0;
    for (int i = n - 1; i >= 0; --i) {
      const int v = v_next;
      const NodeRec nr = node_at(v);
      const double d = d_next;
      if (i > 0) {   // one node ahead: off the chain
        v_next = cv.topo[i - 1];
        d_next = g_dur[(node_at(v_next).slot) * SS];
      }
      double best = 0.0;
      auto rank_of = [&](int sx) {
        const int px = l_pos[sx];
        return (win > 0 && px - i <= win) ? ring[(px & (win - 1)) * KE_WAVE] : g_rank[(sx) * SS];
      };
      int j = 0;
      for (; j + 2 <= nr.n_succ; j += 2) {   // two successors' reads in flight at once
        const int s0 = l_succ[nr.succ_begin + j], s1 = l_succ[nr.succ_begin + j + 1];
        const double r0 = rank_of(s0), r1 = rank_of(s1);
        best = r0 > best ? r0 : best;
        best = r1 > best ? r1 : best;
      }
      if (j < nr.n_succ) {
        const double r = rank_of(l_succ[nr.succ_begin + j]);
        best = r > best ? r : best;
      }
      const double rk = d + best;
      g_rank[(v) * SS] = rk;
      if (win > 0) ring[(i & (win - 1)) * KE_WAVE] = rk;
    }
    __syncthreads();
  } else {
    for (int i = n - 1; i >= 0; --i) {
      const int v = cv.topo[i];
      const NodeRec nr = cv.node[v];
      double best = 0.0;
      for (int j = 0; j < nr.n_succ; ++j) {
        const double r = g_rank[(cv.succ[nr.succ_begin + j]) * SS];
        best = r > best ? r : best;
      }
      g_rank[(v) * SS] = g_dur[(nr.slot) * SS] + best;
    }
  }
  for (unsigned g = 0; g < cv.h->n_groups; ++g) {
    const GroupRec gr = cv.group[g];
    double top = g_rank[(cv.gmember[gr.begin]) * SS];
    for (int j = 1; j < gr.count; ++j) {
      const double r = g_rank[(cv.gmember[gr.begin + j]) * SS];
      top = r > top ? r : top;
    }
    for (int j = 0; j < gr.count; ++j) g_rank[(cv.gmember[gr.begin + j]) * SS] = top;
  }
  for (int v = 0; v < n; ++v) {   // (the node records from their LDS copies: a scalar load from the pool per node waited for each)
    NodeRec nr;
    const uint64_t bits = l_node[v];
    __builtin_memcpy(&nr, &bits, 8);
    g_deg[(v) * SS] = nr.indeg;
    g_time[(v) * SS] = 0.0;
  }

  KE_STAMP(4);
  // ---- list scheduling (scheduler.py:399-546 with the lazy heap replaced by a position-ordered list)
  //
  // The reference pops the minimum of (est, comm_prio, topo_idx, -rank, tie) from a heap whose keys may
  // be stale: a popped entry whose true est (device availability included) exceeds its key is pushed
  // back with the true est and a fresh tie.  Here the ready list is kept sorted by the part of the key
  // that never changes while an entry waits: (comm_prio*8+topo_idx ascending, rank descending, push
  // order).  A new entry goes behind every entry that is not after it; an entry pushed back (fresh tie)
  // moves behind the entries that agree with it in (prio, rank).  The heap's pop is then the FIRST entry
  // of minimum key: one load, one compare and three selects per entry.
  //
  // An entry is its key (8 bytes) and a meta word: node | prio << 12 | x << 16 | y << 19 | same << 22,
  // x and y the (one or two) vertices whose devices the node reserves, `same` set when the entry agrees
  // in (prio, rank) with the entry before it.  Ranks stay in the per-plan state and are read only when
  // entries are inserted.
  //
  // Each outer iteration first takes the heap's pops up to the next dispatch (a short inner loop: pop,
  // and if the key is stale push back), then dispatches one node for all plans of the wavefront together.
  double lf[RPEG_MAX_V];
#pragma unroll
  for (int x = 0; x < RPEG_MAX_V; ++x) lf[x] = 0.0;
  int n_ready = 0, done = 0, max_ready = 0;
  bool ovf = false, limit = false;
  const int rcap = (int)L.rcap;   // a multiple of eight
  const double inf = __builtin_inf();
  constexpr uint32_t SAME = 1u << 22;
  for (int j = 0; j < rcap; ++j) {   // entries past n_ready never win a scan
    r_key[j * RW] = inf;
    r_nt[j * RW] = 0;
  }
  auto make_meta = [&](int v, const NodeRec& r) -> uint32_t {
    const unsigned blk = blocked_mask(r, dpne);
    const unsigned x = (unsigned)__builtin_ctz(blk | 0x100u);
    const unsigned rest = blk & (blk - 1u);
    const unsigned y = rest ? (unsigned)__builtin_ctz(rest) : x;
    if (rest & (rest - 1u)) err = limit = true;   // more than two reserved vertices cannot be packed
    return (uint32_t)v | ((uint32_t)r.ptkey << 12) | (x << 16) | (y << 19);
  };
  // Up to NQ pushes at once, with the result of pushing them one after the other: a stable merge in
  // which a new entry goes behind the waiting entries and the earlier new entries that are not after it.
  // The list is read and written once, from the top down (entries only move up).  NQ bounds the number
  // of new entries of any plan of the wavefront.  A waiting entry keeps its `same` flag: no new entry
  // can land between two entries that agree.
  auto push_many = [&](auto nq_tag, int cnt, const uint32_t (&nm)[4], const double (&nk)[4], const double (&nr)[4]) {
    constexpr int NQ = decltype(nq_tag)::value;
    unsigned npt[NQ];
    int c[NQ];                 // waiting entries not after new entry q
    bool eq[NQ];               // a waiting entry agrees with new entry q in (prio, rank)
#pragma unroll
    for (int q = 0; q < NQ; ++q) { npt[q] = (nm[q] >> 12) & 15u; c[q] = 0; eq[q] = false; }
    for (int j1 = (n_ready + 7) & ~7; j1 > 0; j1 -= 8) {
      const int j0 = j1 - 8;
      double k[8], r[8];
      uint32_t m[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        k[u] = r_key[(j0 + u) * RW];
        m[u] = r_nt[(j0 + u) * RW];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {   // slots past the end of the list hold anything: keep the read inside the plan's rows
        const uint32_t node = m[u] & 0xFFFu;
        r[u] = g_rank[(int)(node < L.ws_nodes ? node : 0u) * SS];
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (j0 + u >= n_ready) continue;
        const unsigned pu = (m[u] >> 12) & 15u;
        int up = 0;
#pragma unroll
        for (int q = 0; q < NQ; ++q) {
          const bool after = pu > npt[q] || (pu == npt[q] && r[u] < nr[q]);   // the waiting entry is after new entry q
          up += (q < cnt && after) ? 1 : 0;
          c[q] += after ? 0 : 1;
          eq[q] = eq[q] || (pu == npt[q] && r[u] == nr[q]);
        }
        if (up) {
          r_key[(j0 + u + up) * RW] = k[u];
          r_nt[(j0 + u + up) * RW] = m[u];
        }
      }
    }
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
      if (q >= cnt) break;
      int idx = c[q];
      bool same = eq[q];
#pragma unroll
      for (int o = 0; o < NQ; ++o) {
        if (o == q || o >= cnt) continue;
        const bool o_after = npt[o] > npt[q] || (npt[o] == npt[q] && nr[o] < nr[q]);     // o strictly after q
        const bool o_before = npt[o] < npt[q] || (npt[o] == npt[q] && nr[o] > nr[q]);    // o strictly before q
        idx += (o < q ? !o_after : o_before) ? 1 : 0;
        same = same || (o < q && npt[o] == npt[q] && nr[o] == nr[q]);
      }
      r_key[idx * RW] = nk[q];
      r_nt[idx * RW] = nm[q] | (same ? SAME : 0u);
    }
    n_ready += cnt;
    max_ready = n_ready > max_ready ? n_ready : max_ready;
  };
  for (unsigned i = 0; i < cv.h->n_init && !err; ++i) {
    const int v = cv.init[i];
    if (n_ready >= rcap - 1) { err = ovf = true; break; }
    const uint32_t nm[4] = {make_meta(v, cv.node[v]), 0u, 0u, 0u};
    const double nk[4] = {0.0, 0.0, 0.0, 0.0}, nrk[4] = {g_rank[(v) * SS], 0.0, 0.0, 0.0};
    push_many(std::integral_constant<int, 1>{}, 1, nm, nk, nrk);
  }
  double makespan = 0.0;
  const long guard_max = (long)n * n + 64;
  long guard_total = 0;
  // KE_FINE_PROF (a build of its own, for measurements): shader clocks of the four sections of the loop, summed
  // over the dispatches of the wavefront, in place of the phase stamps 1-4 of the profile row
#ifdef KE_FINE_PROF
  long long fp_pop = 0, fp_rm = 0, fp_succ = 0, fp_push = 0, fp_t = 0;
#define FP_MARK(acc) do { const long long _t = clock64(); acc += _t - fp_t; fp_t = _t; } while (0)
#else
#define FP_MARK(acc) do {} while (0)
#endif
  for (long guard = 0; !err && done < n && guard < guard_max; ++guard) {
    ++guard_total;
    if (n_ready == 0) { err = true; break; }
    int bj = 0;
    double est = 0.0;
#ifdef KE_FINE_PROF
    fp_t = clock64();
#endif
    for (long inner = 0; inner < guard_max; ++inner) {
      double bk = inf;
      bj = 0;
      for (int j0 = 0; j0 < n_ready; j0 += 8) {
        double k[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) k[u] = r_key[(j0 + u) * RW];
        const bool c01 = k[1] < k[0], c23 = k[3] < k[2], c45 = k[5] < k[4], c67 = k[7] < k[6];
        const double a0 = c01 ? k[1] : k[0], a1 = c23 ? k[3] : k[2], a2 = c45 ? k[5] : k[4], a3 = c67 ? k[7] : k[6];
        const int i0 = c01 ? 1 : 0, i1 = c23 ? 3 : 2, i2 = c45 ? 5 : 4, i3 = c67 ? 7 : 6;
        const bool d0 = a1 < a0, d1 = a3 < a2;
        const double b0 = d0 ? a1 : a0, b1 = d1 ? a3 : a2;
        const int x0 = d0 ? i1 : i0, x1 = d1 ? i3 : i2;
        const bool e0 = b1 < b0;
        const double c = e0 ? b1 : b0;
        if (c < bk) { bk = c; bj = j0 + (e0 ? x1 : x0); }
      }
      const uint32_t m0 = r_nt[bj * RW];
      const uint32_t m1 = r_nt[(bj + 1 < rcap ? bj + 1 : bj) * RW];
      const double dv = ke_dev_max((1u << ((m0 >> 16) & 7u)) | (1u << ((m0 >> 19) & 7u)), lf);
      est = dv > bk ? dv : bk;
      if (!(est > bk)) break;
      ++guard_total;
      r_key[bj * RW] = est;   // scheduler.py:437-443
      if (bj + 1 < n_ready && (m1 & SAME)) {
        // behind its equals: the next entry takes this place (and this entry's relation to the entry before)
        uint32_t mine = m0;
        uint32_t nxt = m1;
        while (true) {
          const double k2 = r_key[(bj + 1) * RW];
          r_key[bj * RW] = k2;
          r_nt[bj * RW] = (nxt & ~SAME) | (mine & SAME);
          ++bj;
          mine |= SAME;
          r_key[bj * RW] = est;
          r_nt[bj * RW] = mine;
          if (bj + 1 >= n_ready) break;
          nxt = r_nt[(bj + 1) * RW];
          if (!(nxt & SAME)) break;
        }
      }
    }
    FP_MARK(fp_pop);
    const uint32_t bm = r_nt[bj * RW];
    const int bv = (int)(bm & 0xFFFu);
    const unsigned blocked = (1u << ((bm >> 16) & 7u)) | (1u << ((bm >> 19) & 7u));
    const uint64_t nbits = l_node[bv];
    NodeRec nr;
    __builtin_memcpy(&nr, &nbits, 8);
    // dispatch bv: issue every load of this step before using any of them
    const double d = g_dur[(nr.slot) * SS];
    int wv[4];
    double wt[4], wr[4];
    uint8_t wd[4];
    const int ns = nr.n_succ;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      wv[j] = j < ns ? (int)l_succ[nr.succ_begin + j] : 0;
      if (j < ns) {
        wt[j] = g_time[(wv[j]) * SS];
        wd[j] = g_deg[(wv[j]) * SS];
        wr[j] = g_rank[(wv[j]) * SS];
      }
    }
    // remove the entry, keeping the order
    --n_ready;
    for (int j0 = bj; j0 < n_ready; j0 += 8) {    // entries (bj, n_ready] move one down, eight per round trip
      double k[8];
      uint32_t m[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int src = j0 + 1 + u < rcap ? j0 + 1 + u : rcap - 1;
        k[u] = r_key[src * RW];
        m[u] = r_nt[src * RW];
      }
      // the entry that follows the removed one agrees with its new neighbour only if both did
      if (j0 == bj) m[0] &= ~SAME | (bm & SAME);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (j0 + u >= n_ready) continue;
        r_key[(j0 + u) * RW] = k[u];
        r_nt[(j0 + u) * RW] = m[u];
      }
    }
    r_key[n_ready * RW] = inf;
    FP_MARK(fp_rm);
    const double fin = est + d;
    makespan = fin > makespan ? fin : makespan;
    ++done;
    if (L.mass) {  // keep the trace: a dispatched node needs neither its ready time nor its rank again
      g_time[(bv) * SS] = fin;
      g_rank[(bv) * SS] = est;
    }
    unsigned touched = 0;
#pragma unroll
    for (int x = 0; x < RPEG_MAX_V; ++x)
      if ((blocked >> x) & 1u) touched |= mask_row(ovl, x);
#pragma unroll
    for (int x = 0; x < RPEG_MAX_V; ++x)
      if (((touched >> x) & 1u) && fin > lf[x]) lf[x] = fin;
    for (int j0 = 0; j0 < ns; j0 += 4) {
      if (j0 > 0) {  // rare: more than four successors
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          wv[j] = j0 + j < ns ? (int)l_succ[nr.succ_begin + j0 + j] : 0;
          if (j0 + j < ns) {
            wt[j] = g_time[(wv[j]) * SS];
            wd[j] = g_deg[(wv[j]) * SS];
            wr[j] = g_rank[(wv[j]) * SS];
          }
        }
      }
      // successors that become ready are collected in successor order and pushed together
      uint32_t nm[4] = {0, 0, 0, 0};
      double nk[4] = {0.0, 0.0, 0.0, 0.0}, nrk[4] = {0.0, 0.0, 0.0, 0.0};
      int cnt = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (j0 + j >= ns) break;
        const int wn = wv[j];
        double t = fin > wt[j] ? fin : wt[j];
        const uint8_t left = (uint8_t)(wd[j] - 1);
        if (left == 0) {
          uint64_t wb = l_node[wn];
          NodeRec wrc;
          __builtin_memcpy(&wrc, &wb, 8);
          const double d2 = ke_dev_max(blocked_mask(wrc, dpne), lf);
          t = d2 > t ? d2 : t;
          const uint32_t meta = make_meta(wn, wrc);
#pragma unroll
          for (int q = 0; q < 4; ++q)
            if (q == cnt) { nm[q] = meta; nk[q] = t; nrk[q] = wr[j]; }
          ++cnt;
        } else {
          g_time[(wn) * SS] = t;
          g_deg[(wn) * SS] = left;
        }
      }
      if (n_ready + cnt >= rcap) { err = ovf = true; break; }
      FP_MARK(fp_succ);
      // the widest push of the wavefront selects the code: most dispatches release one or two successors
      if (__ballot(cnt > 2)) {
        if (cnt) push_many(std::integral_constant<int, 4>{}, cnt, nm, nk, nrk);
      } else if (__ballot(cnt > 1)) {
        if (cnt) push_many(std::integral_constant<int, 2>{}, cnt, nm, nk, nrk);
      } else if (cnt) {
        push_many(std::integral_constant<int, 1>{}, cnt, nm, nk, nrk);
      }
      FP_MARK(fp_push);
    }
  }
#ifdef KE_FINE_PROF
  if (L.prof && lane == first_lane) {
    L.prof[w * 8 + 1] = fp_pop; L.prof[w * 8 + 2] = fp_rm; L.prof[w * 8 + 3] = fp_succ; L.prof[w * 8 + 4] = fp_push;
  }
#endif
  if (done != n) err = true;
  if (limit || (ovf && (!L.ovf || (L.flags & KE_FIXUP)))) ke_flag_limit(L, pi, L.wave_cls[w] & ~KE_CLS_LDS);
  if (L.ovf) {
    const bool fix = (L.flags & KE_FIXUP) != 0;
    if (fix) L.ovf[pi] = 0;
    else if (ovf) L.ovf[pi] = 1;
    // the count of flagged plans lets a fix-up launch that has nothing to redo end at once
    const int k = __builtin_popcountll(__ballot(fix || ovf));
    if (k && L.need && lane == first_lane) {
      if (fix) atomicSub(L.need + KE_NEED_SHARDS, (uint32_t)k);
      else atomicAdd(L.need + KE_NEED_SHARDS, (uint32_t)k);
    }
  }
  if (L.need) {   // longest ready list of the wavefront, folded into one of the running maxima
    int m = max_ready;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const int o = __shfl_xor(m, off);
      m = o > m ? o : m;
    }
    uint32_t* slot = L.need + (blockIdx.x & (KE_NEED_SHARDS - 1));
    if (lane == first_lane && (uint32_t)m > *slot) atomicMax(slot, (uint32_t)m);
  }
  KE_STAMP(5);
  if (L.prof) atomicMax(&L.prof[w * 8 + 7], ((unsigned long long)n << 32) | (unsigned long long)guard_total);
  if (LS == 0 && L.cstat && !(L.flags & KE_FIXUP) && n > 0) {
    // what the wavefront paid per dispatch: the pops of its slowest plan.  The host reads it to decide which
    // classes are worth four lanes per plan.
    uint32_t g = (uint32_t)guard_total;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const uint32_t o = (uint32_t)__shfl_xor((int)g, off);
      g = o > g ? o : g;
    }
    const uint32_t per16 = g * 16u / (uint32_t)n;
    const unsigned long long us = (wall_clock64() - t_begin) / 100ull;
    const uint32_t word = ((uint32_t)(us < 0xFFFFFull ? us : 0xFFFFFull) << 12) | (per16 < 0xFFFu ? per16 : 0xFFFu);
    uint32_t* slot = L.cstat + cv.h->id;
    if (lane == first_lane && word > *slot) atomicMax(slot, word);
  }

  // ---- outputs
  uint8_t mask = RPEG_MASK_VALID;
  if (stale_ok) mask |= RPEG_MASK_STALE_OK;
  if (mem_ok) mask |= RPEG_MASK_MEM_OK;
  double out_makespan, out_score;
  if (err || makespan == 0.0) {
    out_makespan = out_score = __builtin_nan("");
    mask |= RPEG_MASK_ERROR;
    if (ovf || limit) mask |= RPEG_MASK_LIMIT;
  } else {
    double score = P.score_num / makespan;
    if (!mem_ok) score = score * pen;
    if ((L.flags & RPEG_GATE_STALE) && !stale_ok) score = 0.0;
    out_makespan = makespan;
    out_score = score;
  }
  if (L.makespan) L.makespan[pi] = out_makespan;   // (the peak is the prologue launch's output)
  if (L.score) L.score[pi] = out_score;
  if (L.mask) L.mask[pi] = mask;
  if (L.mass) {
    double m[RPEG_MAX_V];
    if (err) {
#pragma unroll
      for (int x = 0; x < RPEG_MAX_V; ++x) m[x] = __builtin_nan("");
    } else {
      critical_mass(cv, [&](int i) { return g_time[(i) * SS]; }, [&](int i) { return g_rank[(i) * SS]; }, m);
    }
#pragma unroll
    for (int x = 0; x < RPEG_MAX_V; ++x) L.mass[pi * RPEG_MAX_V + x] = m[x];
  }
  KE_STAMP(6);
}

#endif  // __HIPCC__

}  // namespace rpeg
#endif
