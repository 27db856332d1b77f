// rpeg_kernel_prologue.h - the part of a plan's evaluation that is plain arithmetic, as launches of their own
// (device only).
//
// The list scheduler is a chain of dependent steps: the kernels that run it (rpeg_kernel_eval.h, _quad.h, _plan.h)
// keep one or two wavefronts on a SIMD and issue an instruction every ten clocks or so.  Inside those kernels the
// cost model (NodeCostModel.time of every duration slot, cost.py:66-686) and the memory model (per-device peaks,
// memory.py:608-887) cost the same ten clocks an instruction, a fifth to a quarter of a wavefront's time, although
// nothing in them waits for anything.
//
// Neither depends on the lowering class of a plan: a duration is a function of the plan fields and of which slot
// it is -- so every slot a class of the plan's structure COULD have (slot_universe) is evaluated, and a class picks
// its own through ClassView::umap --, and the vertex order that fixes the memory model's float sums follows from the
// plan (plan_vorder).  Both launches therefore run on the plans in the caller's own order, straight from the
// caller's tensors (coalesced), right behind the signature kernel: while the class totals are on their way to the
// host, which lays the batch out, i.e. off the critical path of the call.
//
//   k_prologue   one wavefront per (64 plans, row); a row is one slot of the universe, or the pair relations, or one
//                vertex's memory terms -- a wavefront holds one short piece of arithmetic, so that many are resident
//                dur[u][i]            duration of universe slot u for plan i (rows dur_stride apart), NaN where the
//                                     reference would raise ZeroDivisionError; not written for the phases a plan's
//                                     split variant does not have
//                aux_ovl / _eq / _dpne  pair relations (PlanMasks), per plan
//                vm[v * 4 + f][i]     per-vertex memory terms (VMem)
//   k_peaks      peak[i]              the call's own output: largest device peak
//                aux_pen[i]           factor of the soft OOM penalty (evaluate.py:396-401), 1.0 where the plan fits
//                aux_mask[i]          RPEG_MASK_VALID | _STALE_OK | _MEM_OK
#ifndef RPEG_KERNEL_PROLOGUE_H
#define RPEG_KERNEL_PROLOGUE_H

#include "rpeg_kernel_eval.h"

namespace rpeg {

constexpr int KPRO_PARTS = 6;                    // wavefronts that share the rows of a block of 64 plans
constexpr uint32_t KPRO_INVALID = 0xFFFFFFFFu;   // class id of a plan that breaks an integer rule: not evaluated

struct PrologueLaunch {
  const rpeg_problem_t* P;
  const int16_t* vert;         // the caller's plan tensors
  const uint8_t* head;
  uint64_t stride, n;
  const uint32_t* cid;         // per plan: KPRO_INVALID for a plan the gate rejected
  const SlotDesc* uni;         // [structure][RPEG_MAX_UNIVERSE]
  uint32_t n_uni[RPEG_MAX_STRUCT];
  uint32_t max_uni;            // rows of the grid: max_uni durations, one row of pair relations, then one per vertex
  uint32_t max_v;              // largest vertex count of the problem's structures (sizes the LDS of the second launch)
  double* dur;
  uint64_t dur_stride;         // plans per row of dur and vm
  uint64_t* aux_ovl;
  uint64_t* aux_eq;
  uint64_t* aux_dpne;
  double* vm;                  // [vertex * 4 + field][plan]: w_shard, mem_w, opt, extra (VMem) of every vertex
  double* aux_pen;
  uint8_t* aux_mask;
  double* peak;                // or null
};

#if defined(__HIPCC__)

__device__ inline VPlan kpro_vplan(const int16_t* p, uint64_t stride, int v) {
  p += (uint64_t)v * RPEG_FIELDS * stride;
  VPlan a;
  a.dp = p[0 * stride]; a.pp = p[1 * stride]; a.tp = p[2 * stride]; a.mb = p[3 * stride];
  a.o[0] = p[4 * stride]; a.o[1] = p[5 * stride]; a.o[2] = p[6 * stride];
  a.e[0] = p[7 * stride]; a.e[1] = p[8 * stride]; a.e[2] = p[9 * stride];
  return a;
}

// (the pieces are functions of their own, not inlined: each gets the registers it needs instead of the kernel holding
// the union of all of them, which costs it its residency)
// (NaN where the reference would raise ZeroDivisionError: a flag handed in by address would live in scratch memory)
__device__ __attribute__((noinline)) double kpro_op_time(const rpeg_problem_t& P, const rpeg_vertex_t& vx, const rpeg_opconst_t& oc,
                                                         const int16_t* pl, uint64_t stride, int v) {
  bool zero_div = false;
  const double t = op_time(P, vx, oc, kpro_vplan(pl, stride, v), &zero_div);
  return zero_div ? __builtin_nan("") : t;
}

__device__ inline double kpro_slot_duration(const rpeg_problem_t& P, const rpeg_struct_t& st, int split, const SlotDesc sd,
                                            const int16_t* pl, uint64_t stride) {
  switch (sd.type) {
    case SLOT_OP_UNSPLIT:
      return kpro_op_time(P, st.vertex[sd.a], st.vertex[sd.a].unsplit, pl, stride, sd.a);
    case SLOT_OP_SUB:
      return kpro_op_time(P, st.vertex[sd.a], st.vertex[sd.a].sub[split][sd.q], pl, stride, sd.a);
    case SLOT_COMM_DATA: {
      const rpeg_edge_t& e = st.edge[sd.a];
      const int64_t payload = sd.q == 0xFF ? e.full_bytes : e.sub_bytes[split][sd.q];
      return comm_time(P, kpro_vplan(pl, stride, e.src), kpro_vplan(pl, stride, e.dst), payload, e.is_weight != 0);
    }
    case SLOT_COMM_PUB: {
      const rpeg_pub_t& p = st.pub[sd.a];
      const VPlan s = kpro_vplan(pl, stride, p.src), d = kpro_vplan(pl, stride, p.dst);
      return comm_time(P, s, d, pub_payload(P, s, d, p.model), true);
    }
    default:
      return reshard_time(P, kpro_vplan(pl, stride, sd.a), sd.b);
  }
}

// (these take what they need by value: the address of the launch record would force a copy of it into scratch memory
// in every wavefront)
__device__ __attribute__((noinline)) void kpro_masks(const int16_t* pl, const uint64_t stride, const int nv, uint64_t* ovl,
                                                     uint64_t* eq, uint64_t* dpne) {
  VPlan a[RPEG_MAX_V];
#pragma unroll
  for (int v = 0; v < RPEG_MAX_V; ++v)
    if (v < nv) a[v] = kpro_vplan(pl, stride, v);
  const PlanMasks pm = plan_masks(a, nv);
  *ovl = pm.ovl;
  *eq = pm.eq;
  *dpne = pm.dpne;
}

__device__ __attribute__((noinline)) void kpro_vmem(const rpeg_problem_t& P, const int16_t* pl, const uint64_t stride,
                                                    const rpeg_struct_t& st, const int v, double* out, const uint64_t out_stride) {
  const VMem m = vertex_memory(P, st.vertex[v], kpro_vplan(pl, stride, v), struct_coresident(st));
  out[0 * out_stride] = (double)m.w_shard;
  out[1 * out_stride] = m.mem_w;
  out[2 * out_stride] = m.opt;
  out[3 * out_stride] = m.extra;
}

// Plan i of this lane, structure su (uniform), one row of the first launch's grid (uniform): the duration of one slot
// of the universe; or the pair relations of the plan; or the memory terms of one vertex.
__device__ inline void kpro_row(const PrologueLaunch& L, const uint64_t i, const int su, const int split, const int row) {
  const rpeg_problem_t& P = *L.P;
  const rpeg_struct_t& st = P.st[su];
  const int16_t* pl = L.vert + i;
  if (row < (int)L.max_uni) {
    if (row >= (int)L.n_uni[su]) return;
    const SlotDesc sd = L.uni[(size_t)su * RPEG_MAX_UNIVERSE + row];   // uniform
    if (!slot_in_split(P, split, sd)) return;                          // this lane's split variant has no such phase
    L.dur[(uint64_t)row * L.dur_stride + i] = kpro_slot_duration(P, st, split, sd, pl, L.stride);
  } else if (row == (int)L.max_uni) {
    kpro_masks(pl, L.stride, st.n_vertex, L.aux_ovl + i, L.aux_eq + i, L.aux_dpne + i);
  } else {
    const int v = row - (int)L.max_uni - 1;
    if (v < st.n_vertex) kpro_vmem(P, pl, L.stride, st, v, L.vm + (uint64_t)(v * 4) * L.dur_stride + i, L.dur_stride);
  }
}

struct KproOrder {   // the vertex order of a plan in LDS, [position][lane]
  uint8_t* p;
  __device__ uint8_t operator[](int k) const { return p[k * KE_WAVE]; }
};

// plan_vorder (rpeg_class.h) from the pair relations instead of the plan fields: two allocations are disjoint exactly
// when they do not intersect
__device__ inline void kpro_vorder(const rpeg_problem_t& P, const rpeg_struct_t& st, int split, uint64_t ovl, uint8_t* order_lds) {
  const int nv = st.n_vertex, nph = split > 0 ? P.n_phase[split] : 0;
  unsigned gen_split = 0, moved = 0;
  int c = 0;
  auto disjoint = [&](int u, int v) { return !((ovl >> (8 * u + v)) & 1ull); };
  if (nph > 0) {
    for (int e = 0; e < st.n_edge; ++e)
      if (st.edge[e].gen_inf && disjoint(st.edge[e].src, st.edge[e].dst)) gen_split |= 1u << st.edge[e].src;
    for (int e = 0; e < st.n_edge; ++e) {
      const int u = st.edge[e].src, v = st.edge[e].dst;
      if (((gen_split >> u) & 1u) && st.vertex[v].role == RPEG_ROLE_INF && disjoint(u, v)) moved |= 1u << v;
    }
  }
  for (int v = 0; v < nv; ++v)
    if (!((moved >> v) & 1u)) order_lds[(c++) * KE_WAVE] = (uint8_t)v;
  unsigned done = 0;   // the vertices taken out, in the order of the edges that split them
  for (int e = 0; e < st.n_edge; ++e) {
    const int u = st.edge[e].src, v = st.edge[e].dst;
    if (!((moved >> v) & 1u) || ((done >> v) & 1u)) continue;
    if (((gen_split >> u) & 1u) && st.vertex[v].role == RPEG_ROLE_INF && disjoint(u, v)) {
      done |= 1u << v;
      order_lds[(c++) * KE_WAVE] = (uint8_t)v;
    }
  }
}

// The second launch: largest device peak, penalty factor and gate bits of plan i of this lane, structure su (uniform),
// from the pair relations and the per-vertex memory terms the first launch left.  l_vm: [vertex * 4 + field][lane]
// doubles and l_ord: [position][lane] bytes in LDS (the peak indexes both with run-time values, which would put
// per-thread arrays into scratch memory).
__device__ inline void kpro_peaks(const PrologueLaunch& L, const uint64_t i, const int su, const PlanHead h, double* l_vm,
                                  uint8_t* l_ord) {
  const rpeg_problem_t& P = *L.P;
  const rpeg_struct_t& st = P.st[su];
  const int nv = st.n_vertex;
  PlanMasks pm;
  pm.ovl = L.aux_ovl[i];
  pm.eq = L.aux_eq[i];
  pm.dpne = 0;
  {   // every load in flight at once
    double x[RPEG_MAX_V * 4];
#pragma unroll
    for (int k = 0; k < RPEG_MAX_V * 4; ++k)
      if (k < nv * 4) x[k] = L.vm[(uint64_t)k * L.dur_stride + i];
#pragma unroll
    for (int k = 0; k < RPEG_MAX_V * 4; ++k)
      if (k < nv * 4) l_vm[k * KE_WAVE] = x[k];
  }
  kpro_vorder(P, st, h.split, pm.ovl, l_ord);
  const KeVMem<KE_WAVE> kvm{l_vm};
  const double peak = device_peak_max(P, st, KproOrder{l_ord}, pm, kvm);
  const bool stale_ok = stale_layout_ok(st, h, pm.ovl);
  const bool mem_ok = !(peak > P.cap);
  L.aux_pen[i] = mem_ok ? 1.0 : oom_penalty(peak, P.cap);
  L.aux_mask[i] = (uint8_t)(RPEG_MASK_VALID | (stale_ok ? RPEG_MASK_STALE_OK : 0) | (mem_ok ? RPEG_MASK_MEM_OK : 0));
  if (L.peak) L.peak[i] = peak;
}

#endif  // __HIPCC__

}  // namespace rpeg
#endif
