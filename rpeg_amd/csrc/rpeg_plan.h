// rpeg_plan.h - one plan, end to end, given its lowering class: plan fields -> durations ->
// makespan -> per-device memory peak -> score and mask.  Compiled for the device (kernel body) and
// for the host (unit checks).
#ifndef RPEG_PLAN_H
#define RPEG_PLAN_H

#include "rpeg_class.h"

namespace rpeg {

struct PlanHead { int structure, split, tau0, tau1; };

struct PlanOut { double makespan, peak, score; uint8_t mask; };

// Loads the header and the vertex fields of plan i from the structure-of-arrays tensors.
RPEG_HD PlanHead load_head(const uint8_t* head, uint64_t stride, uint64_t i) {
  PlanHead h;
  h.structure = head[0 * stride + i];
  h.split = head[1 * stride + i];
  h.tau0 = head[2 * stride + i];
  h.tau1 = head[3 * stride + i];
  return h;
}

RPEG_HD void load_vertex(const int16_t* vert, uint64_t stride, uint64_t i, int slot, VPlan* a) {
  const int16_t* p = vert + (uint64_t)slot * RPEG_FIELDS * stride + i;
  a->dp = p[0 * stride]; a->pp = p[1 * stride]; a->tp = p[2 * stride]; a->mb = p[3 * stride];
  a->o[0] = p[4 * stride]; a->o[1] = p[5 * stride]; a->o[2] = p[6 * stride];
  a->e[0] = p[7 * stride]; a->e[1] = p[8 * stride]; a->e[2] = p[9 * stride];
}

// Integer gate: header ranges plus evaluate.py:172-196 per vertex.
template <class PLANS>
RPEG_HD bool plan_valid(const rpeg_problem_t& P, const PlanHead& h, const PLANS& a) {
  if (h.structure < 0 || h.structure >= P.n_struct) return false;
  if (h.split < 0 || h.split >= P.n_split) return false;
  if (h.tau0 > 3 || h.tau1 > 3) return false;
  const rpeg_struct_t& st = P.st[h.structure];
  for (int v = 0; v < st.n_vertex; ++v)
    if (!vertex_valid(P, a[v], P.model[st.vertex[v].model].L)) return false;
  return true;
}

// evaluate.py:115-140
RPEG_HD bool stale_layout_ok(const rpeg_struct_t& st, const PlanHead& h, uint64_t ovl) {
  for (int p = 0; p < st.n_pub; ++p) {
    int tau = st.pub[p].tau_slot == 0 ? h.tau0 : h.tau1;
    if (tau <= 0) continue;
    if ((ovl >> (8 * st.pub[p].src + st.pub[p].dst)) & 1ull) return false;
  }
  return true;
}

// Pair relations of one plan.  The loops run over the compile-time vertex bound so that `a` is only
// ever indexed statically (register-resident on the device).
RPEG_HD PlanMasks plan_masks(const VPlan* a, int nv) {
  PlanMasks m;
  m.ovl = m.eq = m.dpne = 0;
  // the three relations are symmetric: every pair is tested once and entered for both orders
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
#endif
  for (int u = 0; u < RPEG_MAX_V; ++u) {
    if (u >= nv) continue;
    const uint64_t self = 1ull << (9 * u);
    if (!alloc_disjoint(a[u], a[u])) m.ovl |= self;
    m.eq |= self;
#if defined(__HIP_DEVICE_COMPILE__)
#pragma unroll
#endif
    for (int v = u + 1; v < RPEG_MAX_V; ++v) {
      if (v >= nv) continue;
      const uint64_t bits = (1ull << (8 * u + v)) | (1ull << (8 * v + u));
      if (!alloc_disjoint(a[u], a[v])) m.ovl |= bits;
      if (alloc_equal(a[u], a[v])) m.eq |= bits;
      if (a[u].dp != a[v].dp) m.dpne |= bits;
    }
  }
  return m;
}

struct VMemArray {   // host-side accessor over an array of VMem
  const VMem* vm;
  RPEG_HD double w_shard(int v) const { return (double)vm[v].w_shard; }
  RPEG_HD double mem_w(int v) const { return vm[v].mem_w; }
  RPEG_HD double opt(int v) const { return vm[v].opt; }
  RPEG_HD double extra(int v) const { return vm[v].extra; }
};

// Everything after the class is known.  MEM additionally provides set_dur(slot, value).
template <class MEM>
RPEG_HD PlanOut eval_plan(const rpeg_problem_t& P, const ClassView& c, const PlanHead& h, const VPlan* a, MEM& mem,
                          int ready_cap, uint32_t flags) {
  const rpeg_struct_t& st = P.st[h.structure];
  PlanOut out;
  bool err = c.h->error != 0, zero_div = false;
  const PlanMasks pm = plan_masks(a, st.n_vertex);
  uint8_t ovl[RPEG_MAX_V];
  for (int v = 0; v < RPEG_MAX_V; ++v) ovl[v] = (uint8_t)mask_row(pm.ovl, v);
  for (unsigned s = 0; s < c.h->n_slots; ++s) mem.set_dur(s, slot_duration(P, st, h.split, c.slot[s], a, &zero_div));
  err = err || zero_div;
  double makespan = 0.0;
  if (!err) makespan = list_schedule(c, mem, ovl, pm.dpne, st.n_vertex, ready_cap, &err);
  VMem vm[RPEG_MAX_V];
  const bool coresident = struct_coresident(st);
  for (int v = 0; v < st.n_vertex; ++v) vm[v] = vertex_memory(P, st.vertex[v], a[v], coresident);
  const VMemArray vma{vm};
  const double peak = device_peak_max(P, st, c.h->vorder, pm, vma);
  const bool stale_ok = stale_layout_ok(st, h, pm.ovl);
  const bool mem_ok = !(peak > P.cap);
  uint8_t mask = RPEG_MASK_VALID;
  if (stale_ok) mask |= RPEG_MASK_STALE_OK;
  if (mem_ok) mask |= RPEG_MASK_MEM_OK;
  if (err || makespan == 0.0) {  // Python raises ZeroDivisionError on a zero makespan (trace.py:51)
    out.makespan = out.score = __builtin_nan("");
    out.peak = peak;
    out.mask = (uint8_t)(mask | RPEG_MASK_ERROR);
    return out;
  }
  double score = P.score_num / makespan;
  if (!mem_ok) score = score * oom_penalty(peak, P.cap);
  if ((flags & RPEG_GATE_STALE) && !stale_ok) score = 0.0;
  out.makespan = makespan;
  out.peak = peak;
  out.score = score;
  out.mask = mask;
  return out;
}

}  // namespace rpeg
#endif
