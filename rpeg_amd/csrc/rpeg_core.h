// rpeg_core.h - per-plan arithmetic of the batched plan evaluator.
//
// Everything here is written once and compiled twice: as device code inside the HIP kernels and
// as host code for host-side unit checks.  All floating-point expressions keep the association
// and operand order of the reference's Python expressions, and the translation unit must be
// compiled with -ffp-contract=off so that no multiply-add is fused (Python never fuses).
//
// Reference files restated here:
//   RPEG/model/cost.py     node durations        (rpeg::op_time, comm_time, reshard_time)
//   RPEG/model/memory.py   per-vertex footprints (rpeg::vertex_memory) and per-device peaks
//   RPEG/model/hardware.py tier selection
//   RPEG/core/types.py, RPEG/search/evaluate.py  integer validity rules
//   RPEG/schedule/scheduler.py  list scheduler (rpeg::list_schedule)
#ifndef RPEG_CORE_H
#define RPEG_CORE_H

#include <stdint.h>
#include "../../include/rpeg_eval.h"

#if defined(__HIPCC__)
#define RPEG_HD __host__ __device__ inline
#else
#define RPEG_HD inline
#endif

namespace rpeg {

struct VPlan {  // plan fields of one vertex
  int dp, pp, tp, mb;
  int o[3];
  int e[3];
};

RPEG_HD int imin(int a, int b) { return a < b ? a : b; }
RPEG_HD int imax(int a, int b) { return a > b ? a : b; }
RPEG_HD double dmax(double a, double b) { return a > b ? a : b; }  // Python max(a, b): b only if b > a
RPEG_HD double dmin(double a, double b) { return b < a ? b : a; }  // Python min(a, b): b only if b < a
RPEG_HD int64_t cdiv64(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ------------------------------------------------------------------------------------- exp
// exp(x) as glibc's FMA build computes it (table of 2^(i/128) split into a rounded head and a
// relative tail, degree-5 polynomial, fused operations where an FMA-enabled build of that
// algorithm fuses them).  Valid for the finite, non-subnormal results the OOM penalty needs
// (|x| < 700).  math.exp of the reference's score (evaluate.py:398) is this function on the hosts
// the reference runs on, so the penalised score is reproduced bit for bit.
#include "rpeg_exp_table.inc"

RPEG_HD double exp_libm(double x) {
  const double inv_ln2_n = 0x1.71547652b82fep0 * 128.0;
  const double neg_ln2_hi_n = -0x1.62e42fefa0000p-8;
  const double neg_ln2_lo_n = -0x1.cf79abc9e3b3ap-47;
  const double shift = 0x1.8p52;
  const double c2 = 0x1.ffffffffffdbdp-2, c3 = 0x1.555555555543cp-3;
  const double c4 = 0x1.55555cf172b91p-5, c5 = 0x1.1111167a4d017p-7;
  double z = inv_ln2_n * x;
  double kd = z + shift;
  uint64_t ki;
  __builtin_memcpy(&ki, &kd, 8);
  kd -= shift;
  double r = __builtin_fma(kd, neg_ln2_lo_n, __builtin_fma(kd, neg_ln2_hi_n, x));
  uint64_t idx = 2 * (ki % 128);
  uint64_t tbits = exp_table(idx);
  uint64_t sbits = exp_table(idx + 1) + (ki << 45);
  double tail, scale;
  __builtin_memcpy(&tail, &tbits, 8);
  __builtin_memcpy(&scale, &sbits, 8);
  double r2 = r * r;
  double p23 = __builtin_fma(r, c3, c2);
  double p45 = __builtin_fma(r, c5, c4);
  double tmp = __builtin_fma(r2 * r2, p45, __builtin_fma(r2, p23, tail + r));
  return __builtin_fma(scale, tmp, scale);
}

// ------------------------------------------------------------------------------------- geometry
RPEG_HD int alloc_size(const VPlan& a) { return a.e[0] * a.e[1] * a.e[2]; }

RPEG_HD bool alloc_equal(const VPlan& a, const VPlan& b) {
  return a.o[0] == b.o[0] && a.o[1] == b.o[1] && a.o[2] == b.o[2] && a.e[0] == b.e[0] && a.e[1] == b.e[1] &&
         a.e[2] == b.e[2];
}

// lower.py:223-239
RPEG_HD bool alloc_disjoint(const VPlan& a, const VPlan& b) {
  for (int ax = 0; ax < 3; ++ax)
    if (a.o[ax] + a.e[ax] <= b.o[ax] || b.o[ax] + b.e[ax] <= a.o[ax]) return true;
  return false;
}

// lower.py:242-262
RPEG_HD int alloc_overlap_size(const VPlan& a, const VPlan& b) {
  int vol = 1;
  for (int ax = 0; ax < 3; ++ax) {
    int lo = imax(a.o[ax], b.o[ax]);
    int hi = imin(a.o[ax] + a.e[ax], b.o[ax] + b.e[ax]);
    if (hi <= lo) return 0;
    vol *= hi - lo;
  }
  return vol;
}

// core/types.py:16-57; returns false for "None"
RPEG_HD bool packing_geometry(int dp, int pp, int tp, int G, int* g_ext, int* nodes) {
  int s = imin(pp, G / tp);
  if (s == 0 || pp % s != 0) return false;
  int per_rep = s * tp, span = pp / s;
  if (span != 1) { *g_ext = G; *nodes = dp * span; return true; }
  int fit = G / per_rep;
  if (dp <= fit) { *g_ext = dp * per_rep; *nodes = 1; return true; }
  if (dp % fit == 0) { *g_ext = G; *nodes = dp / fit; return true; }
  return false;
}

// evaluate.py:172-196 for one vertex (coverage is implied by the dense plan tensor)
RPEG_HD bool vertex_valid(const rpeg_problem_t& P, const VPlan& a, int L) {
  if (a.dp < 1 || a.pp < 1 || a.tp < 1 || a.mb < 1) return false;
  if (P.B % a.dp != 0 || P.G % a.tp != 0 || L % a.pp != 0) return false;
  if (a.pp == 1) { if (a.mb != 1) return false; }
  else if ((P.B / a.dp) % a.mb != 0) return false;
  if (a.tp > P.G) return false;
  int g_ext, nodes;
  if (!packing_geometry(a.dp, a.pp, a.tp, P.G, &g_ext, &nodes)) return false;
  if (a.e[2] != g_ext) return false;
  // (r_ext, n_ext) must be one of rectangular_node_layouts(nodes, R, N)  (types.py:60-85)
  if (nodes <= 0) return false;
  if (a.e[0] < 1 || a.e[0] > imin(P.R, nodes) || nodes % a.e[0] != 0) return false;
  if (a.e[1] != nodes / a.e[0] || a.e[1] > P.N) return false;
  if (a.o[0] < 0 || a.o[1] < 0 || a.o[2] < 0) return false;
  if (a.o[0] + a.e[0] > P.R || a.o[1] + a.e[1] > P.N || a.o[2] + a.e[2] > P.G) return false;
  return true;
}

// ------------------------------------------------------------------------------------- tiers
// hardware.py:70-110: bounding span of one or two allocations
RPEG_HD int tier_of(const VPlan& a, const VPlan* b) {
  int r0 = a.o[0], r1 = a.o[0] + a.e[0], n0 = a.o[1], n1 = a.o[1] + a.e[1];
  if (b) {
    r0 = imin(r0, b->o[0]); r1 = imax(r1, b->o[0] + b->e[0]);
    n0 = imin(n0, b->o[1]); n1 = imax(n1, b->o[1] + b->e[1]);
  }
  if (r1 - r0 > 1) return 2;
  if (n1 - n0 > 1) return 1;
  return 0;
}
RPEG_HD double coll_alpha(const rpeg_problem_t& P, int t) { return P.hw[RPEG_HW_A_COLL_G + 2 * t]; }
RPEG_HD double coll_beta(const rpeg_problem_t& P, int t) { return P.hw[RPEG_HW_B_COLL_G + 2 * t]; }
RPEG_HD double p2p_alpha(const rpeg_problem_t& P, int t) { return P.hw[RPEG_HW_A_P2P_G + 2 * t]; }
RPEG_HD double p2p_beta(const rpeg_problem_t& P, int t) { return P.hw[RPEG_HW_B_P2P_G + 2 * t]; }

// ------------------------------------------------------------------------------------- cost model
// cost.py:147-159
RPEG_HD int effective_mb(const rpeg_opconst_t& oc, const VPlan& a) {
  return imax(1, imin(a.mb, oc.n_eff / imax(1, a.dp)));
}

struct PipeComm {  // closure state of pp_p2p / tp_allreduce in cost.py:562-601
  int e_total, e_inter, e_intra;
  double a_in, b_in, a_x, b_x, a_tp, b_tp;
};

RPEG_HD double tp_allreduce(const PipeComm& c, double M, int p) {
  return (double)(2 * (p - 1)) * c.a_tp + (double)(2 * (p - 1)) / (double)p * M * c.b_tp;
}

RPEG_HD double pp_p2p(const PipeComm& c, double M, int64_t n_steps) {
  if (c.e_total == 0 || n_steps == 0) return 0.0;
  double intra = ((double)c.e_intra / (double)c.e_total) * (double)n_steps * (c.a_in + M * c.b_in);
  double inter = ((double)c.e_inter / (double)c.e_total) * (double)n_steps * (c.a_x + M * c.b_x);
  return intra + inter;
}

// cost.py:655-686 for the collectives the path uses; kind: 0 all-gather/reduce-scatter, 1 all-reduce, 2 all-to-all
RPEG_HD double collective(double alpha, double beta, int kind, double M, int p) {
  if (kind == 0) return (double)(p - 1) * alpha + (double)(p - 1) / (double)p * M * beta;
  if (kind == 1) return (double)(2 * (p - 1)) * alpha + (double)(2 * (p - 1)) / (double)p * M * beta;
  return (double)(p - 1) * alpha + M * beta;
}

// cost.py:538-652
RPEG_HD double intra_comm(const rpeg_problem_t& P, const rpeg_vertex_t& vx, const rpeg_opconst_t& oc,
                          const VPlan& a, int m) {
  const rpeg_model_t& md = P.model[vx.model];
  const int pd = a.dp, pp = a.pp, pt = a.tp;
  const int64_t d = md.d, sb = md.sb;
  const int64_t S = P.S, T = P.T;
  PipeComm c;
  c.a_tp = P.hw[RPEG_HW_A_COLL_G];
  c.b_tp = P.hw[RPEG_HW_B_COLL_G];
  int s = a.e[2] / pt;
  int per_rep = s > 0 ? (pp + s - 1) / s : pp;
  c.e_total = pp - 1;
  c.e_inter = per_rep - 1;
  c.e_intra = c.e_total - c.e_inter;
  int t_inter = a.e[0] > 1 ? 2 : (a.e[1] > 1 ? 1 : 0);
  c.a_x = p2p_alpha(P, t_inter);
  c.b_x = p2p_beta(P, t_inter);
  c.a_in = p2p_alpha(P, 0);
  c.b_in = p2p_beta(P, 0);
  const double Lpp = (double)md.L / (double)pp;
  const double den = (double)((int64_t)pd * m);
  const int64_t n = oc.n_eff;
  if (vx.role == RPEG_ROLE_GEN) {
    if (oc.sub) {
      const int64_t steps = oc.steps;
      double cost = 0.0;
      if (oc.prefill) {
        double M1 = (double)(n * S * d * sb) / den;
        cost += pp_p2p(c, M1, m + pp - 2);
        cost += 2.0 * Lpp * (double)m * tp_allreduce(c, M1, pt);
      }
      double M2 = (double)(n * d * sb) / den;
      cost += pp_p2p(c, M2, steps * (int64_t)(m + pp - 2));
      cost += (double)(2 * steps) * Lpp * (double)m * tp_allreduce(c, M2, pt);
      return cost;
    }
    double M1 = (double)(n * S * d * sb) / den;
    double M2 = (double)(n * d * sb) / den;
    return pp_p2p(c, M1, m + pp - 2) + pp_p2p(c, M2, (T - 1) * (int64_t)(m + pp - 2)) +
           2.0 * Lpp * (double)m * tp_allreduce(c, M1, pt) +
           (double)(2 * (T - 1)) * Lpp * (double)m * tp_allreduce(c, M2, pt);
  }
  if (vx.role == RPEG_ROLE_INF) {
    double M = (double)(n * (S + T) * d * sb) / den;
    return pp_p2p(c, M, m + pp - 2) + 2.0 * Lpp * (double)m * tp_allreduce(c, M, pt);
  }
  // training
  int64_t params = md.params_formula + ((md.kind == RPEG_MODEL_CRITIC || md.kind == RPEG_MODEL_AC_SHARE) ? d : 0);
  double msg = (double)(params * sb) / (double)((int64_t)pp * pt);
  int tc = tier_of(a, nullptr);
  double al = coll_alpha(P, tc), be = coll_beta(P, tc);
  double dp_comm;
  if (P.optimizer_stage == 0) dp_comm = collective(al, be, 1, msg, pd);
  else if (P.optimizer_stage == 1) dp_comm = collective(al, be, 1, msg, pd) + collective(al, be, 0, msg, pd);
  else dp_comm = collective(al, be, 0, msg, pd) + collective(al, be, 0, msg, pd);
  double n_tp = P.ckpt ? 6.0 : 4.0;
  double M = (double)((int64_t)P.B * P.K * (S + T) * d * sb) / den;
  return dp_comm + pp_p2p(c, M, m + 2 * pp - 3) + n_tp * Lpp * (double)m * tp_allreduce(c, M, pt);
}

// cost.py:212-269
RPEG_HD double non_gemm(const rpeg_problem_t& P, const rpeg_vertex_t& vx, const rpeg_opconst_t& oc,
                        const VPlan& a, int m) {
  const double cst = P.hw[RPEG_HW_NG_CONST], scl = P.hw[RPEG_HW_NG_SCALE];
  if (cst == 0.0 && scl == 0.0) return 0.0;
  if (vx.role == RPEG_ROLE_GEN) return 0.0;
  const double Lpp = (double)P.model[vx.model].L / (double)a.pp;
  double b_local = (double)oc.n_eff / (double)((int64_t)a.dp * m);
  double bcal = P.hw[RPEG_HW_NG_BCAL];
  double scale = bcal > 0 ? b_local / bcal : 1.0;
  double at_tp = Lpp * (cst + scl / (double)a.tp);
  double at_tp1 = Lpp * (cst + scl) / (double)a.tp;
  double extra = (at_tp - at_tp1) * scale;
  if (vx.role == RPEG_ROLE_TRAIN) extra *= P.ckpt ? 4.0 : 3.0;
  return dmax(0.0, extra);
}

// cost.py:271-328, 406-444 (inference / training) and :330-404 (generation)
RPEG_HD double effective_flops(const rpeg_problem_t& P, const rpeg_vertex_t& vx, const rpeg_opconst_t& oc,
                               const VPlan& a, int m, bool* zero_div) {
  const rpeg_model_t& md = P.model[vx.model];
  const int pd = a.dp, pp = a.pp, pt = a.tp;
  const double flops = P.hw[RPEG_HW_FLOPS], bw = P.hw[RPEG_HW_BW], m_half = P.hw[RPEG_HW_M_HALF];
  const double Lpp = (double)md.L / (double)pp;
  const double b_local = (double)oc.n_eff / (double)((int64_t)pd * m);
  const double i_star = flops / bw;
  const double wl = (double)md.w_layer;
  const double sb = (double)md.sb;
  const double omega_W = (Lpp / (double)pt) * wl * sb;
  const int64_t S = P.S, T = P.T, d = md.d;
  if (vx.role != RPEG_ROLE_GEN) {
    const int64_t seq = S + T;
    double fl = b_local * (double)seq * (2.0 * Lpp / (double)pt) * (double)(md.w_layer + seq * d);
    double omega_A = 2.0 * b_local * (double)seq * (double)d * Lpp * sb;
    double tot = omega_W + omega_A;
    double I = tot <= 0 ? __builtin_inf() : fl / tot;
    double M_eff = b_local * (double)seq;
    double eta_b = m_half > 0 ? M_eff / (M_eff + m_half) : 1.0;
    double eta_t = 1.0;
    double k_half = P.hw[RPEG_HW_K_HALF];
    if (pt > 1 && k_half > 0) {
      double k_min = (double)imin(md.d / pt, md.d_ff / pt);
      eta_t = k_min / (k_min + k_half);
    }
    double eta = eta_b * eta_t;
    return I >= i_star ? flops * eta : I * bw;
  }
  const double P_all = (double)((int64_t)pd * pp * pt);
  const double eff_w = P.hw[RPEG_HW_DECODE_EFF];
  const double eff_kv = dmin(1.0, eff_w * 3.5);
  double total = 0.0;
  if (oc.prefill) {
    double bs = b_local * (double)S;
    double eta = m_half > 0 ? bs / (bs + m_half) : 1.0;
    double fl = b_local * (double)S * (2.0 * Lpp / (double)pt) * (double)(md.w_layer + S * d);
    double omega_A = 2.0 * b_local * (double)S * (double)d * Lpp * sb;
    double I = (omega_W + omega_A) > 0 ? fl / (omega_W + omega_A) : __builtin_inf();
    double F = I >= i_star ? flops * eta : I * bw;
    total += F > 0 ? oc.W_prefill / (P_all * F) : 0.0;
  }
  if (oc.steps > 0) {
    double eta = m_half > 0 ? b_local / (b_local + m_half) : 1.0;
    double fl = b_local * (2.0 * Lpp / (double)pt) * ((double)md.w_layer + oc.avg_past * (double)d);
    double omega_A = 2.0 * b_local * (double)d * Lpp * sb;
    double omega_KV = 2.0 * oc.avg_past * ((double)d / (double)pt) * sb * b_local * Lpp;
    double omega = omega_W + omega_A + omega_KV;
    double eff = omega > 0 ? (omega_W * eff_w + omega_KV * eff_kv + omega_A * 1.0) / omega : eff_w;
    double bwd = bw * eff;
    double I = omega > 0 ? fl / omega : __builtin_inf();
    double F = I >= i_star ? flops * eta : I * bwd;
    double W_decode = oc.prefill ? oc.W - oc.W_prefill : oc.W;
    total += F > 0 ? W_decode / (P_all * F) : 0.0;
  }
  if (total > 0) return oc.W / (P_all * total);
  (void)zero_div;
  return flops;
}

// cost.py:161-193
RPEG_HD double op_time(const rpeg_problem_t& P, const rpeg_vertex_t& vx, const rpeg_opconst_t& oc, const VPlan& a,
                       bool* zero_div) {
  const int pd = a.dp, pp = a.pp, pt = a.tp;
  const int m = effective_mb(oc, a);
  const double bubble = (double)(m + pp - 1) / (double)m;
  const double F = effective_flops(P, vx, oc, a, m, zero_div);
  const double den = F * (double)pd * (double)pp * (double)pt;
  if (den == 0.0) *zero_div = true;  // Python raises ZeroDivisionError here
  double t = (oc.W / den) * bubble + intra_comm(P, vx, oc, a, m);
  t += non_gemm(P, vx, oc, a, m);
  double scale = P.hw[RPEG_HW_SCALE_INF];
  if (vx.role == RPEG_ROLE_GEN) scale = P.hw[RPEG_HW_SCALE_GEN];
  if (vx.role == RPEG_ROLE_TRAIN) {
    scale = P.hw[RPEG_HW_SCALE_TRAIN];
    int odp = P.optimizer_stage >= 1 ? pd : 1;
    double per_rank = (double)P.model[vx.model].params_formula / (double)((int64_t)odp * pp * pt);
    t += (per_rank * 18.0) / P.hw[RPEG_HW_BW];
  }
  return t * scale;
}

// cost.py:446-462
RPEG_HD double comm_time(const rpeg_problem_t& P, const VPlan& src, const VPlan& dst, int64_t payload,
                         bool is_weight) {
  int t = tier_of(src, &dst);
  int p_min = imin(alloc_size(src), alloc_size(dst));
  double v = p2p_alpha(P, t) + ((double)payload / (double)p_min) * p2p_beta(P, t);
  return is_weight ? v * P.hw[RPEG_HW_W_COMM_SCALE] : v + P.hw[RPEG_HW_ACT_OVERHEAD];
}

// cost.py:464-479 (both allocations are identical)
RPEG_HD double reshard_time(const rpeg_problem_t& P, const VPlan& a, int model) {
  int Pn = alloc_size(a);
  int64_t payload = P.model[model].n_params * P.model[model].sb;
  int t = tier_of(a, nullptr);
  double M = (double)payload / (double)Pn;
  return P.hw[RPEG_HW_RESHARD_SCALE] * collective(coll_alpha(P, t), coll_beta(P, t), 2, M, Pn);
}

// lower.py:711-718: payload of a publication COMM
RPEG_HD int64_t pub_payload(const rpeg_problem_t& P, const VPlan& src, const VPlan& dst, int model) {
  int64_t full = P.model[model].n_params * P.model[model].sb;
  int64_t n_max = imax(alloc_size(src), alloc_size(dst));
  int64_t n_ov = alloc_overlap_size(src, dst);
  if (n_max <= 0) return full;
  // Python: full * (n_max - n_ov) // n_max on unbounded ints; the product stays below 2^63 here
  return full * (n_max - n_ov) / n_max;
}

// ------------------------------------------------------------------------------------- memory
struct VMem {       // per-vertex quantities of memory.py:367-553
  int64_t w_shard;  // parameters per device
  double mem_w;     // _mem_weights
  double opt;       // 12 * w_shard / opt_dp
  double x1;        // gradients (training) | KV cache (generation) | 0
  double x2;        // activations
  double extra;     // role extras as the per-device pass sums them: x1 + x2 (x2 alone for inference)
};

RPEG_HD int isqrt_small(int n) {
  int r = 0;
  while ((r + 1) * (r + 1) <= n) ++r;
  return r;
}

// `dp_for_opt`: the co-resident sum model (memory.py:706-742) needs the vertex's dp where the worker-liveness model
// needs its optimizer shard; the record then carries (double)dp in `opt`.
RPEG_HD VMem vertex_memory(const rpeg_problem_t& P, const rpeg_vertex_t& vx, const VPlan& a, bool dp_for_opt = false) {
  const rpeg_model_t& md = P.model[vx.model];
  const int dp = a.dp, pp = a.pp, tp = a.tp;
  const int64_t emb = (int64_t)md.V * md.d, head = md.d;
  const int64_t L_pp = cdiv64(md.L, pp);
  const int64_t split = L_pp * md.w_layer;
  // memory.py:312-365: first pipeline stage with the largest total
  int64_t rest;
  if (md.kind == RPEG_MODEL_ACTOR || md.kind == RPEG_MODEL_REFERENCE) rest = pp == 1 ? 2 * emb : emb;
  else if (md.kind == RPEG_MODEL_AC_SHARE) rest = pp == 1 ? 2 * emb + head : emb + head;
  else rest = pp == 1 ? emb + head : (emb >= head ? emb : head);
  VMem r;
  r.w_shard = cdiv64(split, tp) + rest;
  const double sb = (double)md.sb;
  r.mem_w = (double)(r.w_shard * md.sb);
  int odp = P.optimizer_stage >= 1 ? dp : 1;
  r.opt = dp_for_opt ? (double)dp : (double)(12 * r.w_shard) / (double)odp;
  const double d = (double)md.d;
  const int64_t BK = (int64_t)P.B * P.K;
  const double b_local = (double)BK / (double)((int64_t)dp * a.mb);
  const double attn = (double)(2 * md.d) + (double)(6 * md.d) / (double)tp;
  const double ffn = (double)(2 * md.d) + (double)(2 * (int64_t)md.d_ff) / (double)tp;
  if (vx.role == RPEG_ROLE_TRAIN) {
    int gdp = P.optimizer_stage >= 2 ? dp : 1;
    double grad = (double)(md.sb * r.w_shard) / (double)gdp;
    double layer_peak = dmax(attn, ffn);
    double per_token;
    if (P.ckpt) {
      int c = imax(1, isqrt_small((int)L_pp));
      int64_t n_ckpt = cdiv64(L_pp, c);
      per_token = (double)(n_ckpt * md.d) + (double)c * layer_peak;
    } else {
      per_token = (double)L_pp * layer_peak;
    }
    double per_mb = sb * b_local * (double)(P.S + P.T) * per_token;
    double act = (double)imin(a.mb, pp) * per_mb;
    r.x1 = grad;
    r.x2 = act;
    r.extra = grad + act;
    return r;
  }
  const int64_t seq = vx.role == RPEG_ROLE_GEN ? P.S : P.S + P.T;
  double per_token = dmax(dmax(attn, ffn), (double)(md.d + md.V));
  double act_inf = sb * b_local * (double)seq * per_token;
  if (vx.role == RPEG_ROLE_GEN) {
    double kv = (double)(2 * md.sb) * ((double)P.B / (double)dp) * (double)P.K * (double)(P.S + P.T) *
                ((double)md.L / (double)pp) * (d / (double)tp);
    r.x1 = kv;
    r.x2 = act_inf;
    r.extra = kv + act_inf;
  } else {
    r.x1 = 0.0;
    r.x2 = act_inf;
    r.extra = act_inf;
  }
  return r;
}

// memory.py:273-288
RPEG_HD double isolated_peak(const rpeg_vertex_t& vx, const VMem& m) {
  if (vx.role == RPEG_ROLE_TRAIN) return m.mem_w + m.opt + m.x1 + m.x2;
  if (vx.role == RPEG_ROLE_GEN) return m.mem_w + m.x1 + m.x2;
  return m.mem_w + m.x2;
}

// Pair relations of one plan packed 8 bits per vertex: bit (8*u + v) of the word.
struct PlanMasks {
  uint64_t ovl;  // allocations of u and v intersect (u == v included)
  uint64_t eq;   // allocations of u and v are identical
  uint64_t dpne; // dp of u differs from dp of v
};
RPEG_HD unsigned mask_row(uint64_t m, int v) { return (unsigned)(m >> (8 * v)) & 0xFFu; }

// Plan-independent vertex sets of one structure (bit v = vertex v).
struct StructMasks {                // (rows of 8 bits packed into words, read with mask_row: byte arrays indexed with
                                    // run-time values would live in scratch memory on the GPU)
  uint64_t same_model;              // row v: vertices invoking the same model as v
  uint64_t train_same;              // row v: TRAIN vertices of v's model
  uint64_t before;                  // row i: vertices that precede order[i] in first-appearance order
  uint8_t train, trainable;         // TRAIN vertices; vertices of trainable models
  bool coresident;                  // the memory model lists no trainable model at all: co-resident sum model
};
// NodeMemoryModel.trainable is empty (memory.py:647: `use_worker_liveness_model = len(mem_model.trainable) > 0`)
RPEG_HD bool struct_coresident(const rpeg_struct_t& st) {
  bool any = false;
  for (unsigned m = 0; m < sizeof(st.mem_trainable); ++m) any = any || st.mem_trainable[m] != 0;
  return !any;
}
template <class ORD>   // `order`: the vertices in order of first appearance, a byte array or anything indexable like one
RPEG_HD StructMasks struct_masks(const rpeg_struct_t& st, const ORD& order) {
  StructMasks m;
  m.train = m.trainable = 0;
  unsigned seen = 0;
  m.same_model = m.train_same = m.before = 0;
  for (int v = 0; v < st.n_vertex; ++v) {
    if (st.vertex[v].role == RPEG_ROLE_TRAIN) m.train |= (uint8_t)(1u << v);
    if (st.mem_trainable[st.vertex[v].model]) m.trainable |= (uint8_t)(1u << v);
    for (int w = 0; w < st.n_vertex; ++w)
      if (st.vertex[w].model == st.vertex[v].model) {
        m.same_model |= 1ull << (8 * v + w);
        if (st.vertex[w].role == RPEG_ROLE_TRAIN) m.train_same |= 1ull << (8 * v + w);
      }
  }
  for (int i = 0; i < st.n_vertex; ++i) { m.before |= (uint64_t)seen << (8 * i); seen |= 1u << order[i]; }
  m.coresident = struct_coresident(st);
  return m;
}

// Largest per-device peak (memory.py:608-841, worker-liveness model).  A device's peak depends
// only on the set of vertices whose allocation contains it, and grows with that set; boxes have
// the Helly property, so the maximum over devices is the maximum over the maximal cliques of the
// pairwise-overlap graph.  `order` lists the vertices in order of first appearance among the
// lowered operator nodes (it fixes the insertion order of the reference's dicts and hence the
// order of its float sums).  VM provides w_shard(v) (as double), mem_w(v), opt(v), extra(v).
// Peak of the devices covered by exactly the vertex set M.
template <class VM, class ORD>
RPEG_HD double device_class_peak(const rpeg_problem_t& P, const rpeg_struct_t& st, const ORD& order,
                                 const StructMasks& sm, const PlanMasks& pm, const VM& vm, unsigned M) {
  const int nv = st.n_vertex;
  double persistent = 0.0;
  int groups = 0;
  for (int i = 0; i < nv; ++i) {  // distinct (model, allocation) worker keys
    const int v = order[i];
    if (!((M >> v) & 1u)) continue;
    if ((mask_row(pm.eq, v) & M & mask_row(sm.same_model, v) & mask_row(sm.before, i)) == 0) ++groups;
  }
  if (sm.coresident) {
    // memory.py:706-742: every model present keeps its static footprint -- its largest shard among the vertices
    // here; with a training vertex of the model here also optimizer state and gradients at that vertex's dp (the
    // last such vertex in node order) -- summed in order of first appearance; the transients share their room.
    // vm.opt(v) carries dp of vertex v in this mode.
    double stat = 0.0, transient = 0.0;
    for (int i = 0; i < nv; ++i) {
      const int v = order[i];
      if (!((M >> v) & 1u)) continue;
      transient = dmax(transient, vm.extra(v));
      const unsigned same = M & mask_row(sm.same_model, v);
      if (same & mask_row(sm.before, i)) continue;   // the model's entry exists
      double wmax = 0.0, dp = vm.opt(v);
      bool trained = false;
      for (int j = 0; j < nv; ++j) {
        const int w = order[j];
        if (!((same >> w) & 1u)) continue;
        wmax = dmax(wmax, vm.w_shard(w));
        if ((sm.train >> w) & 1u) { trained = true; dp = vm.opt(w); }
      }
      const double sbw = (double)P.model[st.vertex[v].model].sb * wmax;
      double x = sbw;
      if (trained) x = (sbw + 12.0 * wmax / (P.optimizer_stage >= 1 ? dp : 1.0)) + sbw / (P.optimizer_stage >= 2 ? dp : 1.0);
      stat += x;
    }
    double peak = ((double)groups * P.group_overhead + stat) + transient;
    if (P.max_groups > 0 && groups > P.max_groups) peak = __builtin_inf();
    return peak;
  }
  for (int i = 0; i < nv; ++i) {  // optimizer shards of the training vertices
    const int v = order[i];
    if (((M & sm.train & sm.trainable) >> v) & 1u) persistent += vm.opt(v);
  }
  unsigned serving = 0;           // serving shards: one per worker key that is not a training worker
  for (int i = 0; i < nv; ++i) {
    const int v = order[i];
    if (!(((M & sm.trainable & ~(unsigned)sm.train) >> v) & 1u)) continue;
    const unsigned same_key = mask_row(pm.eq, v) & M & mask_row(sm.same_model, v);
    if (same_key & mask_row(sm.train_same, v)) continue;
    const bool first = (same_key & serving) == 0;
    serving |= 1u << v;
    if (!first) continue;
    double ws = 0.0;
    for (int w = 0; w < nv; ++w)
      if (((same_key & ~(unsigned)sm.train) >> w) & 1u) ws = dmax(ws, vm.w_shard(w));
    persistent += (double)P.model[st.vertex[v].model].sb * ws;
  }
  for (int i = 0; i < nv; ++i) {  // frozen weights: one entry per model, its largest shard
    const int v = order[i];
    if (!(((M & ~(unsigned)sm.trainable) >> v) & 1u)) continue;
    const unsigned same = M & mask_row(sm.same_model, v);
    if (same & mask_row(sm.before, i)) continue;
    double wb = 0.0;
    for (int w = 0; w < nv; ++w)
      if ((same >> w) & 1u) wb = dmax(wb, vm.mem_w(w));
    persistent += wb;
  }
  double top = 0.0;
  for (int i = 0; i < nv; ++i) {
    const int v = order[i];
    if (!((M >> v) & 1u)) continue;
    const bool resident = !((sm.trainable >> v) & 1u) || (mask_row(pm.eq, v) & serving & mask_row(sm.same_model, v)) != 0;
    const double c = resident ? vm.extra(v) : vm.mem_w(v) + vm.extra(v);
    top = dmax(top, c);
  }
  double peak = (double)groups * P.group_overhead + persistent + top;
  if (P.max_groups > 0 && groups > P.max_groups) peak = __builtin_inf();  // memory.py:699-704
  return peak;
}

// The maximal cliques of the overlap graph among the vertex sets that contain no vertex below V, given the
// set M of the vertices below V already chosen and c, the vertices that intersect every one of those: bit M of
// `found` is set for every maximal clique M.  The relation is symmetric, so a vertex outside M that intersects
// every member of M is in c, and one inside M that misses a member is not: M is a maximal clique exactly when
// c == M.  (All 63 sets in 63 ANDs and 63 comparisons; rows of vertices the structure does not have are zero.)
template <int V, unsigned M>
RPEG_HD void clique_sets(const unsigned (&row)[RPEG_MAX_V], unsigned c, uint64_t& found) {
  if constexpr (V == RPEG_MAX_V) {
    if (M != 0u && c == M) found |= 1ull << M;
  } else {
    clique_sets<V + 1, M>(row, c, found);
    clique_sets<V + 1, M | (1u << V)>(row, c & row[V], found);
  }
}

template <class VM, class ORD>
RPEG_HD double device_peak_max(const rpeg_problem_t& P, const rpeg_struct_t& st, const ORD& order,
                               const PlanMasks& pm, const VM& vm) {
  static_assert(RPEG_MAX_V <= 6, "a vertex set is one bit of a 64-bit word below");
  const StructMasks sm = struct_masks(st, order);
  const unsigned full = (1u << st.n_vertex) - 1u;
  double best = -1.0;
  // First the maximal cliques of this plan, then their peaks in ascending order of the sets.  On the GPU the lanes
  // of a wavefront carry different plans: finding the sets is cheap, the peak of a set is not, and this way a
  // wavefront computes as many peaks as its plan with the most cliques has, not one for every set that is a clique
  // in some lane.
  unsigned row[RPEG_MAX_V];
  for (int v = 0; v < RPEG_MAX_V; ++v) row[v] = v < st.n_vertex ? (mask_row(pm.ovl, v) & full) : 0u;
  uint64_t found = 0;
  clique_sets<0, 0u>(row, full, found);
  while (found) {
    const unsigned M = (unsigned)__builtin_ctzll(found);
    found &= found - 1ull;
    const double peak = device_class_peak(P, st, order, sm, pm, vm, M);
    if (peak > best) best = peak;
  }
  return best;
}

// evaluate.py:396-401
RPEG_HD double oom_penalty(double peak, double cap) {
  double over = dmax(0.0, peak / cap - 1.0);
  double x = -40.0 * over;
  // exp(x) < 1e-12 for every x < -27.7, so the clamp decides there and exp_libm stays inside its range
  double e = x < -64.0 ? 0.0 : exp_libm(x);
  return dmax(e, 1e-12);
}

}  // namespace rpeg
#endif
