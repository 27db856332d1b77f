// cpu_port.cpp - host build of the evaluator's per-plan arithmetic.  TEST INFRASTRUCTURE ONLY.
//
// Compiles the same headers the HIP kernels are built from (rpeg_amd/csrc/rpeg_*.h) with the host
// compiler and runs them plan by plan.  It exists so that the arithmetic can be checked against the
// Python oracle without a GPU and timed as a multi-core CPU baseline; the shipped library never
// loads or links it.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../rpeg_amd/csrc/rpeg_lower.h"
#include "../rpeg_amd/csrc/rpeg_plan.h"
#include "../rpeg_amd/csrc/rpeg_sa.h"

using namespace rpeg;

namespace {
struct HostMem {
  std::vector<double> t, r, d;
  std::vector<uint8_t> deg;
  std::vector<uint16_t> ready;
  int max_ready = 0;
  void fit(const ClassHdr* h) {
    t.assign(h->n_nodes, 0.0); r.assign(h->n_nodes, 0.0); deg.assign(h->n_nodes, 0);
    d.assign(h->n_slots, 0.0); ready.assign(h->n_nodes + 1, 0);
  }
  double& time(int i) { return t[i]; }
  double& rank(int i) { return r[i]; }
  uint8_t& indeg(int i) { return deg[i]; }
  double dur(int s) const { return d[s]; }
  void set_dur(int s, double v) { d[s] = v; }
  uint16_t& rd_node(int j) { if (j + 1 > max_ready) max_ready = j + 1; return ready[j]; }
  std::vector<double>* trace_start = nullptr;
  std::vector<double>* trace_finish = nullptr;
  void on_schedule(int v, double s, double f) { if (trace_start) { (*trace_start)[v] = s; (*trace_finish)[v] = f; } }
};

struct Port {
  rpeg_problem_t P;
  std::unordered_map<uint64_t, LoweredClass> classes;
  std::mutex mu;
  std::string err;
  const LoweredClass* get(uint64_t sig) {
    std::lock_guard<std::mutex> g(mu);
    auto it = classes.find(sig);
    if (it != classes.end()) return &it->second;
    return &(classes[sig] = lower_class(P, sig));
  }
};
}  // namespace

extern "C" {

void* port_create(const rpeg_problem_t* p) {
  Port* e = new Port();
  e->P = *p;
  return e;
}
void port_destroy(void* h) { delete (Port*)h; }
const char* port_error(void* h) { return ((Port*)h)->err.c_str(); }
long port_n_classes(void* h) { return (long)((Port*)h)->classes.size(); }

// host arrays, same layout as the device tensors; returns 0 or -1
int port_eval(void* h, uint64_t n, const int16_t* vert, const uint8_t* head, uint64_t stride, uint32_t flags,
              double* makespan, double* peak, double* score, uint8_t* mask, uint64_t* sig_out, int32_t* max_ready,
              int threads, double* mass) {
  Port* e = (Port*)h;
  int rc = 0;
  int mr = 0;
#pragma omp parallel for schedule(dynamic, 64) num_threads(threads) reduction(max : mr)
  for (int64_t i = 0; i < (int64_t)n; ++i) {
    PlanHead ph = load_head(head, stride, i);
    VPlan a[RPEG_MAX_V];
    std::memset(a, 0, sizeof a);
    const int nvs = (ph.structure >= 0 && ph.structure < e->P.n_struct) ? e->P.st[ph.structure].n_vertex : 0;
    for (int v = 0; v < nvs; ++v) load_vertex(vert, stride, i, v, &a[v]);
    PlanOut o;
    uint64_t sig = SIG_INVALID;
    if (!plan_valid(e->P, ph, a)) {
      o.makespan = o.peak = o.score = NAN;
      o.mask = 0;
    } else {
      sig = plan_signature(e->P, ph.structure, ph.split, ph.tau0, ph.tau1, a);
      try {
        const LoweredClass* lc = e->get(sig);
        ClassView cv = class_view(lc->blob.data());
        HostMem mem;
        mem.fit(cv.h);
        std::vector<double> ts, tf;
        if (mass) {
          ts.assign(cv.h->n_nodes, 0.0); tf.assign(cv.h->n_nodes, 0.0);
          mem.trace_start = &ts; mem.trace_finish = &tf;
        }
        o = eval_plan(e->P, cv, ph, a, mem, (int)cv.h->n_nodes + 1, flags);
        if (mem.max_ready > mr) mr = mem.max_ready;
        if (mass) {
          double m[RPEG_MAX_V];
          if (o.mask & RPEG_MASK_ERROR) for (double& x : m) x = NAN;
          else critical_mass(cv, [&](int k) { return tf[k]; }, [&](int k) { return ts[k]; }, m);
          for (int x = 0; x < RPEG_MAX_V; ++x) mass[i * RPEG_MAX_V + x] = m[x];
        }
      } catch (const std::exception& ex) {
#pragma omp critical
        { e->err = ex.what(); rc = -1; }
        o.makespan = o.peak = o.score = NAN;
        o.mask = RPEG_MASK_VALID | RPEG_MASK_ERROR;
      }
    }
    if (makespan) makespan[i] = o.makespan;
    if (peak) peak[i] = o.peak;
    if (score) score[i] = o.score;
    if (mask) mask[i] = o.mask;
    if (sig_out) sig_out[i] = sig;
    if (mass && sig == SIG_INVALID)
      for (int x = 0; x < RPEG_MAX_V; ++x) mass[i * RPEG_MAX_V + x] = NAN;
  }
  if (max_ready) *max_ready = mr;
  return rc;
}

// per-node view of one plan: kinds, vertices, steps, durations, and the class sizes
int port_lower(void* h, const int16_t* vert, const uint8_t* head, int32_t* kind, int32_t* vertex, int32_t* step,
               int32_t* sub, double* dur, int32_t* edges, int32_t cap, int32_t* n_edges) {
  Port* e = (Port*)h;
  PlanHead ph = load_head(head, 1, 0);
  VPlan a[RPEG_MAX_V];
  std::memset(a, 0, sizeof a);
  if (ph.structure < 0 || ph.structure >= e->P.n_struct) return -1;
  for (int v = 0; v < e->P.st[ph.structure].n_vertex; ++v) load_vertex(vert, 1, 0, v, &a[v]);
  if (!plan_valid(e->P, ph, a)) return -1;
  uint64_t sig = plan_signature(e->P, ph.structure, ph.split, ph.tau0, ph.tau1, a);
  const LoweredClass* lc;
  try { lc = e->get(sig); } catch (const std::exception& ex) { e->err = ex.what(); return -2; }
  int n = (int)lc->nodes.size();
  if (n > cap || (int)lc->edges.size() > cap) return -3;
  ClassView cv = class_view(lc->blob.data());
  bool zd = false;
  for (int i = 0; i < n; ++i) {
    kind[i] = lc->nodes[i].kind; vertex[i] = lc->nodes[i].kind == 0 ? lc->nodes[i].vertex : lc->nodes[i].a1;
    step[i] = lc->nodes[i].step; sub[i] = lc->nodes[i].sub;
    dur[i] = slot_duration(e->P, e->P.st[ph.structure], ph.split, cv.slot[lc->nodes[i].slot], a, &zd);
  }
  for (size_t j = 0; j < lc->edges.size(); ++j) { edges[2 * j] = lc->edges[j].first; edges[2 * j + 1] = lc->edges[j].second; }
  *n_edges = (int)lc->edges.size();
  return n;
}

// isolated operator time / peak of mock nodes (candidate directory)
int port_op_time(void* h, uint64_t n, int structure, int vertex, const int16_t* strat, uint64_t stride, double* time,
                 double* peak) {
  Port* e = (Port*)h;
  const rpeg_struct_t& st = e->P.st[structure];
  for (uint64_t i = 0; i < n; ++i) {
    VPlan a;
    a.dp = strat[0 * stride + i]; a.pp = strat[1 * stride + i]; a.tp = strat[2 * stride + i]; a.mb = strat[3 * stride + i];
    a.o[0] = a.o[1] = a.o[2] = 0;
    a.e[0] = strat[4 * stride + i]; a.e[1] = strat[5 * stride + i]; a.e[2] = strat[6 * stride + i];
    bool zd = false;
    time[i] = op_time(e->P, st.vertex[vertex], st.vertex[vertex].unsplit, a, &zd);
    if (zd) time[i] = NAN;
    peak[i] = isolated_peak(st.vertex[vertex], vertex_memory(e->P, st.vertex[vertex], a));
  }
  return 0;
}

// ---- simulated annealing: the host logic of rpeg_sa.h with this CPU evaluator behind it
namespace {
struct CpuSaBackend : SaBackend {
  Port* e;
  uint8_t head_of[256][4] = {};
  int threads = 1;
  int evaluate(int n, const SaPlan* plans, const uint8_t* variant, SaEval* out) override {
    const size_t V = RPEG_MAX_V * RPEG_FIELDS;
    std::vector<int16_t> vert(V * n);
    std::vector<uint8_t> head(4 * (size_t)n), mask(n);
    std::vector<double> score(n), mass((size_t)n * RPEG_MAX_V);
    for (int i = 0; i < n; ++i) {
      const int16_t* f = &plans[i].f[0][0];
      for (size_t x = 0; x < V; ++x) vert[x * n + i] = f[x];
      for (int x = 0; x < 4; ++x) head[(size_t)x * n + i] = head_of[variant[i]][x];
    }
    int rc = port_eval(e, n, vert.data(), head.data(), n, 0u, nullptr, nullptr, score.data(), mask.data(), nullptr,
                       nullptr, threads, mass.data());
    for (int i = 0; i < n; ++i) {
      out[i].score = score[i];
      out[i].mask = mask[i];
      for (int x = 0; x < RPEG_MAX_V; ++x) out[i].mass[x] = mass[(size_t)i * RPEG_MAX_V + x];
    }
    return rc;
  }
};

void sa_context(Port* e, const rpeg_sa_params_t* prm, SaContext& cx) {
  cx.init(e->P, prm->structure);
  for (int v = 0; v < cx.nv; ++v) cx.set_directory(v, prm->dir[v], prm->dir_n[v]);
}
}  // namespace

// groups of chains that SaRun steps in turn (1: all chains in one batch per step); the result must not depend on it
static int g_sa_groups = 1;
void port_set_sa_groups(int groups) { g_sa_groups = groups < 1 ? 1 : groups; }

int port_sa_run(void* h, const rpeg_sa_params_t* prm, const int16_t* base_plan, rpeg_sa_result_t* res, int threads) {
  Port* e = (Port*)h;
  SaContext cx;
  sa_context(e, prm, cx);
  SaSettings st;
  sa_settings_from(*prm, &st);
  CpuSaBackend be;
  be.e = e; be.threads = threads;
  be.host_lanes = g_sa_groups;
  for (int k = 0; k < prm->n_variants; ++k) {
    be.head_of[k][0] = (uint8_t)prm->structure; be.head_of[k][1] = (uint8_t)prm->split;
    be.head_of[k][2] = prm->tau[k][0]; be.head_of[k][3] = prm->tau[k][1];
  }
  SaRun run(cx, st, be);
  SaPlan base;
  if (base_plan) std::memcpy(&base, base_plan, sizeof base);
  if (int rc = run.run(base_plan ? &base : nullptr)) return rc;
  sa_run_result(run, res);
  return 0;
}

int port_sa_optimize_families(void* h, int32_t n_families, const rpeg_sa_family_t* families, const uint8_t* base_tau,
                              int32_t E_max, int32_t E_struct, int32_t R_max, uint64_t ka, uint64_t kb, uint64_t kc,
                              const int16_t* base_plan, rpeg_sa_serial_result_t* res, int threads) {
  Port* e = (Port*)h;
  CpuSaBackend be;
  be.e = e; be.threads = threads;
  SaFamilySetup setup;
  if (setup.init(e->P, n_families, families, base_tau, be.head_of)) return -1;
  const rpeg_sa_params_t* prm = families[0].params;
  SaSettings st;
  sa_settings_from(*prm, &st);
  SaSerial run(setup.fam, st, be, E_max, E_struct, R_max, prm->seed, ka, kb, kc);
  SaPlan base;
  std::memcpy(&base, base_plan, sizeof base);
  if (int rc = run.run(base, setup.base_variant)) return rc;
  sa_serial_result(run, res);
  return 0;
}

int port_sa_optimize(void* h, const rpeg_sa_params_t* prm, int32_t E_max, int32_t E_struct, int32_t R_max, uint64_t ka,
                     uint64_t kb, uint64_t kc, const int16_t* base_plan, rpeg_sa_serial_result_t* res, int threads) {
  const rpeg_sa_family_t one{prm, 1.0, 0, prm->structure};
  return port_sa_optimize_families(h, 1, &one, prm->tau[0], E_max, E_struct, R_max, ka, kb, kc, base_plan, res, threads);
}

// single proposals with the stream (seed, a, b, c): what = 0 move_gen, 1 pair, 2 region sample of vertex `v`
// in racks [r_lo, r_hi).  Returns the number of plans (or rows) written; *draws = words consumed (in: words
// to skip).
int port_sa_propose(void* h, const rpeg_sa_params_t* prm, int what, uint64_t seed, uint64_t a, uint64_t b, uint64_t c,
                    const int16_t* plan, const double* mass, double T, int v, int r_lo, int r_hi, int16_t* out,
                    int64_t* draws, int32_t* fallback) {
  Port* e = (Port*)h;
  SaContext cx;
  sa_context(e, prm, cx);
  SaRng rng(seed, a, b, c);
  if (draws) rng.k = (uint64_t)*draws;   // continue a stream
  SaPlan cur;
  if (plan) std::memcpy(&cur, plan, sizeof cur);
  int n = 0;
  int fb = 0;
  if (what == 0) {
    std::vector<SaPlan> o(prm->K_x);
    n = sa_move_gen(rng, cx, cur, mass, prm->K_x, prm->T_max, T, prm->T_init, o.data(), &fb);
    std::memcpy(out, o.data(), sizeof(SaPlan) * n);
  } else if (what == 1) {
    SaPlan o;
    n = sa_move_pair(rng, cx, cur, &o) ? 1 : 0;
    if (n) std::memcpy(out, &o, sizeof o);
  } else {
    n = sa_sample_region(rng, cx, v, r_lo, r_hi, out) ? 1 : 0;
  }
  if (draws) *draws = (int64_t)rng.k;
  if (fallback) *fallback = fb;
  return n;
}

void port_exp(uint64_t n, const double* x, double* y) {
  for (uint64_t i = 0; i < n; ++i) y[i] = exp_libm(x[i]);
}
}
