// rpeg_sa.h - host side of the batched simulated annealing: proposal kernels, restarts, elites and the
// Metropolis-Hastings step for a population of independent chains (host only, C++17).
//
// The proposals are integer work of a few hundred instructions per chain and step; they run on the
// host.  Every candidate of every chain of a step is evaluated in ONE batched call of the backend
// (the GPU evaluator), which is where the time goes.
//
// Follows RPEG/search/moves.py (strategy space :97-176, samplers :180-278, candidate directory lookup
// :554-586, single-vertex kernel move_gen :645-825, donor/receiver kernel multi_move_pair :845-950)
// and RPEG/search/optimizer.py (elites :158-198, restarts :201-362, chain loop :690-946).  The
// reference draws from Python's MT19937; here every draw is word k of a counter-based stream keyed by
// (seed, chain, step, purpose), so a trajectory can be replayed anywhere.
#ifndef RPEG_SA_H
#define RPEG_SA_H

#include <algorithm>
#include <array>
#include <chrono>
#include <cmath>
#include <cstring>
#include <map>
#include <set>
#include <string>
#include <unordered_map>
#include <vector>

#include "rpeg_core.h"

namespace rpeg {

// ------------------------------------------------------------------------------------- generator
struct SaRng {
  uint64_t h, k = 0;
  static uint64_t mix(uint64_t x) {
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
  }
  SaRng(uint64_t seed, uint64_t a, uint64_t b, uint64_t c) {
    const uint64_t g = 0x9E3779B97F4A7C15ull;
    h = mix(seed + g * (0x5Aull + 1));
    h = mix(h + g * (a + 1));
    h = mix(h + g * (b + 1));
    h = mix(h + g * (c + 1));
  }
  uint64_t word() { return mix(h + 0x9E3779B97F4A7C15ull * ++k); }
  double random() { return (double)(word() >> 11) * (1.0 / 9007199254740992.0); }
  int below(int n) { return (int)(((word() >> 32) * (uint64_t)n) >> 32); }
  // random.choices(population, weights, k=1): bisect of random()*total in the running sums
  int weighted(const double* w, int n) {
    double cum[RPEG_MAX_V];
    double acc = 0.0;
    for (int i = 0; i < n; ++i) { acc = i == 0 ? w[0] : acc + w[i]; cum[i] = acc; }
    const double x = random() * (cum[n - 1] + 0.0);
    int lo = 0, hi = n - 1;
    while (lo < hi) {
      const int mid = (lo + hi) / 2;
      if (x < cum[mid]) hi = mid; else lo = mid + 1;
    }
    return lo;
  }
};

// ------------------------------------------------------------------------------------- plans
enum { SA_DP = 0, SA_PP, SA_TP, SA_MB, SA_OR, SA_ON, SA_OG, SA_ER, SA_EN, SA_EG };

struct SaPlan { int16_t f[RPEG_MAX_V][RPEG_FIELDS]; };

struct SaEval {          // what one evaluation returns
  double score;          // throughput times the soft memory penalty, without the stale-layout gate
  double mass[RPEG_MAX_V];
  double util = 0.0;     // Trace.utilization(), filled only where the utilisation objective asks for it
  uint8_t mask;          // RPEG_MASK_*
};

struct SaEntry { SaPlan plan; SaEval ev; };

struct SaBackend {
  virtual ~SaBackend() {}
  // evaluates n plans; variant[i] selects the staleness variant of plan i
  virtual int evaluate(int n, const SaPlan* plans, const uint8_t* variant, SaEval* out) = 0;
  // the same with Trace.utilization() of every plan (out[i].util) from the same evaluation when with_util is set;
  // returns 1 when the backend cannot do that for this batch (the caller then asks plan by plan)
  virtual int evaluate(int n, const SaPlan* plans, const uint8_t* variant, SaEval* out, bool with_util) {
    if (with_util) return 1;
    return evaluate(n, plans, variant, out);
  }
  // Trace.utilization() of one plan (trace.py:53-101); backends without traces refuse
  virtual int utilization(const SaPlan& plan, uint8_t variant, double* out) { (void)plan; (void)variant; (void)out; return -1; }
  // The same evaluation in two halves, for a caller that has other work while it runs: submit() starts the evaluation of
  // `n` plans in lane `lane` (0 .. lanes() - 1; the arrays stay the caller's and must live until collect), collect()
  // waits for it and fills `out`.  One evaluation per lane at a time; evaluate() may be called in between.  The default
  // evaluates in collect().
  virtual int lanes() const { return host_lanes; }
  virtual int submit(int lane, int n, const SaPlan* plans, const uint8_t* variant) {
    if ((int)pend.size() <= lane) pend.resize((size_t)lane + 1);
    pend[(size_t)lane] = Pending{n, plans, variant};
    return 0;
  }
  virtual int collect(int lane, SaEval* out) {
    const Pending& q = pend[(size_t)lane];
    return q.n > 0 ? evaluate(q.n, q.plans, q.variant, out) : 0;
  }
  int host_lanes = 1;
  struct Pending { int n; const SaPlan* plans; const uint8_t* variant; };
  std::vector<Pending> pend;
};

struct SaSettings {
  int n_chains = 64, n_steps = 2000, K_x = 6, T_max = 50, K_elite = 3, stag_window = 20, restart_attempts = 50;
  int gate_candidates = 0, geometric_cooling = 0, n_variants = 1;
  double T_init = 0.30, T_warm = 0.05, T_min = 0.01, T_cool = 1.0, alpha_pair = 0.28, score_eps = 1e-4;
  double max_throughput_loss = 0.0;
  uint64_t seed = 42;
  int hard_oom = 0;                       // OptimizerConfig.hard_oom: a plan that does not fit scores 0 (evaluate.py:392, 437)
  int timed = 0;                          // bit 0: deadline_s holds, bit 1: deadline_struct_s holds
  double deadline_s = 0.0, deadline_struct_s = 0.0;   // readings of the clock at which rpeg_sa_optimize* ends the run / a setting
  double (*clock)(void*) = nullptr;       // seconds; null: the steady clock, zero when the run starts
  void* clock_ctx = nullptr;
};

struct SaContext {
  int nv = 0, R = 1, N = 1, G = 1, B = 1;
  bool fixed_mb = false;         // moves.py:155-156, 182-188: one micro-batch count per (dp, pp)
  bool uniform_vertex = false;   // moves.py:157-158, 688: no critical-chain bias when a vertex is drawn
  int L[RPEG_MAX_V] = {0};
  std::vector<int> tps, dps;
  std::vector<int> pps[RPEG_MAX_V];
  std::vector<std::array<int16_t, 6>> dir[RPEG_MAX_V];       // dp pp tp r_ext n_ext mb, ascending by time
  std::unordered_map<uint64_t, int> dir_index[RPEG_MAX_V];

  static uint64_t key6(int dp, int pp, int tp, int re, int ne, int mb) {
    return (uint64_t)dp | (uint64_t)pp << 10 | (uint64_t)tp << 20 | (uint64_t)re << 30 | (uint64_t)ne << 40 |
           (uint64_t)mb << 50;
  }

  // moves.py:97-137
  void init(const rpeg_problem_t& P, int structure) {
    const rpeg_struct_t& st = P.st[structure];
    nv = st.n_vertex; R = P.R; N = P.N; G = P.G; B = P.B;
    const int total = R * N * G;
    tps.clear(); dps.clear();
    for (int t = 1; t <= G; ++t) if (G % t == 0) tps.push_back(t);
    for (int d = 1; d <= total; ++d) if (B % d == 0) dps.push_back(d);
    for (int v = 0; v < nv; ++v) {
      L[v] = P.model[st.vertex[v].model].L;
      pps[v].clear();
      for (int d = 1; d <= total; ++d) if (L[v] % d == 0 && (d == 1 || d % 2 == 0)) pps[v].push_back(d);
    }
  }

  // returns an error text or null
  const char* set_directory(int v, const int16_t* rows, int n) {
    dir[v].assign(n, {});
    dir_index[v].clear();
    for (int j = 0; j < n; ++j) {
      for (int x = 0; x < 6; ++x) {
        if (rows[j * 6 + x] < 0 || rows[j * 6 + x] >= 1024) return "directory field outside 0..1023";
        dir[v][j][x] = rows[j * 6 + x];
      }
      const int16_t* r = rows + j * 6;
      dir_index[v][key6(r[0], r[1], r[2], r[3], r[4], r[5])] = j;   // a later duplicate wins, as dict does
    }
    return nullptr;
  }
};

// moves.py:162-199
inline void sa_valid_mb(int pp, int dp, int B, std::vector<int>& out, bool fixed_mb = false) {
  out.clear();
  const int local = B / dp;
  if (local < 8 && dp > 1) return;
  if (pp == 1) { out.push_back(1); return; }
  if (fixed_mb) { out.push_back(local % pp != 0 ? 1 : pp); return; }
  const int max_mb = local / 8;
  for (int mb = pp; mb <= std::min(max_mb, local); ++mb)
    if (local % mb == 0) out.push_back(mb);
}

// moves.py:685-694: three draws, also when only one origin exists
inline void sa_sample_origin(SaRng& rng, const SaContext& cx, int re, int ne, int ge, int16_t* o) {
  o[0] = (int16_t)(rng.below(cx.R / re) * re);
  o[1] = (int16_t)(rng.below(cx.N / ne) * ne);
  o[2] = (int16_t)(rng.below(cx.G / ge) * ge);
}

// moves.py:645-825 without intra-stage fusion.  Writes up to K_x plans, returns their number.
inline int sa_move_gen(SaRng& rng, const SaContext& cx, const SaPlan& plan, const double* mass, int K_x, int T_max,
                       double T, double T_init, SaPlan* out, int* fallback = nullptr) {
  int v;
  if (!cx.uniform_vertex && rng.random() >= 0.4) {   // (no draw at all under uniform_vertex, moves.py:688)
    double w[RPEG_MAX_V];
    for (int x = 0; x < cx.nv; ++x) w[x] = mass[x] + 1e-6;
    v = rng.weighted(w, cx.nv);
  } else {
    v = rng.below(cx.nv);
  }
  const auto& tab = cx.dir[v];
  const int len = (int)tab.size();
  const double frac = std::min(1.0, T / T_init);
  const int w = std::max(5, (int)((double)len * frac));
  const int16_t* cur = plan.f[v];
  int j_star;
  {
    auto it = cx.dir_index[v].find(SaContext::key6(cur[SA_DP], cur[SA_PP], cur[SA_TP], cur[SA_ER], cur[SA_EN], cur[SA_MB]));
    if (it != cx.dir_index[v].end()) j_star = it->second;
    else { j_star = len / 2; if (fallback) ++*fallback; }
  }
  const int low = std::max(0, j_star - w), high = std::min(len - 1, j_star + w);

  int n_out = 0;
  std::array<int16_t, 7> seen[64];
  int n_seen = 0;
  auto add = [&](int dp, int pp, int tp, int mb, const int16_t* o, int re, int ne, int ge) {
    SaPlan& q = out[n_out++];
    q = plan;
    int16_t* r = q.f[v];
    r[SA_DP] = (int16_t)dp; r[SA_PP] = (int16_t)pp; r[SA_TP] = (int16_t)tp; r[SA_MB] = (int16_t)mb;
    r[SA_OR] = o[0]; r[SA_ON] = o[1]; r[SA_OG] = o[2];
    r[SA_ER] = (int16_t)re; r[SA_EN] = (int16_t)ne; r[SA_EG] = (int16_t)ge;
    seen[n_seen++] = {(int16_t)dp, (int16_t)pp, (int16_t)tp, o[0], o[1], o[2], (int16_t)mb};
  };

  for (int t = 0; t < std::min(5, T_max); ++t) {   // placement only, best effort
    int16_t o[3];
    sa_sample_origin(rng, cx, cur[SA_ER], cur[SA_EN], cur[SA_EG], o);
    if (o[0] != cur[SA_OR] || o[1] != cur[SA_ON] || o[2] != cur[SA_OG]) {
      add(cur[SA_DP], cur[SA_PP], cur[SA_TP], cur[SA_MB], o, cur[SA_ER], cur[SA_EN], cur[SA_EG]);
      break;
    }
  }
  for (int t = 0; t < T_max; ++t) {                // strategy changes from the window around j_star
    if (n_out >= K_x || high < low || n_seen >= 64) break;
    const int j = low + rng.below(high - low + 1);
    if (j == j_star) continue;
    const auto& e = tab[j];
    int ge, nodes;
    if (!packing_geometry(e[0], e[1], e[2], cx.G, &ge, &nodes)) continue;
    int16_t o[3];
    sa_sample_origin(rng, cx, e[3], e[4], ge, o);
    const std::array<int16_t, 7> key = {e[0], e[1], e[2], o[0], o[1], o[2], e[5]};
    bool dup = false;
    for (int s = 0; s < n_seen; ++s) dup = dup || seen[s] == key;
    if (dup) continue;
    add(e[0], e[1], e[2], e[5], o, e[3], e[4], ge);
  }
  return n_out;
}

// moves.py:180-278: a random (allocation, strategy, mb) of vertex v within racks [r_lo, r_hi)
inline bool sa_sample_region(SaRng& rng, const SaContext& cx, int v, int r_lo, int r_hi, int16_t* row) {
  const int R_eff = r_hi - r_lo;
  const int tp = cx.tps[rng.below((int)cx.tps.size())];
  if (cx.pps[v].empty()) return false;
  const int pp = cx.pps[v][rng.below((int)cx.pps[v].size())];
  const int s = std::min(pp, cx.G / tp);
  if (pp % s != 0) return false;
  int dcand[1024];
  int nd = 0;
  for (int d : cx.dps) {
    int ge, nodes;
    if (packing_geometry(d, pp, tp, cx.G, &ge, &nodes) && nodes <= R_eff * cx.N && nd < 1024) dcand[nd++] = d;
  }
  if (nd == 0) return false;
  const int dp = dcand[rng.below(nd)];
  int ge = 1, need = 1;
  packing_geometry(dp, pp, tp, cx.G, &ge, &need);
  int lay[64][2];
  int nl = 0;
  for (int re = 1; re <= std::min(R_eff, need); ++re)
    if (need % re == 0 && need / re <= cx.N && nl < 64) { lay[nl][0] = re; lay[nl][1] = need / re; ++nl; }
  if (nl == 0) return false;
  const int li = rng.below(nl);
  const int re = lay[li][0], ne = lay[li][1];
  if (R_eff / re == 0) return false;
  const int r_o = r_lo + rng.below(R_eff / re) * re;
  const int n_o = rng.below(cx.N / ne) * ne;
  const int g_o = rng.below(cx.G / ge) * ge;
  std::vector<int> mbs;
  sa_valid_mb(pp, dp, cx.B, mbs, cx.fixed_mb);
  if (mbs.empty()) return false;
  const int mb = mbs[rng.below((int)mbs.size())];
  row[SA_DP] = (int16_t)dp; row[SA_PP] = (int16_t)pp; row[SA_TP] = (int16_t)tp; row[SA_MB] = (int16_t)mb;
  row[SA_OR] = (int16_t)r_o; row[SA_ON] = (int16_t)n_o; row[SA_OG] = (int16_t)g_o;
  row[SA_ER] = (int16_t)re; row[SA_EN] = (int16_t)ne; row[SA_EG] = (int16_t)ge;
  return true;
}

inline bool sa_boxes_overlap(const int16_t* a, const int16_t* b) {
  for (int x = 0; x < 3; ++x)
    if (a[SA_OR + x] + a[SA_ER + x] <= b[SA_OR + x] || b[SA_OR + x] + b[SA_ER + x] <= a[SA_OR + x]) return false;
  return true;
}

// moves.py:845-950 without intra-stage fusion
inline bool sa_move_pair(SaRng& rng, const SaContext& cx, const SaPlan& plan, SaPlan* out, int max_retries = 100) {
  double w[RPEG_MAX_V], sum = 0.0;
  for (int v = 0; v < cx.nv; ++v) {
    w[v] = (double)(plan.f[v][SA_ER] * plan.f[v][SA_EN] * plan.f[v][SA_EG]);
    sum = v == 0 ? w[0] : sum + w[v];
  }
  if (sum == 0.0) return false;
  const int vd = rng.weighted(w, cx.nv);
  int ov[RPEG_MAX_V], n_ov = 0;
  for (int v = 0; v < cx.nv; ++v)
    if (v != vd && sa_boxes_overlap(plan.f[v], plan.f[vd])) ov[n_ov++] = v;
  if (n_ov == 0) return false;
  const int vr = ov[rng.below(n_ov)];

  const int d_lo = plan.f[vd][SA_OR], d_ext = plan.f[vd][SA_ER];
  int new_lo, new_ext;
  if (d_ext > 1) {
    new_ext = 1 + rng.below(d_ext - 1);
    new_lo = d_lo + rng.below(d_ext - new_ext + 1);
  } else {
    new_lo = d_lo; new_ext = 1;
  }
  int16_t donor[RPEG_FIELDS], recv[RPEG_FIELDS];
  bool ok = false;
  for (int t = 0; t < max_retries && !ok; ++t) ok = sa_sample_region(rng, cx, vd, new_lo, new_lo + new_ext, donor);
  if (!ok) return false;

  int recv_lo = 0, recv_hi = cx.R;
  if (new_ext < d_ext) {   // some racks were freed
    const int freed_min = new_lo > d_lo ? d_lo : new_lo + new_ext;
    const int freed_max = new_lo + new_ext < d_lo + d_ext ? d_lo + d_ext - 1 : new_lo - 1;
    const int r_o = plan.f[vr][SA_OR], r_e = plan.f[vr][SA_ER];
    recv_lo = std::min(r_o, freed_min);
    recv_hi = std::max(r_o + r_e - 1, freed_max) + 1;
  }
  ok = false;
  for (int t = 0; t < max_retries && !ok; ++t) ok = sa_sample_region(rng, cx, vr, recv_lo, recv_hi, recv);
  if (!ok) return false;
  *out = plan;
  std::memcpy(out->f[vd], donor, sizeof donor);
  std::memcpy(out->f[vr], recv, sizeof recv);
  return true;
}

// optimizer.py:201-256 without fusion; false where the reference raises
inline bool sa_sample_all(SaRng& rng, const SaContext& cx, SaPlan* out) {
  std::memset(out, 0, sizeof *out);
  for (int v = 0; v < cx.nv; ++v) {
    bool ok = false;
    for (int t = 0; t < 100 && !ok; ++t) ok = sa_sample_region(rng, cx, v, 0, cx.R, out->f[v]);
    if (!ok) return false;
  }
  return true;
}

// ------------------------------------------------------------------------------------- chains
struct SaChain {
  SaEntry cur;
  double score = 0.0, T = 0.0;
  int rej = 0, restarts = 0;
  bool dead = false;
  std::vector<SaEntry> elite;                       // descending by score
  std::set<std::vector<int16_t>> seen;
  bool has_best = false, has_feasible = false;
  SaEntry best, best_feasible;
  double best_score = -INFINITY, best_feasible_score = -INFINITY;
  int best_step = -1, best_feasible_step = -1;
  double best_feasible_time = 0.0;
  long n_eval = 0;
};

struct SaRun {
  const SaContext& cx;
  const SaSettings& p;
  SaBackend& be;
  std::vector<SaChain> chains;
  std::vector<uint8_t> log;     // [chain][step]: kind | n_candidates << 1 | verdict << 4 | restart << 6
  std::chrono::steady_clock::time_point t0;
  std::string err;

  SaRun(const SaContext& c, const SaSettings& s, SaBackend& b) : cx(c), p(s), be(b) {}

  double now() const { return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count(); }
  uint8_t variant(int chain) const { return (uint8_t)(chain % p.n_variants); }

  static bool full_ok(uint8_t m) {   // is_valid (evaluate.py:143-232) of a plan the samplers built
    return (m & RPEG_MASK_VALID) && (m & RPEG_MASK_STALE_OK) && (m & RPEG_MASK_MEM_OK) && !(m & RPEG_MASK_ERROR);
  }
  static double gated(const SaEval& e) { return (e.mask & RPEG_MASK_STALE_OK) ? e.score : 0.0; }
  // OptimizerConfig.hard_oom (evaluate.py:392, 437): a plan that does not fit scores 0
  void hard_oom(SaEval* ev, int n) const {
    if (!p.hard_oom) return;
    for (int i = 0; i < n; ++i)
      if (!(ev[i].mask & RPEG_MASK_MEM_OK)) ev[i].score = 0.0;
  }

  std::vector<int16_t> fingerprint(const SaPlan& q) const {   // optimizer.py:158-172: pi, origin, mb
    std::vector<int16_t> fp;
    for (int v = 0; v < cx.nv; ++v)
      for (int x : {SA_DP, SA_PP, SA_TP, SA_OR, SA_ON, SA_OG, SA_MB}) fp.push_back(q.f[v][x]);
    return fp;
  }

  void elite_insert(SaChain& ch, const SaEntry& e) {          // optimizer.py:175-198
    auto fp = fingerprint(e.plan);
    if (ch.seen.count(fp)) return;
    if ((int)ch.elite.size() >= p.K_elite && e.ev.score <= ch.elite.back().ev.score) return;
    ch.elite.push_back(e);
    std::stable_sort(ch.elite.begin(), ch.elite.end(),
                     [](const SaEntry& a, const SaEntry& b) { return a.ev.score > b.ev.score; });
    if ((int)ch.elite.size() > p.K_elite) ch.elite.resize(p.K_elite);
    ch.seen.insert(fp);
  }

  void note(SaChain& ch, const SaEntry& e, double score, int step, bool feasible) {   // optimizer.py:676-686, 846-861
    if (feasible) elite_insert(ch, e);
    if (!ch.has_best || score > ch.best_score * (1.0 + p.score_eps)) {
      ch.has_best = true; ch.best = e; ch.best_score = score; ch.best_step = step;
    }
    if (feasible && score > ch.best_feasible_score) {
      ch.has_feasible = true; ch.best_feasible = e; ch.best_feasible_score = score; ch.best_feasible_step = step;
      ch.best_feasible_time = now();
    }
  }

  void enter(SaChain& ch, const SaEntry& e, int step, double T) {   // optimizer.py:666-694
    ch.cur = e;
    ch.score = gated(e.ev);
    const bool feasible = (e.ev.mask & RPEG_MASK_MEM_OK) && (e.ev.mask & RPEG_MASK_STALE_OK);
    note(ch, e, ch.score, step, feasible);
    ch.T = T;
    ch.rej = 0;
  }

  // optimizer.py:259-289 for every chain of `who`: the first valid one of restart_attempts random plans
  // (found = 1), else the first attempt as it is (found = 2), else nothing (found = 0: the sampler failed)
  int random_restart(const std::vector<int>& who, int step, std::vector<int>& found, std::vector<SaEntry>& entry) {
    found.assign(who.size(), 0);
    entry.assign(who.size(), SaEntry{});
    std::vector<SaPlan> plans;
    std::vector<uint8_t> var;
    std::vector<int> first(who.size() + 1, 0);
    for (size_t i = 0; i < who.size(); ++i) {
      for (int a = 0; a < p.restart_attempts; ++a) {
        SaRng rng(p.seed, (uint64_t)who[i], (uint64_t)(step + 1), (uint64_t)(1 + a));
        SaPlan q;
        if (!sa_sample_all(rng, cx, &q)) break;
        plans.push_back(q);
        var.push_back(variant(who[i]));
      }
      first[i + 1] = (int)plans.size();
    }
    std::vector<SaEval> ev(plans.size());
    if (!plans.empty())
      if (int rc = be.evaluate((int)plans.size(), plans.data(), var.data(), ev.data())) return rc;
    hard_oom(ev.data(), (int)plans.size());
    for (size_t i = 0; i < who.size(); ++i) {
      SaChain& ch = chains[who[i]];
      // a sampler failure ends the restart where the reference raises; attempts before it still count
      for (int j = first[i]; j < first[i + 1]; ++j) {
        ++ch.n_eval;
        if (full_ok(ev[j].mask)) { found[i] = 1; entry[i].plan = plans[j]; entry[i].ev = ev[j]; break; }
      }
      if (!found[i] && first[i + 1] > first[i] && (ev[first[i]].mask & RPEG_MASK_VALID) &&
          !(ev[first[i]].mask & RPEG_MASK_ERROR)) {
        found[i] = 2; entry[i].plan = plans[first[i]]; entry[i].ev = ev[first[i]];
      }
    }
    return 0;
  }

  int run(const SaPlan* base_plan) {
    t0 = std::chrono::steady_clock::now();
    chains.assign(p.n_chains, SaChain{});
    log.assign((size_t)p.n_chains * p.n_steps, 0);
    // ---- start: the base plan if valid, else a valid random plan, else the base plan as it is (the soft
    // memory penalty guides the search, optimizer.py:612-616), else the first random plan as it is
    {
      std::vector<int> need;
      std::vector<SaEntry> base(p.n_chains);
      if (base_plan) {
        std::vector<SaPlan> plans(p.n_chains, *base_plan);
        std::vector<uint8_t> var(p.n_chains);
        std::vector<SaEval> ev(p.n_chains);
        for (int c = 0; c < p.n_chains; ++c) var[c] = variant(c);
        if (int rc = be.evaluate(p.n_chains, plans.data(), var.data(), ev.data())) return rc;
        hard_oom(ev.data(), p.n_chains);
        for (int c = 0; c < p.n_chains; ++c) {
          ++chains[c].n_eval;
          base[c].plan = *base_plan; base[c].ev = ev[c];
          if (full_ok(ev[c].mask)) enter(chains[c], base[c], -1, p.T_init); else need.push_back(c);
        }
      } else {
        for (int c = 0; c < p.n_chains; ++c) need.push_back(c);
      }
      std::vector<int> found;
      std::vector<SaEntry> entry;
      if (int rc = random_restart(need, -1, found, entry)) return rc;
      for (size_t i = 0; i < need.size(); ++i) {
        SaChain& ch = chains[need[i]];
        if (found[i] == 1) enter(ch, entry[i], -1, p.T_init);
        else if (base_plan && !(base[need[i]].ev.mask & RPEG_MASK_ERROR) && (base[need[i]].ev.mask & RPEG_MASK_VALID))
          enter(ch, base[need[i]], -1, p.T_init);
        else if (found[i] == 2) enter(ch, entry[i], -1, p.T_init);
        else ch.dead = true;
      }
    }

    // The chains are independent of each other: they are dealt to `G` groups that take their steps in turn, so that
    // the host proposes for one group and merges its results while the evaluations of the others run.  Every chain
    // draws from its own stream keyed by (seed, chain, step), so its trajectory does not depend on the grouping.
    const int G = std::max(1, std::min(be.lanes(), p.n_chains));
    struct Group {
      std::vector<int> who;              // chains of the group
      std::vector<SaPlan> cand;
      std::vector<uint8_t> var;
      std::vector<SaEval> ev;
      std::vector<int> first, kind;      // by position in `who`
      std::vector<SaRng> rngs;
      int total = 0;
    };
    std::vector<Group> groups(G);
    for (int c = 0; c < p.n_chains; ++c) groups[c % G].who.push_back(c);
    for (Group& g : groups) {
      g.cand.resize(g.who.size() * (size_t)p.K_x);
      g.var.resize(g.cand.size());
      g.ev.resize(g.cand.size());
      g.first.resize(g.who.size() + 1);
      g.kind.resize(g.who.size());
    }
    // ---- proposals of every live chain of a group, and the start of their evaluation
    auto propose = [&](int gi, int step) -> int {
      Group& g = groups[gi];
      g.rngs.clear();
      int total = 0;
      for (size_t k = 0; k < g.who.size(); ++k) {
        const int c = g.who[k];
        SaChain& ch = chains[c];
        g.rngs.emplace_back(p.seed, (uint64_t)c, (uint64_t)(step + 1), 0);
        g.first[k] = total;
        g.kind[k] = -1;
        if (ch.dead) continue;
        SaRng& rng = g.rngs.back();
        const double frac = std::min(1.0, ch.T / p.T_init);
        if (rng.random() < p.alpha_pair * frac) {
          g.kind[k] = 1;
          if (sa_move_pair(rng, cx, ch.cur.plan, &g.cand[total])) total += 1;
          else { ch.T = std::max(p.T_min, ch.T * p.T_cool); g.kind[k] = 2; }   // optimizer.py:737-740
        } else {
          g.kind[k] = 0;
          total += sa_move_gen(rng, cx, ch.cur.plan, ch.cur.ev.mass, p.K_x, p.T_max, ch.T, p.T_init, &g.cand[total]);
        }
        for (int j = g.first[k]; j < total; ++j) g.var[j] = variant(c);
      }
      g.first[g.who.size()] = total;
      g.total = total;
      return be.submit(gi, total, g.cand.data(), g.var.data());
    };
    // ---- best of K, one Metropolis-Hastings step, stagnation
    auto merge = [&](int gi, int step) -> int {
      Group& g = groups[gi];
      if (int rc = be.collect(gi, g.ev.data())) return rc;
      hard_oom(g.ev.data(), g.total);
      std::vector<int> random_who;
      for (size_t k = 0; k < g.who.size(); ++k) {
        const int c = g.who[k];
        SaChain& ch = chains[c];
        if (ch.dead || g.kind[k] < 0) continue;
        uint8_t& lg = log[(size_t)c * p.n_steps + step];
        if (g.kind[k] == 2) { lg = 1; continue; }
        const int nc = g.first[k + 1] - g.first[k];
        lg = (uint8_t)(g.kind[k] | nc << 1);
        bool restart = false;
        if (nc == 0) {
          restart = true;   // "chain stuck" (optimizer.py:767-769)
        } else {
          int bi = -1;
          double bs = -INFINITY;
          for (int j = g.first[k]; j < g.first[k + 1]; ++j) {
            ++ch.n_eval;
            SaEntry e; e.plan = g.cand[j]; e.ev = g.ev[j];
            const bool stale_ok = (g.ev[j].mask & RPEG_MASK_STALE_OK) != 0;
            double sc = p.gate_candidates ? gated(g.ev[j]) : g.ev[j].score;
            if (g.ev[j].mask & RPEG_MASK_ERROR) sc = -INFINITY;
            const bool feas = (g.ev[j].mask & RPEG_MASK_MEM_OK) && !(g.ev[j].mask & RPEG_MASK_ERROR) &&
                              (stale_ok || !p.gate_candidates);
            if (!(g.ev[j].mask & RPEG_MASK_ERROR)) note(ch, e, sc, step, feas);
            if (sc > bs) { bs = sc; bi = j; }
          }
          if (bi >= 0) {
            const double delta = (bs - ch.score) / (std::fabs(ch.score) + 1e-12);
            if (std::fabs(delta) >= 1e-6) {
              const double prob = delta >= 0.0 ? 1.0 : exp_libm(delta / ch.T);
              const bool acc = g.rngs[k].random() < prob;
              if (acc) { ch.cur.plan = g.cand[bi]; ch.cur.ev = g.ev[bi]; ch.score = bs; ch.rej = 0; }
              else ++ch.rej;
              lg |= (uint8_t)((acc ? 2 : 1) << 4);
            }
          }
          if (p.geometric_cooling) ch.T = std::max(p.T_min, ch.T * p.T_cool);
          if (p.stag_window > 0 && ch.rej >= p.stag_window) restart = true;
        }
        if (restart) {
          lg |= 1 << 6;
          ++ch.restarts;
          if (!ch.elite.empty() && full_ok(ch.elite[0].ev.mask)) enter(ch, ch.elite[0], step, p.T_warm);
          else random_who.push_back(c);
        }
      }
      if (!random_who.empty()) {
        std::vector<int> found;
        std::vector<SaEntry> entry;
        if (int rc = random_restart(random_who, step, found, entry)) return rc;
        for (size_t i = 0; i < random_who.size(); ++i) {
          SaChain& ch = chains[random_who[i]];
          if (found[i] == 1) enter(ch, entry[i], step, p.T_warm);
          else { ch.T = p.T_warm; ch.rej = 0; }   // no valid restart: go on from the current plan
        }
      }
      return 0;
    };
    if (p.n_steps > 0)
      for (int gi = 0; gi < G; ++gi)
        if (int rc = propose(gi, 0)) return rc;
    for (int step = 0; step < p.n_steps; ++step)
      for (int gi = 0; gi < G; ++gi) {
        if (int rc = merge(gi, step)) return rc;
        if (step + 1 < p.n_steps)
          if (int rc = propose(gi, step + 1)) return rc;
      }
    return 0;
  }
};

// ------------------------------------------------------------------------------------- one chain at a time
// optimize() as the reference runs it (optimizer.py:365-946): the structural families one after the other
// (the separate template, then AC-share: inter_model.py:68-121 without the fused settings), within a family
// its staleness variants one after the other, each a sequence of restarts of ONE chain on one continuous
// random stream; an evaluation cache (hits cost no budget and are merged before fresh results); the
// budgets E_max / E_struct counted in cache misses; elites shared by the variants of a family; warm
// restarts from the best elite plan, random restarts otherwise.  The K_x candidates of a step are one
// batched evaluation.
struct SaFamily {
  const SaContext* cx = nullptr;  // template and candidate directory
  int first_variant = 0;          // backend variants first_variant .. first_variant + n_variants - 1, walked in order
  int n_variants = 1;
  int first_valid = 0;            // backend variants whose masks stand for is_valid(): the reference checks restarts
                                  // with the memory model of the base configuration (optimizer.py:449-458), which can
                                  // differ from the one evaluate_cached builds; == first_variant when they agree
  double scale = 1.0;             // 1 - lambda_ac for the AC-share template (optimizer.py:132-145)
  int elite_family = 0;           // families with one number share elites (optimizer.py:500-515)
};

struct SaSerial {
  std::vector<SaFamily> fam;
  const SaSettings& p;
  SaBackend& be;
  int E_max, E_struct, R_max;
  SaRng rng;

  struct Stored { double score; bool feasible; SaEval ev; };
  std::unordered_map<std::string, Stored> cache;
  std::vector<SaPlan> eval_log;          // every plan handed to the evaluator as a cache miss, in order
  std::vector<uint8_t> eval_log_variant;
  std::vector<Stored> eval_log_stored;   // what the cache holds for each of them
  std::map<int, std::vector<SaEntry>> elites;
  std::map<int, std::set<std::vector<int16_t>>> seens;
  SaEntry best, best_feasible;
  int best_variant = 0, best_feasible_variant = 0;
  bool has_feasible = false;
  double best_score = 0.0, best_feasible_score = -INFINITY;
  long E = 0, n_uncounted = 0;

  SaSerial(const std::vector<SaFamily>& f, const SaSettings& s, SaBackend& b, int e_max, int e_struct, int r_max,
           uint64_t seed, uint64_t ka, uint64_t kb, uint64_t kc)
      : fam(f), p(s), be(b), E_max(e_max), E_struct(e_struct), R_max(r_max), rng(seed, ka, kb, kc) {}

  std::string key(const SaPlan& q, int variant) const {
    std::string k((const char*)&q, sizeof q);
    k.push_back((char)variant);
    return k;
  }
  static std::vector<int16_t> fingerprint(const SaPlan& q, int nv) {
    std::vector<int16_t> fp;
    for (int v = 0; v < nv; ++v)
      for (int x : {SA_DP, SA_PP, SA_TP, SA_OR, SA_ON, SA_OG, SA_MB}) fp.push_back(q.f[v][x]);
    return fp;
  }
  void elite_insert(const SaFamily& f, double raw, const SaPlan& q, const SaEval& ev) {
    std::vector<SaEntry>& elite = elites[f.elite_family];
    std::set<std::vector<int16_t>>& seen = seens[f.elite_family];
    auto fp = fingerprint(q, f.cx->nv);
    if (seen.count(fp)) return;
    if ((int)elite.size() >= p.K_elite && raw <= elite.back().ev.score) return;
    SaEntry e; e.plan = q; e.ev = ev; e.ev.score = raw;
    elite.push_back(e);
    std::stable_sort(elite.begin(), elite.end(), [](const SaEntry& a, const SaEntry& b) { return a.ev.score > b.ev.score; });
    if ((int)elite.size() > p.K_elite) elite.resize(p.K_elite);
    seen.insert(fp);
  }
  static bool mask_valid(uint8_t m) {
    return (m & RPEG_MASK_VALID) && (m & RPEG_MASK_STALE_OK) && (m & RPEG_MASK_MEM_OK) && !(m & RPEG_MASK_ERROR);
  }
  // is_valid (evaluate.py:143-232) costs no budget and does not touch the cache
  int is_valid(const SaPlan& q, int variant, int valid_variant, bool* ok) {
    if (variant == valid_variant) {
      auto it = cache.find(key(q, variant));
      if (it != cache.end()) { *ok = mask_valid(it->second.ev.mask); return 0; }
    }
    SaEval ev;
    const uint8_t var = (uint8_t)valid_variant;
    if (int rc = be.evaluate(1, &q, &var, &ev)) return rc;
    ++n_uncounted;
    *ok = mask_valid(ev.mask);
    return 0;
  }
  // evaluates the cache misses among `plans` in one batch; gated: evaluate_cached's score, else _eval_worker's
  int evaluate(int n, const SaPlan* plans, int variant, bool gated, std::vector<Stored>& out, std::vector<char>& miss) {
    out.resize(n);
    miss.assign(n, 0);
    std::vector<SaPlan> todo;
    std::vector<int> idx;
    for (int i = 0; i < n; ++i) {
      auto it = cache.find(key(plans[i], variant));
      if (it != cache.end()) { out[i] = it->second; continue; }
      bool dup = false;   // the same plan twice among the misses is evaluated once
      for (size_t j = 0; j < todo.size() && !dup; ++j) dup = std::memcmp(&todo[j], &plans[i], sizeof(SaPlan)) == 0;
      if (!dup) { todo.push_back(plans[i]); idx.push_back(i); }
      miss[i] = 1;
    }
    if (!todo.empty()) {
      std::vector<uint8_t> var(todo.size(), (uint8_t)variant);
      std::vector<SaEval> ev(todo.size());
      const bool with_util = p.max_throughput_loss > 0.0;
      int rc = be.evaluate((int)todo.size(), todo.data(), var.data(), ev.data(), with_util);
      if (rc == 1 && with_util) {   // no utilisation from the batched evaluation: one trace per plan
        if ((rc = be.evaluate((int)todo.size(), todo.data(), var.data(), ev.data())) != 0) return rc;
        for (size_t j = 0; j < todo.size(); ++j)
          if ((rc = be.utilization(todo[j], (uint8_t)variant, &ev[j].util)) != 0) return rc;
      }
      if (rc) return rc;
      for (size_t j = 0; j < todo.size(); ++j) {
        const bool stale_ok = (ev[j].mask & RPEG_MASK_STALE_OK) != 0, mem_ok = (ev[j].mask & RPEG_MASK_MEM_OK) != 0;
        Stored st;
        st.ev = ev[j];
        st.score = (gated && !stale_ok) || (p.hard_oom && !mem_ok) ? 0.0 : ev[j].score;
        st.feasible = mem_ok && (stale_ok || !gated);
        cache[key(todo[j], variant)] = st;
        eval_log.push_back(todo[j]);
        eval_log_variant.push_back((uint8_t)variant);
        eval_log_stored.push_back(st);
      }
      for (int i = 0; i < n; ++i)
        if (miss[i]) out[i] = cache[key(plans[i], variant)];
    }
    return 0;
  }
  // optimizer.py:461-486: throughput x utilisation above the floor (1 - loss) x best throughput so far
  double best_raw = 0.0;
  double eff(double raw, double util) {
    if (!(p.max_throughput_loss > 0.0)) return raw;
    if (raw > best_raw) best_raw = raw;
    if (raw < (1.0 - p.max_throughput_loss) * best_raw) return raw * 1e-12;
    return raw * std::max(util, 1e-6);
  }
  // optimizer.py:676-686, 846-861; returns the score as the family compares it
  double note(const SaFamily& f, const SaPlan& q, const Stored& s, int variant) {
    const double score = eff(s.score, s.ev.util) * f.scale;
    if (s.feasible) elite_insert(f, s.score, q, s.ev);
    if (score > best_score * (1.0 + p.score_eps)) { best.plan = q; best.ev = s.ev; best_score = score; best_variant = variant; }
    if (s.feasible && score > best_feasible_score) {
      has_feasible = true; best_feasible.plan = q; best_feasible.ev = s.ev; best_feasible_score = score;
      best_feasible_variant = variant;
    }
    return score;
  }
  // optimizer.py:259-289 on the continuous stream
  int random_restart(const SaFamily& f, int variant, int valid_variant, SaPlan* out, bool* found) {
    *found = false;
    for (int a = 0; a < 50; ++a) {
      SaPlan q;
      if (!sa_sample_all(rng, *f.cx, &q)) return 0;
      bool ok = false;
      if (int rc = is_valid(q, variant, valid_variant, &ok)) return rc;
      if (ok) { *out = q; *found = true; return 0; }
    }
    return 0;
  }

  // `base` is a plan of family 0's template; base_variant the backend variant of the base configuration
  // seconds on the run's clock (optimizer.py reads time.perf_counter())
  std::chrono::steady_clock::time_point t_start = std::chrono::steady_clock::now();
  double now() const {
    if (p.clock) return p.clock(p.clock_ctx);
    return std::chrono::duration<double>(std::chrono::steady_clock::now() - t_start).count();
  }
  bool timed_out = false;   // the run ended at its wall-clock deadline

  int run(const SaPlan& base, int base_variant) {
    std::vector<Stored> st;
    std::vector<char> miss;
    const bool timed = (p.timed & 1) != 0, timed_struct = (p.timed & 3) != 0;
    const double deadline = p.deadline_s;
    int n_structs = 0, s_idx = 0;
    for (const SaFamily& f : fam) n_structs += f.n_variants;
    if (int rc = evaluate(1, &base, base_variant, true, st, miss)) return rc;   // optimizer.py:466-478
    best.plan = base; best.ev = st[0].ev; best_score = eff(st[0].score, st[0].ev.util); best_variant = base_variant;
    if (st[0].feasible) {
      has_feasible = true; best_feasible = best; best_feasible_score = best_score; best_feasible_variant = base_variant;
      elite_insert(fam[0], st[0].score, base, st[0].ev);
    }
    E = 1;
    std::vector<SaPlan> cand(p.K_x);
    for (const SaFamily& f : fam)
     for (int k = 0; k < f.n_variants; ++k) {
      const SaContext& cx = *f.cx;
      const int variant = f.first_variant + k, valid_variant = f.first_valid + k;
      const bool own_template = f.cx == fam[0].cx;
      // the time left is split evenly among the settings still to come (optimizer.py:571-579)
      double deadline_struct = p.deadline_struct_s;
      if (timed) {   // two readings of the clock, as the reference takes them
        const double left = deadline - now();
        const int structs_left = n_structs - s_idx;
        const double t = now();
        deadline_struct = structs_left > 0 && left > 0.0 ? t + left / structs_left : t;
      }
      ++s_idx;
      SaPlan config = base;
      bool ok = false;
      if (own_template)
        if (int rc = is_valid(base, variant, valid_variant, &ok)) return rc;
      if (!ok) {   // optimizer.py:596-626
        bool found = false;
        if (int rc = random_restart(f, variant, valid_variant, &config, &found)) return rc;
        if (!found) {
          if (!own_template) continue;   // the base plan has no meaning on another template: setting skipped
          config = base;
        }
      }
      long E_s = 0;
      int r = 0, no_progress = 0;
      bool exhausted = false;
      SaEval cur_ev{};
      while (r < R_max && !exhausted) {
        const long restart_E_s = E_s;
        if (r > 0) {   // optimizer.py:640-663
          bool restarted = false;
          const std::vector<SaEntry>& elite = elites[f.elite_family];
          if (!elite.empty()) {
            bool w_ok = false;
            if (int rc = is_valid(elite[0].plan, variant, valid_variant, &w_ok)) return rc;
            if (w_ok) { config = elite[0].plan; restarted = true; }
          }
          if (!restarted) {
            bool found = false;
            if (int rc = random_restart(f, variant, valid_variant, &config, &found)) return rc;
            if (!found) {
              ++r; ++no_progress;
              if (no_progress >= 2) exhausted = true;
              continue;
            }
          }
          no_progress = 0;
        }
        if (int rc = evaluate(1, &config, variant, true, st, miss)) return rc;
        cur_ev = st[0].ev;
        if (miss[0]) { ++E; ++E_s; }
        double score_curr = note(f, config, st[0], variant);
        double T = r > 0 ? p.T_warm : p.T_init;
        int rej = 0;
        while (true) {
          const double t_top = p.timed ? now() : 0.0;   // optimizer.py:703-720: deadline, budget, setting's share, setting's budget
          if (timed && t_top >= deadline) { timed_out = true; return 0; }
          if (E >= E_max) return 0;
          if (timed_struct && t_top >= deadline_struct) { exhausted = true; break; }
          if (E_s >= E_struct) { exhausted = true; break; }
          const double frac = std::min(1.0, T / p.T_init);
          int nc = 0;
          if (rng.random() < p.alpha_pair * frac) {
            if (!sa_move_pair(rng, cx, config, &cand[0])) { T = std::max(p.T_min, T * p.T_cool); continue; }
            nc = 1;
          } else {
            nc = sa_move_gen(rng, cx, config, cur_ev.mass, p.K_x, p.T_max, T, p.T_init, cand.data());
          }
          if (nc == 0) break;   // "chain stuck"
          if (int rc = evaluate(nc, cand.data(), variant, false, st, miss)) return rc;
          int bi = -1;
          double bs = -INFINITY;
          for (int pass = 0; pass < 2; ++pass)        // cache hits first, then fresh results (optimizer.py:807-861)
            for (int i = 0; i < nc; ++i) {
              if ((miss[i] != 0) != (pass == 1)) continue;
              if (miss[i]) { ++E; ++E_s; }
              const double sc = note(f, cand[i], st[i], variant);
              if (sc > bs) { bs = sc; bi = i; }
            }
          const double t_batch = p.timed ? now() : 0.0;   // optimizer.py:848-865
          if (timed && t_batch >= deadline) { timed_out = true; return 0; }
          if (E >= E_max) return 0;
          if (timed_struct && t_batch >= deadline_struct) exhausted = true;
          if (E_s >= E_struct) exhausted = true;
          if (bi >= 0 && !exhausted) {
            const double delta = (bs - score_curr) / (std::fabs(score_curr) + 1e-12);
            if (std::fabs(delta) >= 1e-6) {
              const double prob = delta >= 0.0 ? 1.0 : exp_libm(delta / T);
              if (rng.random() < prob) { config = cand[bi]; cur_ev = st[bi].ev; score_curr = bs; rej = 0; }
              else ++rej;
            }
          }
          if (p.geometric_cooling) T = std::max(p.T_min, T * p.T_cool);
          if (exhausted) break;
          if (p.stag_window > 0 && rej >= p.stag_window) break;
        }
        ++r;
        if (E_s == restart_E_s) { if (++no_progress >= 2) exhausted = true; }
        else no_progress = 0;
      }
    }
    return 0;
  }
};

// What rpeg_sa_optimize_families and its CPU twin share: contexts, families and the backend's variant table
// (family f, variant k -> backend variant f * 8 + k for evaluation, 128 + f * 8 + k for is_valid; the base
// configuration is the variant of family 0 with its staleness, else 255).  Returns an error text or null.
struct SaFamilySetup {
  std::vector<SaContext> cx;
  std::vector<SaFamily> fam;
  int base_variant = 0;
  const char* init(const rpeg_problem_t& P, int n_families, const rpeg_sa_family_t* families, const uint8_t* base_tau,
                   uint8_t (*head_of)[4]) {
    if (n_families < 1 || n_families > 8 || !families) return "bad number of families";
    cx.resize(n_families);
    fam.resize(n_families);
    for (int f = 0; f < n_families; ++f) {
      const rpeg_sa_params_t* prm = families[f].params;
      if (!prm) return "family without parameters";
      const int vs = families[f].valid_structure;
      if (prm->structure < 0 || prm->structure >= P.n_struct || vs < 0 || vs >= P.n_struct ||
          P.st[vs].n_vertex != P.st[prm->structure].n_vertex || prm->split < 0 || prm->split >= P.n_split ||
          prm->n_variants < 1 || prm->n_variants > 8)
        return "bad family parameters";
      cx[f].init(P, prm->structure);
      cx[f].fixed_mb = prm->fixed_mb != 0;
      cx[f].uniform_vertex = prm->uniform_vertex != 0;
      for (int v = 0; v < cx[f].nv; ++v) {
        if (prm->dir_n[v] < 0 || (prm->dir_n[v] > 0 && !prm->dir[v])) return "bad candidate directory";
        if (const char* msg = cx[f].set_directory(v, prm->dir[v], prm->dir_n[v])) return msg;
      }
      fam[f].n_variants = prm->n_variants;
      fam[f].first_variant = f * 8;
      fam[f].first_valid = vs == prm->structure ? f * 8 : 128 + f * 8;
      fam[f].scale = families[f].score_scale;
      fam[f].elite_family = families[f].elite_family;
      for (int k = 0; k < prm->n_variants; ++k) {
        uint8_t* h = head_of[f * 8 + k];
        h[0] = (uint8_t)prm->structure; h[1] = (uint8_t)prm->split; h[2] = prm->tau[k][0]; h[3] = prm->tau[k][1];
        uint8_t* hv = head_of[128 + f * 8 + k];
        hv[0] = (uint8_t)vs; hv[1] = h[1]; hv[2] = h[2]; hv[3] = h[3];
      }
    }
    for (int f = 0; f < n_families; ++f) fam[f].cx = &cx[f];   // cx no longer moves
    const rpeg_sa_params_t* p0 = families[0].params;
    base_variant = 255;
    uint8_t* hb = head_of[255];
    hb[0] = (uint8_t)p0->structure; hb[1] = (uint8_t)p0->split; hb[2] = base_tau[0]; hb[3] = base_tau[1];
    const int n_tau = P.st[p0->structure].n_tau;
    for (int k = p0->n_variants - 1; k >= 0; --k)
      if (p0->tau[k][0] == base_tau[0] && (n_tau < 2 || p0->tau[k][1] == base_tau[1])) base_variant = k;
    return nullptr;
  }
};

inline void sa_settings_from(const rpeg_sa_params_t& prm, SaSettings* st) {
  st->n_chains = prm.n_chains; st->n_steps = prm.n_steps; st->K_x = prm.K_x; st->T_max = prm.T_max;
  st->K_elite = prm.K_elite; st->stag_window = prm.stag_window; st->restart_attempts = prm.restart_attempts;
  st->gate_candidates = prm.gate_candidates; st->geometric_cooling = prm.geometric_cooling;
  st->n_variants = prm.n_variants; st->T_init = prm.T_init; st->T_warm = prm.T_warm; st->T_min = prm.T_min;
  st->T_cool = prm.T_cool; st->alpha_pair = prm.alpha_pair; st->score_eps = prm.score_eps; st->seed = prm.seed;
  st->max_throughput_loss = prm.max_throughput_loss;
  st->hard_oom = prm.hard_oom; st->timed = prm.timed; st->deadline_s = prm.deadline_s;
  st->deadline_struct_s = prm.deadline_struct_s; st->clock = prm.clock; st->clock_ctx = prm.clock_ctx;
}

inline void sa_run_result(const SaRun& run, rpeg_sa_result_t* res) {
  const size_t V = RPEG_MAX_V * RPEG_FIELDS;
  for (int c = 0; c < run.p.n_chains; ++c) {
    const SaChain& ch = run.chains[c];
    const bool feas = ch.has_feasible;
    const SaEntry& b = feas ? ch.best_feasible : ch.best;
    if (res->best_plan) std::memcpy(res->best_plan + c * V, &b.plan, V * 2);
    if (res->best_score) res->best_score[c] = feas ? ch.best_feasible_score : (ch.has_best ? ch.best_score : NAN);
    if (res->best_step) res->best_step[c] = feas ? ch.best_feasible_step : ch.best_step;
    if (res->best_time) res->best_time[c] = feas ? ch.best_feasible_time : -1.0;
    if (res->best_feasible) res->best_feasible[c] = feas;
    if (res->cur_plan) std::memcpy(res->cur_plan + c * V, &ch.cur.plan, V * 2);
    if (res->cur_score) res->cur_score[c] = ch.score;
    if (res->restarts) res->restarts[c] = ch.restarts;
    if (res->n_eval) res->n_eval[c] = ch.n_eval;
    if (res->dead) res->dead[c] = ch.dead;
  }
  if (res->log) std::memcpy(res->log, run.log.data(), run.log.size());
  res->wall_s = run.now();
}

inline void sa_serial_result(const SaSerial& run, rpeg_sa_serial_result_t* res) {
  const bool feas = run.has_feasible;
  const SaEntry& b = feas ? run.best_feasible : run.best;
  std::memcpy(res->best_plan, &b.plan, sizeof(SaPlan));
  const int bv = feas ? run.best_feasible_variant : run.best_variant;
  res->best_family = 0;
  res->best_variant = bv;   // the base configuration's own variant when no family holds it
  for (size_t f = 0; f < run.fam.size(); ++f)
    if (bv >= run.fam[f].first_variant && bv < run.fam[f].first_variant + run.fam[f].n_variants) {
      res->best_family = (int32_t)f;
      res->best_variant = bv - run.fam[f].first_variant;
    }
  res->best_score = feas ? run.best_feasible_score : run.best_score;
  res->best_feasible = feas;
  res->timed_out = run.timed_out ? 1 : 0;
  res->E = run.E;
  res->n_draws = (int64_t)run.rng.k;
  res->n_uncounted = run.n_uncounted;
  res->n_eval_log = (int64_t)run.eval_log.size();
  const int64_t keep = std::min<int64_t>(res->n_eval_log, res->eval_log_cap);
  if (res->eval_log)
    for (int64_t i = 0; i < keep; ++i) std::memcpy(res->eval_log + i * RPEG_MAX_V * RPEG_FIELDS, &run.eval_log[i], sizeof(SaPlan));
  if (res->eval_log_variant)
    for (int64_t i = 0; i < keep; ++i) res->eval_log_variant[i] = run.eval_log_variant[i];
  for (int64_t i = 0; i < keep; ++i) {
    if (res->eval_log_score) res->eval_log_score[i] = run.eval_log_stored[i].score;
    if (res->eval_log_feasible) res->eval_log_feasible[i] = run.eval_log_stored[i].feasible;
    if (res->eval_log_util) res->eval_log_util[i] = run.eval_log_stored[i].ev.util;
  }
}

}  // namespace rpeg
#endif
