// flop_count.cpp - counts the fp64 operations one plan evaluation executes.  TEST INFRASTRUCTURE ONLY.
//
// The per-plan arithmetic of the kernels (rpeg_amd/csrc/rpeg_core.h, rpeg_class.h, rpeg_plan.h: cost model,
// list scheduler, memory model, score) is compiled here with `double` replaced by a type that counts every
// addition/subtraction, multiplication, division, fused multiply-add and comparison it takes part in.  The
// counts are those of the arithmetic as the kernels run it: every duration slot of a lowering class is
// evaluated once per plan (the reference's scheduler evaluates NodeCostModel.time once per node,
// RPEG/schedule/scheduler.py:349, i.e. K_eval times more often for the operator nodes).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <map>
#include <set>
#include <stdexcept>
#include <string>
#include <tuple>
#include <type_traits>
#include <unordered_map>
#include <utility>
#include <vector>

namespace flopcount {
struct Counters { uint64_t add = 0, mul = 0, div = 0, fma = 0, cmp = 0; };
thread_local Counters g_cnt;

struct CountD {
  double v;
  CountD() : v(0.0) {}
  template <class T, class = typename std::enable_if<std::is_arithmetic<T>::value>::type>
  CountD(T x) : v((double)x) {}
  template <class T, class = typename std::enable_if<std::is_integral<T>::value>::type>
  explicit operator T() const { return (T)v; }
  CountD& operator+=(CountD o) { ++g_cnt.add; v += o.v; return *this; }
  CountD& operator-=(CountD o) { ++g_cnt.add; v -= o.v; return *this; }
  CountD& operator*=(CountD o) { ++g_cnt.mul; v *= o.v; return *this; }
  CountD& operator/=(CountD o) { ++g_cnt.div; v /= o.v; return *this; }
  CountD operator-() const { CountD r; r.v = -v; return r; }
};
#define RPEG_BINOP(op, field)                                                                                   \
  inline CountD operator op(CountD a, CountD b) { ++g_cnt.field; CountD r; r.v = a.v op b.v; return r; }        \
  template <class T, class = typename std::enable_if<std::is_arithmetic<T>::value>::type>                       \
  inline CountD operator op(CountD a, T b) { ++g_cnt.field; CountD r; r.v = a.v op (double)b; return r; }       \
  template <class T, class = typename std::enable_if<std::is_arithmetic<T>::value>::type>                       \
  inline CountD operator op(T a, CountD b) { ++g_cnt.field; CountD r; r.v = (double)a op b.v; return r; }
RPEG_BINOP(+, add)
RPEG_BINOP(-, add)
RPEG_BINOP(*, mul)
RPEG_BINOP(/, div)
#define RPEG_CMPOP(op)                                                                                          \
  inline bool operator op(CountD a, CountD b) { ++g_cnt.cmp; return a.v op b.v; }                               \
  template <class T, class = typename std::enable_if<std::is_arithmetic<T>::value>::type>                       \
  inline bool operator op(CountD a, T b) { ++g_cnt.cmp; return a.v op (double)b; }                              \
  template <class T, class = typename std::enable_if<std::is_arithmetic<T>::value>::type>                       \
  inline bool operator op(T a, CountD b) { ++g_cnt.cmp; return (double)a op b.v; }
RPEG_CMPOP(<)
RPEG_CMPOP(>)
RPEG_CMPOP(<=)
RPEG_CMPOP(>=)
RPEG_CMPOP(==)
RPEG_CMPOP(!=)
inline CountD count_fma(CountD a, CountD b, CountD c) { ++g_cnt.fma; CountD r; r.v = __builtin_fma(a.v, b.v, c.v); return r; }
static_assert(sizeof(CountD) == 8, "the problem record must keep its layout");
}  // namespace flopcount
using flopcount::CountD;
using flopcount::count_fma;
using flopcount::g_cnt;

#define double CountD
#define __builtin_fma count_fma
#include "../rpeg_amd/csrc/rpeg_lower.h"
#include "../rpeg_amd/csrc/rpeg_plan.h"
#undef __builtin_fma
#undef double

using namespace rpeg;

namespace {
struct CountMem {
  std::vector<CountD> t, r, d;
  std::vector<uint8_t> deg;
  std::vector<uint16_t> ready;
  void fit(const ClassHdr* h) {
    t.assign(h->n_nodes, CountD()); r.assign(h->n_nodes, CountD()); deg.assign(h->n_nodes, 0);
    d.assign(h->n_slots, CountD()); ready.assign(h->n_nodes + 1, 0);
  }
  CountD& time(int i) { return t[i]; }
  CountD& rank(int i) { return r[i]; }
  uint8_t& indeg(int i) { return deg[i]; }
  CountD dur(int s) const { return d[s]; }
  void set_dur(int s, CountD v) { d[s] = v; }
  uint16_t& rd_node(int j) { return ready[j]; }
  void on_schedule(int, CountD, CountD) {}
};
}  // namespace

extern "C" {

// Evaluates plans [0, n) one after the other and returns the fp64 operations they took, summed:
// out[0] additions and subtractions, [1] multiplications, [2] divisions, [3] fused multiply-adds,
// [4] comparisons (max, min and ordering), [5] plans evaluated (valid ones).  Returns 0, or -1 on a lowering error.
int flop_count(const void* problem, uint64_t n, const int16_t* vert, const uint8_t* head, uint64_t stride,
               uint32_t flags, uint64_t* out) {
  const rpeg_problem_t& P = *(const rpeg_problem_t*)problem;
  std::unordered_map<uint64_t, LoweredClass> classes;
  g_cnt = flopcount::Counters();
  uint64_t n_valid = 0;
  for (uint64_t i = 0; i < n; ++i) {
    PlanHead ph = load_head(head, stride, i);
    VPlan a[RPEG_MAX_V];
    std::memset(a, 0, sizeof a);
    const int nvs = (ph.structure >= 0 && ph.structure < P.n_struct) ? P.st[ph.structure].n_vertex : 0;
    for (int v = 0; v < nvs; ++v) load_vertex(vert, stride, i, v, &a[v]);
    if (!plan_valid(P, ph, a)) continue;
    const uint64_t sig = plan_signature(P, ph.structure, ph.split, ph.tau0, ph.tau1, a);
    auto it = classes.find(sig);
    if (it == classes.end()) {
      try { it = classes.emplace(sig, lower_class(P, sig)).first; } catch (const std::exception&) { return -1; }
    }
    ClassView cv = class_view(it->second.blob.data());
    CountMem mem;
    mem.fit(cv.h);
    (void)eval_plan(P, cv, ph, a, mem, (int)cv.h->n_nodes + 1, flags);
    ++n_valid;
  }
  out[0] = g_cnt.add; out[1] = g_cnt.mul; out[2] = g_cnt.div; out[3] = g_cnt.fma; out[4] = g_cnt.cmp; out[5] = n_valid;
  return 0;
}

}  // extern "C"
