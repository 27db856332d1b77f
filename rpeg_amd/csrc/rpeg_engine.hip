// rpeg_engine.hip - HIP kernels and C ABI of the batched plan evaluator (gfx950).
//
// Pipeline of rpeg_eval_batch:
//   k_signature   one thread per plan: integer validity gate, 64-bit class signature
//   host          new signatures are lowered once into class blobs (rpeg_lower.h) and cached in
//                 the engine; plans are ordered by class so that the lanes of a wavefront walk the
//                 same graph tables
//   k_eval        one thread per plan: durations of the class's slots (fp64 cost model), ranks,
//                 list scheduling, per-device memory peaks, score.  Per-plan state lives in a
//                 workspace laid out [row][lane] per wavefront (coalesced whenever lanes agree on
//                 the row); the ready list lives in LDS, [entry][lane].
//
// Build: hipcc --offload-arch=gfx950 -O3 -ffp-contract=off (no fused multiply-add may be formed:
// the scores must equal the reference's Python floats bit for bit).
#include <hip/hip_runtime.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "rpeg_kernel_eval.h"
#include "rpeg_kernel_plan.h"
#include "rpeg_kernel_prologue.h"
#include "rpeg_kernel_quad.h"
#include "rpeg_lower.h"
#include "rpeg_plan.h"
#include "rpeg_sa.h"

using namespace rpeg;

namespace {

constexpr int WAVE = 64;
constexpr uint32_t IDLE_LANE = 0xFFFFFFFFu;  // padding lane of a partly filled wavefront

#define HIP_TRY(e, call)                                                                   \
  do {                                                                                     \
    hipError_t _s = (call);                                                                \
    if (_s != hipSuccess) {                                                                \
      (e)->err = std::string(#call) + ": " + hipGetErrorString(_s);                        \
      return -2;                                                                           \
    }                                                                                      \
  } while (0)

struct DevMem {
  double* t;       // time rows, pre-offset by lane
  double* r;       // rank rows
  double* d;       // duration rows
  uint8_t* deg;    // in-degree rows
  uint16_t* ready; // ready list, one entry per node (the heap of the reference has no capacity), pre-offset by lane
  double* tr_start;   // optional start / finish time per node, elements `tr_stride` apart
  double* tr_finish;
  int32_t* tr_seq;    // optional dispatch index per node
  int32_t seq;
  size_t tr_stride;
  __device__ double& time(int i) { return t[(size_t)i * WAVE]; }
  __device__ double& rank(int i) { return r[(size_t)i * WAVE]; }
  __device__ uint8_t& indeg(int i) { return deg[(size_t)i * WAVE]; }
  __device__ double dur(int s) const { return d[(size_t)s * WAVE]; }
  __device__ void set_dur(int s, double v) { d[(size_t)s * WAVE] = v; }
  __device__ uint16_t& rd_node(int j) { return ready[j * WAVE]; }
  __device__ void on_schedule(int v, double s, double f) {
    if (tr_start) { tr_start[(size_t)v * tr_stride] = s; tr_finish[(size_t)v * tr_stride] = f; }
    if (tr_seq) tr_seq[v] = seq++;
  }
};

// workspace of one wavefront of the generic kernel: time and rank rows, duration rows, in-degree rows, ready list
__host__ __device__ inline size_t wave_ws_bytes(uint32_t nodes, uint32_t slots) {
  size_t b = (size_t)WAVE * (16ull * nodes + 8ull * slots + 2ull * nodes + nodes);
  return (b + 255) & ~size_t(255);
}

constexpr uint32_t CID_INVALID = 0xFFFFFFFFu, CID_UNKNOWN = 0xFFFFFFFEu;
// Every class counts its plans in `shards` counters (the blocks of k_signature spread over them): thousands of
// wavefronts adding to the same few addresses serialise in the L2.  classes * shards stays near COUNT_SLOTS.
constexpr uint32_t COUNT_SLOTS = 16384, MAX_SHARDS = 64;

__host__ __device__ inline uint64_t sig_hash(uint64_t x) {
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

__global__ void k_fill_u32(uint32_t* p, uint64_t n, uint32_t v) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

// The layout of a call from the pinned buffer the host wrote it to (read in place, sixteen bytes per thread: a copy
// command ahead of the kernels costs a dozen microseconds before its first byte moves), and the idle marks of the
// permutation, in one launch.  n_quads: sixteen-byte words of the layout.
__global__ void k_upload_fill(const uint4* __restrict__ host_src, uint4* __restrict__ dst, uint64_t n_quads, uint32_t* __restrict__ p,
                              uint64_t n, uint32_t v) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n_quads) dst[i] = host_src[i];
  if (i < n) p[i] = v;
}

// The counters of the signature kernel, summed over the shards of every class by a block of its own.  The shards'
// counters become their offsets within the class, in place (k_scatter reads them there); the totals go to the host:
// written into pinned host memory, then a flag the host polls -- there several microseconds before a copy command
// behind the kernel would have moved its first byte.  host_count: n_classes totals, the count of the plans of classes
// not lowered yet, then the KE_NEED_SHARDS running maxima of the ready-list length.
constexpr int HAND_BLOCK = 1024;
__global__ __launch_bounds__(HAND_BLOCK) void k_hand_counts(uint32_t* __restrict__ count, const uint32_t* __restrict__ need, uint32_t n_classes,
                                                            uint32_t shards, uint32_t* __restrict__ host_count, uint32_t* __restrict__ host_flag,
                                                            uint32_t tag) {
  // the totals first, and on their way to the host before anything else is written
  for (uint32_t c = threadIdx.x; c < n_classes; c += HAND_BLOCK) {
    const uint32_t* row = count + (size_t)c * shards;
    uint32_t total = 0;
    for (uint32_t s0 = 0; s0 < shards; s0 += 16) {   // sixteen loads in flight
      uint32_t v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = s0 + u < shards ? row[s0 + u] : 0u;
#pragma unroll
      for (int u = 0; u < 16; ++u) total += v[u];
    }
    host_count[c] = total;
  }
  if (threadIdx.x == 0) host_count[n_classes] = count[(size_t)n_classes * shards];
  if (threadIdx.x < KE_NEED_SHARDS) host_count[n_classes + 1 + threadIdx.x] = need[threadIdx.x];
  __threadfence_system();
  __syncthreads();
  if (threadIdx.x == 0) __hip_atomic_store(host_flag, tag, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  // then the shards' counters become their offsets within the class (for the kernels that follow on the device)
  for (uint32_t c = threadIdx.x; c < n_classes; c += HAND_BLOCK) {
    uint32_t* row = count + (size_t)c * shards;
    uint32_t total = 0;
    for (uint32_t s0 = 0; s0 < shards; s0 += 16) {
      uint32_t v[16];
#pragma unroll
      for (int u = 0; u < 16; ++u) v[u] = s0 + u < shards ? row[s0 + u] : 0u;
#pragma unroll
      for (int u = 0; u < 16; ++u)
        if (s0 + u < shards) { row[s0 + u] = total; total += v[u]; }
    }
  }
}

// Integer validity gate, class signature, class id (open-addressing table of the classes lowered so far)
// and the per-class plan counts.  Blocks of SIG_BLOCK plans; shard = block mod shards.
constexpr int SIG_BLOCK = 256, SIG_TABLE = 512;
constexpr size_t DIRECT_MAX_CLASSES = 32;   // engines of at most this many classes evaluate small batches without a layout,
constexpr uint64_t DIRECT_WAVES_PER_CU = 8; // and so does every batch of at most this many plans per compute unit
constexpr uint32_t N_QUEUES = 4;   // task counters of a call's evaluation launches (main kernel, k_quad, k_plan, spare)
struct SigPlans {   // the plan fields of one thread's plan, a column of an LDS array [field][thread]
  const int16_t* col;
  __device__ VPlan operator[](int v) const { return ke_vplan<SIG_BLOCK>(col, v); }
};
// Validity gate and class signature of the plan of this thread (SIG_INVALID for an inactive thread or a plan
// that breaks a rule).  s_plan: LDS, [field][thread]; the gate and the signature index the vertices with
// run-time values, which would put a per-thread array into scratch memory.
// The structure decides which tables the gate and the signature read.  It is made uniform (one pass per
// distinct structure among the plans of the wavefront) so that those reads are scalar loads.
__device__ inline uint64_t sig_of_thread(const rpeg_problem_t* __restrict__ P, const bool active, const uint64_t i,
                                         const PlanHead h, const int16_t* __restrict__ vert, const uint64_t stride,
                                         int16_t* s_plan) {
  uint64_t sg = SIG_INVALID;
  const bool known = active && h.structure >= 0 && h.structure < P->n_struct;
  unsigned long long todo = __ballot(known);
  while (todo) {
    const int su = __builtin_amdgcn_readlane(h.structure, __builtin_ctzll(todo));
    const bool mine = known && h.structure == su;
    todo &= ~__ballot(mine);
    if (mine) {
      const int nv = P->st[su].n_vertex;
      {  // every load of a vertex is issued before the first is waited for
        const int16_t* src = vert + i;
        int16_t* dst = s_plan + threadIdx.x;
#pragma unroll
        for (int v = 0; v < RPEG_MAX_V; ++v) {
          if (v >= nv) break;
          int16_t t[RPEG_FIELDS];
#pragma unroll
          for (int f = 0; f < RPEG_FIELDS; ++f) t[f] = src[(uint64_t)(v * RPEG_FIELDS + f) * stride];
#pragma unroll
          for (int f = 0; f < RPEG_FIELDS; ++f) dst[(v * RPEG_FIELDS + f) * SIG_BLOCK] = t[f];
        }
      }
      const SigPlans a{s_plan + threadIdx.x};
      PlanHead hu = h;
      hu.structure = su;
      if (nv != 0 && plan_valid(*P, hu, a)) sg = plan_signature(*P, su, h.split, h.tau0, h.tau1, a);
    }
  }
  return sg;
}

__global__ __launch_bounds__(SIG_BLOCK) void k_signature(
    const rpeg_problem_t* __restrict__ P, uint64_t n, const int16_t* __restrict__ vert,
    const uint8_t* __restrict__ head, uint64_t stride, uint64_t* __restrict__ sig, double* makespan, double* peak,
    double* score, uint8_t* mask, double* mass, const uint64_t* __restrict__ hkey, const uint32_t* __restrict__ hval,
    uint32_t hmask, uint32_t* __restrict__ cid, uint32_t* __restrict__ kidx, uint32_t* __restrict__ count,
    uint32_t n_classes, uint32_t shards) {
  // counters met in this block: key, plans of the block, and the block's first arrival index
  __shared__ uint32_t t_key[SIG_TABLE], t_cnt[SIG_TABLE], t_base[SIG_TABLE];
  // plan fields: the gate and the signature index the vertices with run-time values, which would put a
  // per-thread array into scratch memory
  __shared__ int16_t s_plan[RPEG_MAX_V * RPEG_FIELDS * SIG_BLOCK];
  constexpr uint32_t NONE = 0xFFFFFFFFu;
  for (int j = threadIdx.x; j < SIG_TABLE; j += SIG_BLOCK) { t_key[j] = NONE; t_cnt[j] = 0u; }
  __syncthreads();
  const uint64_t i = (uint64_t)blockIdx.x * SIG_BLOCK + threadIdx.x;
  const bool active = i < n;
  PlanHead h;
  h.structure = h.split = h.tau0 = h.tau1 = 0;
  if (active) h = load_head(head, stride, i);
  const uint64_t sg = sig_of_thread(P, active, i, h, vert, stride, s_plan);
  uint32_t key = NONE;
  if (active) {
    sig[i] = sg;
    if (sg == SIG_INVALID) {
      const double nan = __builtin_nan("");
      if (makespan) makespan[i] = nan;
      if (peak) peak[i] = nan;
      if (score) score[i] = nan;
      if (mask) mask[i] = 0;
      if (mass)
        for (int x = 0; x < RPEG_MAX_V; ++x) mass[i * RPEG_MAX_V + x] = nan;
      cid[i] = CID_INVALID;
    } else {
      uint32_t c = CID_UNKNOWN;
      for (uint32_t slot = (uint32_t)sig_hash(sg) & hmask, probes = 0; probes <= hmask; slot = (slot + 1) & hmask, ++probes) {
        const uint64_t k = hkey[slot];
        if (k == sg) { c = hval[slot]; break; }
        if (k == SIG_INVALID) break;
      }
      cid[i] = c;
      // count[class * shards + shard]; the plans of classes not lowered yet share count[n_classes * shards]
      key = c == CID_UNKNOWN ? n_classes * shards : c * shards + (blockIdx.x & (shards - 1u));
    }
  }
  // Arrival index within (class, shard): the plans of the block are counted in LDS first, then every counter
  // the block met takes one atomic: thousands of wavefronts adding to the same address serialise in the L2.
  uint32_t slot = 0, local = 0;
  if (key != NONE) {
    slot = (key * 2654435761u >> 16) & (SIG_TABLE - 1);
    for (;;) {   // at most SIG_BLOCK distinct keys in SIG_TABLE slots: a free slot is always found
      const uint32_t prev = atomicCAS(&t_key[slot], NONE, key);
      if (prev == NONE || prev == key) break;
      slot = (slot + 1) & (SIG_TABLE - 1);
    }
    local = atomicAdd(&t_cnt[slot], 1u);
  }
  __syncthreads();
  for (int j = threadIdx.x; j < SIG_TABLE; j += SIG_BLOCK)
    if (t_cnt[j]) t_base[j] = atomicAdd(&count[t_key[j]], t_cnt[j]);
  __syncthreads();
  if (key != NONE) kidx[i] = t_base[slot] + local;
}

// The plan -> class step of the entry point that allocates nothing: validity gate, signature and, through the
// table of the classes lowered so far, the pool offset of the plan's class blob, written to cls[i] for the
// single-plan kernel (KP_SKIP for a plan that is not evaluated).  Plans that break a rule get the outputs
// k_signature gives them; plans of a class that is not on the device yet get NaN outputs, RPEG_MASK_ERROR and
// are counted in counters[0].
__global__ __launch_bounds__(SIG_BLOCK) void k_class_direct(
    const rpeg_problem_t* __restrict__ P, uint64_t n, const int16_t* __restrict__ vert,
    const uint8_t* __restrict__ head, uint64_t stride, double* makespan, double* peak, double* score, uint8_t* mask,
    double* mass, const uint64_t* __restrict__ hkey, const uint32_t* __restrict__ hoff, uint32_t hmask,
    uint32_t* __restrict__ cls, uint32_t* __restrict__ counters) {
  __shared__ int16_t s_plan[RPEG_MAX_V * RPEG_FIELDS * SIG_BLOCK];
  const uint64_t i = (uint64_t)blockIdx.x * SIG_BLOCK + threadIdx.x;
  const bool active = i < n;
  PlanHead h;
  h.structure = h.split = h.tau0 = h.tau1 = 0;
  if (active) h = load_head(head, stride, i);
  const uint64_t sg = sig_of_thread(P, active, i, h, vert, stride, s_plan);
  bool unknown = false;
  if (active) {
    uint32_t off = KP_SKIP;
    if (sg != SIG_INVALID) {
      unknown = true;
      for (uint32_t slot = (uint32_t)sig_hash(sg) & hmask, probes = 0; probes <= hmask; slot = (slot + 1) & hmask, ++probes) {
        const uint64_t k = hkey[slot];
        if (k == sg) { off = hoff[slot]; unknown = false; break; }
        if (k == SIG_INVALID) break;
      }
    }
    cls[i] = off;
    if (off == KP_SKIP) {
      const double nan = __builtin_nan("");
      if (makespan) makespan[i] = nan;
      if (peak) peak[i] = nan;
      if (score) score[i] = nan;
      if (mask) mask[i] = unknown ? (uint8_t)(RPEG_MASK_VALID | RPEG_MASK_ERROR) : (uint8_t)0;
      if (mass)
        for (int x = 0; x < RPEG_MAX_V; ++x) mass[i * RPEG_MAX_V + x] = nan;
    }
  }
  const unsigned long long u = __ballot(unknown);
  if (u && (threadIdx.x & (WAVE - 1)) == 0) atomicAdd(&counters[0], (uint32_t)__builtin_popcountll(u));
}

// cbase[class * shards + shard]: plans of the class in lower shards; shard as in k_signature.
__global__ void k_scatter(uint64_t n, const uint32_t* __restrict__ cid, const uint32_t* __restrict__ kidx,
                          const uint32_t* __restrict__ cfirst, const uint32_t* __restrict__ clpw,
                          const uint32_t* __restrict__ cbase, uint32_t shards, uint32_t* __restrict__ perm,
                          uint32_t pstride, const uint32_t* __restrict__ coff, uint32_t* __restrict__ task_cls,
                          uint32_t first_entry, uint32_t* __restrict__ queues, uint32_t* __restrict__ limit) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < N_QUEUES) queues[i] = 0u;   // the task counters of the evaluation kernels that follow on this stream
  if (i == 0) limit[0] = 0u;          // and the count of plans for the launch that ends the call
  if (i >= n) return;
  const uint32_t c = cid[i];
  if (c >= CID_UNKNOWN) return;
  const uint32_t k = cbase[c * shards + ((uint32_t)(i / SIG_BLOCK) & (shards - 1u))] + kidx[i], l = clpw[c] & 0xFFFFu;
  if (clpw[c] >> 16) {   // a class of single-plan wavefronts: cfirst is its first entry; the task learns its class here
    perm[(uint64_t)cfirst[c] + k] = (uint32_t)i;
    task_cls[cfirst[c] + k - first_entry] = coff[c];
  } else perm[(uint64_t)(cfirst[c] + k / l) * pstride + k % l] = (uint32_t)i;
}

// The prologue launches (rpeg_kernel_prologue.h), a thread per plan in the caller's order.  The structure decides
// which tables a plan reads; it is made uniform (one pass per distinct structure among the plans of the wavefront) so
// that those reads are scalar loads and the walk through the slot universe is one path.
__global__ __launch_bounds__(WAVE) void k_prologue(const PrologueLaunch L) {
  const uint64_t i = (uint64_t)blockIdx.x * WAVE + threadIdx.x;
  const bool active = i < L.n && L.cid[i] != KPRO_INVALID;
  int su = 0, split = 0;
  if (active) { su = L.head[0 * L.stride + i]; split = L.head[1 * L.stride + i]; }
  unsigned long long todo = __ballot(active);
  while (todo) {
    const int s0 = __builtin_amdgcn_readlane(su, __builtin_ctzll(todo));
    const bool mine = active && su == s0;
    todo &= ~__ballot(mine);
    if (mine)
      for (int row = (int)blockIdx.y; row < (int)(L.max_uni + 1 + RPEG_MAX_V); row += (int)gridDim.y) kpro_row(L, i, s0, split, row);
  }
}

// (LDS by the problem's largest vertex count, kpeaks_lds_bytes: beside a resident main kernel the blocks of this launch
// get what LDS that kernel leaves, and with the 12.8 KB of six vertices a DPO batch of three had half as many of them)
static size_t kpeaks_lds_bytes(uint32_t max_v) { return (size_t)max_v * 4 * WAVE * 8 + 8 * WAVE; }
__global__ __launch_bounds__(WAVE) void k_peaks(const PrologueLaunch L) {
  extern __shared__ double kpk_lds[];
  double* l_vm = kpk_lds;                                        // [vertex * 4 + field][lane]
  uint8_t* l_ord = (uint8_t*)(kpk_lds + (size_t)L.max_v * 4 * WAVE);   // [position][lane]
  const uint64_t i = (uint64_t)blockIdx.x * WAVE + threadIdx.x;
  const bool active = i < L.n && L.cid[i] != KPRO_INVALID;
  PlanHead h;
  h.structure = h.split = h.tau0 = h.tau1 = 0;
  if (active) h = load_head(L.head, L.stride, i);
  unsigned long long todo = __ballot(active);
  while (todo) {
    const int su = __builtin_amdgcn_readlane(h.structure, __builtin_ctzll(todo));
    const bool mine = active && h.structure == su;
    todo &= ~__ballot(mine);
    if (mine) kpro_peaks(L, i, su, h, l_vm + threadIdx.x, l_ord + threadIdx.x);
  }
}

// The verdicts of the memory-model launch put into the outputs of the scheduling kernels, where that launch ran beside
// them instead of ahead of them: the gate bits of the mask, the soft OOM penalty and the stale-layout gate of the
// score (evaluate.py:372-374, 396-401), the same operations in the same order as the scheduling kernels apply them.
// (It also clears the class counters for the signature kernel of the engine's next call, which then starts without a
// launch of its own for that: zero_n words at zero_p.)
__global__ void k_finish(uint64_t n, const uint32_t* __restrict__ cid, const double* __restrict__ pen,
                         const uint8_t* __restrict__ gates, uint32_t flags, double* __restrict__ score, uint8_t* __restrict__ mask,
                         uint32_t* __restrict__ zero_p, uint32_t zero_n) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (uint64_t j = i; j < zero_n; j += (uint64_t)gridDim.x * blockDim.x) zero_p[j] = 0u;
  if (i >= n || cid[i] == KPRO_INVALID) return;   // (a plan the gate rejected has its outputs from k_signature)
  const uint8_t g = gates[i];
  const bool stale_ok = (g & RPEG_MASK_STALE_OK) != 0, mem_ok = (g & RPEG_MASK_MEM_OK) != 0;
  if (mask) {
    const uint8_t m = mask[i];
    mask[i] = (uint8_t)((m & ~(RPEG_MASK_STALE_OK | RPEG_MASK_MEM_OK)) | (g & (RPEG_MASK_STALE_OK | RPEG_MASK_MEM_OK)));
  }
  if (score) {
    double sc = score[i];
    if (sc != sc) return;   // RPEG_MASK_ERROR: the NaN stays
    if (!mem_ok) sc = sc * pen[i];
    if ((flags & RPEG_GATE_STALE) && !stale_ok) sc = 0.0;
    score[i] = sc;
  }
}

// The next wave task of a launch whose wavefronts take tasks as they become free (every wavefront ends when the
// counter has passed the last task), or the next of this block's own.
__device__ inline uint64_t next_task(const EvalLaunch& L, uint64_t w) {
  if (!L.queue) return w + gridDim.x;
  uint32_t t = 0;
  if (threadIdx.x == 0) t = atomicAdd(L.queue, 1u);
  return (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((int)t);
}

template <int LS>
__global__ __launch_bounds__(WAVE) void k_eval(const EvalLaunch L) {
  extern __shared__ uint8_t ke_lds[];
  if ((L.flags & KE_FIXUP) && L.need && L.need[KE_NEED_SHARDS] == 0u) return;   // no plan outgrew its list
  for (uint64_t w = L.queue ? next_task(L, 0) : blockIdx.x; w < L.n_waves; w = next_task(L, w)) {
    if (LS == 0 && (L.wave_cls[w] & KE_CLS_LDS)) ke_eval_wave<KE_FEW>(L, w, ke_lds);   // uniform branch
    else ke_eval_wave<LS>(L, w, ke_lds);
  }
}

// Four lanes per plan, sixteen plans per wavefront (rpeg_kernel_quad.h); tasks and permutation as for k_eval.
// At most 128 vector registers, so that a wavefront of it fits beside one of the main kernel and one of k_plan on a
// SIMD (the cost model spills a little; the scheduling loop does not).
__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(4, 8))) void k_quad(const EvalLaunch L) {
  extern __shared__ uint8_t kq_lds[];
  for (uint64_t w = blockIdx.x; w < L.n_waves; w += gridDim.x) kq_eval_wave(L, w, kq_lds);
}

// One plan per wavefront (rpeg_kernel_plan.h); perm[w] is the plan of wavefront task w.
__global__ __launch_bounds__(WAVE) __attribute__((amdgpu_waves_per_eu(4, 8))) void k_plan(const EvalLaunch L) {
  extern __shared__ uint8_t kp_lds[];
  for (uint64_t w = blockIdx.x; w < L.n_waves; w += gridDim.x) {
    const uint64_t pi = L.perm ? L.perm[w] : w;
    const uint32_t off = L.wave_cls[w];
    if (off == KP_SKIP) continue;   // uniform: a task without a plan to evaluate
    kp_eval_plan(L, w, pi, class_view(L.pool + off), kp_lds);
    // (lane 0 wrote the outputs of the task: its release store orders them before the flag)
    if (L.done && threadIdx.x == 0) __hip_atomic_store(&L.done[w], L.done_tag, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
  }
}

// Generic single-wavefront kernel over the host/device-shared scheduler template; used for the
// per-node trace of one plan.
__global__ __launch_bounds__(WAVE) void k_eval_generic(const rpeg_problem_t* __restrict__ P, uint64_t n_sorted,
                                               const int16_t* __restrict__ vert, const uint8_t* __restrict__ head,
                                               uint64_t stride, const uint32_t* __restrict__ perm,
                                               const uint32_t* __restrict__ wave_cls, const uint8_t* __restrict__ pool,
                                               uint8_t* __restrict__ ws, uint32_t ws_nodes, uint32_t ws_slots,
                                               uint32_t flags, double* makespan, double* peak, double* score,
                                               uint8_t* mask, double* tr_start, double* tr_finish, int32_t* tr_seq) {
  const int lane = threadIdx.x;
  const uint64_t n_waves = (n_sorted + WAVE - 1) / WAVE;
  uint8_t* base = ws + (size_t)blockIdx.x * wave_ws_bytes(ws_nodes, ws_slots);
  DevMem mem;
  mem.t = (double*)base + lane;
  mem.r = (double*)base + (size_t)ws_nodes * WAVE + lane;
  mem.d = (double*)base + 2 * (size_t)ws_nodes * WAVE + lane;
  mem.ready = (uint16_t*)(base + 8 * (2 * (size_t)ws_nodes + ws_slots) * WAVE) + lane;
  mem.deg = base + (8 * (2 * (size_t)ws_nodes + ws_slots) + 2 * (size_t)ws_nodes) * WAVE + lane;
  mem.tr_start = tr_start;
  mem.tr_finish = tr_finish;
  mem.tr_seq = tr_seq;
  mem.seq = 0;
  mem.tr_stride = 1;
  for (uint64_t w = blockIdx.x; w < n_waves; w += gridDim.x) {
    // every wavefront works on one class: the class tables are addressed uniformly (scalar loads)
    const ClassView cv = class_view(pool + wave_cls[w]);
    const uint64_t i = perm[w * WAVE + lane];
    if (i == IDLE_LANE) continue;
    PlanHead h = load_head(head, stride, i);
    VPlan a[RPEG_MAX_V];
    const int nv = P->st[h.structure].n_vertex;
    for (int v = 0; v < RPEG_MAX_V; ++v)
      if (v < nv) load_vertex(vert, stride, i, v, &a[v]);
    PlanOut o = eval_plan(*P, cv, h, a, mem, (int)ws_nodes, flags);
    if (makespan) makespan[i] = o.makespan;
    if (peak) peak[i] = o.peak;
    if (score) score[i] = o.score;
    if (mask) mask[i] = o.mask;
  }
}

// The launch that ends a batched call: the plans whose ready set outgrew what the evaluation kernels hold (flagged in
// EvalLaunch::limit) once more, one plan per lane, through the scheduler template with a ready list of one entry per
// node -- the reference's heap has no capacity (scheduler.py:423-546).  Lanes of a wavefront may work on different
// classes.  Ends at once when nothing is flagged, which is the rule: 32 entries hold every plan of the shipped
// configurations.  Per lane in `ws`: ready time, rank, start, finish per node, duration per slot, ready list,
// in-degree, interleaved by lane.
__host__ __device__ inline size_t limit_ws_bytes(uint32_t nodes, uint32_t slots) {
  size_t b = (size_t)WAVE * (32ull * nodes + 8ull * slots + 2ull * nodes + nodes);
  return (b + 255) & ~size_t(255);
}
__global__ __launch_bounds__(WAVE) void k_eval_limit(const EvalLaunch L, uint8_t* __restrict__ ws) {
  const uint32_t n = L.limit[0];
  if (n == 0) return;
  const int lane = threadIdx.x;
  const rpeg_problem_t& P = *L.P;
  uint8_t* base = ws + (size_t)blockIdx.x * limit_ws_bytes(L.ws_nodes, L.ws_slots);
  const size_t rows = (size_t)L.ws_nodes * WAVE;
  DevMem mem;
  mem.t = (double*)base + lane;
  mem.r = mem.t + rows;
  mem.tr_start = mem.r + rows;
  mem.tr_finish = mem.tr_start + rows;
  mem.d = mem.tr_finish + rows;
  mem.ready = (uint16_t*)((double*)base + 4 * rows + (size_t)L.ws_slots * WAVE) + lane;
  mem.deg = (uint8_t*)((uint16_t*)((double*)base + 4 * rows + (size_t)L.ws_slots * WAVE) + rows) + lane;
  mem.tr_seq = nullptr;
  mem.seq = 0;
  mem.tr_stride = WAVE;
  for (uint64_t k = (uint64_t)blockIdx.x * WAVE + lane; k < n; k += (uint64_t)gridDim.x * WAVE) {
    const uint64_t i = L.limit[1 + 2 * k];
    const ClassView cv = class_view(L.pool + L.limit[2 + 2 * k]);
    const PlanHead h = load_head(L.head, L.stride, i);
    VPlan a[RPEG_MAX_V];
    const int nv = P.st[h.structure].n_vertex;
    for (int v = 0; v < RPEG_MAX_V; ++v)
      if (v < nv) load_vertex(L.vert, L.stride, i, v, &a[v]);
    const PlanOut o = eval_plan(P, cv, h, a, mem, (int)cv.h->n_nodes, L.flags & RPEG_GATE_STALE);
    if (L.makespan) L.makespan[i] = o.makespan;
    if (L.peak) L.peak[i] = o.peak;
    if (L.score) L.score[i] = o.score;
    if (L.mask) L.mask[i] = o.mask;
    if (L.mass) {
      double m[RPEG_MAX_V];
      if (o.mask & RPEG_MASK_ERROR) {
        for (int x = 0; x < RPEG_MAX_V; ++x) m[x] = __builtin_nan("");
      } else {
        critical_mass(cv, [&](int v) { return mem.tr_finish[(size_t)v * WAVE]; }, [&](int v) { return mem.tr_start[(size_t)v * WAVE]; }, m);
      }
      for (int x = 0; x < RPEG_MAX_V; ++x) L.mass[i * RPEG_MAX_V + x] = m[x];
    }
  }
}

// Per-node quantities of ONE plan, for the host objects of the reference's API: lane s evaluates
// NodeCostModel.time of the nodes that share duration slot s (cost.py:66-88), lane M (a bit set of template
// vertices) the peak of a device that lies in exactly the allocations of M (memory.py:686-839; 0 for a set whose
// allocations do not all intersect).  All 64 lanes work on the same plan.
__global__ __launch_bounds__(WAVE) void k_plan_detail(const rpeg_problem_t* __restrict__ P, const int16_t* __restrict__ vert,
                                                      const uint8_t* __restrict__ head, const uint8_t* __restrict__ blob,
                                                      double* __restrict__ dur, double* __restrict__ set_peak) {
  const int lane = threadIdx.x;
  const ClassView cv = class_view(blob);
  const PlanHead h = load_head(head, 1, 0);
  const rpeg_struct_t& st = P->st[h.structure];
  const int nv = st.n_vertex;
  VPlan a[RPEG_MAX_V];
  for (int v = 0; v < RPEG_MAX_V; ++v)
    if (v < nv) load_vertex(vert, 1, 0, v, &a[v]);
  for (unsigned s = lane; s < cv.h->n_slots; s += WAVE) {
    bool zd = false;
    const double t = slot_duration(*P, st, h.split, cv.slot[s], a, &zd);
    dur[s] = zd ? __builtin_nan("") : t;
  }
  const PlanMasks pm = plan_masks(a, nv);
  const bool coresident = struct_coresident(st);
  VMem vm[RPEG_MAX_V];
  for (int v = 0; v < RPEG_MAX_V; ++v)
    if (v < nv) vm[v] = vertex_memory(*P, st.vertex[v], a[v], coresident);
  const VMemArray vma{vm};
  const StructMasks sm = struct_masks(st, cv.h->vorder);
  const unsigned M = (unsigned)lane;
  bool clique = M != 0u && M < (1u << nv);
  for (int v = 0; v < nv; ++v)
    if ((M >> v) & 1u) clique = clique && (mask_row(pm.ovl, v) & M) == M;
  set_peak[lane] = clique ? device_class_peak(*P, st, cv.h->vorder, sm, pm, vma, M) : 0.0;
}

__global__ void k_op_time(const rpeg_problem_t* __restrict__ P, uint64_t n, int structure, int vertex,
                          const int16_t* __restrict__ strat, uint64_t stride, double* time, double* peak) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const rpeg_vertex_t& vx = P->st[structure].vertex[vertex];
  VPlan a;
  a.dp = strat[0 * stride + i]; a.pp = strat[1 * stride + i]; a.tp = strat[2 * stride + i]; a.mb = strat[3 * stride + i];
  a.o[0] = a.o[1] = a.o[2] = 0;
  a.e[0] = strat[4 * stride + i]; a.e[1] = strat[5 * stride + i]; a.e[2] = strat[6 * stride + i];
  bool zd = a.dp < 1 || a.pp < 1 || a.tp < 1 || a.mb < 1 || a.e[2] < 1;
  if (zd) {
    if (time) time[i] = __builtin_nan("");
    if (peak) peak[i] = __builtin_nan("");
    return;
  }
  if (time) {
    double t = op_time(*P, vx, vx.unsplit, a, &zd);
    time[i] = zd ? __builtin_nan("") : t;
  }
  if (peak) peak[i] = isolated_peak(vx, vertex_memory(*P, vx, a));
}

__global__ void k_exp(uint64_t n, const double* x, double* y) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) y[i] = exp_libm(x[i]);
}

}  // namespace

// Scratch memory of rpeg_eval_batch_static, the entry point that allocates nothing: per plan the pool offset of
// its class blob (what the single-plan kernel takes as its task list), then a block of counters.  Every GPU
// the library runs on holds its own copy of the array until the process ends; the name below is only a
// host-side handle, the device address is looked up once per device (static_scratch_ptr) and that pointer is
// what kernels and copies get.
constexpr size_t STATIC_CLS_BYTES = (size_t)RPEG_STATIC_MAX_PLANS * 4, STATIC_COUNTER_BYTES = 256;
static __device__ __align__(256) uint8_t scratch[STATIC_CLS_BYTES + STATIC_COUNTER_BYTES];
constexpr int STATIC_MAX_DEVICES = 64;
static uint8_t* g_static_ptr[STATIC_MAX_DEVICES];
static std::mutex g_static_mu;

// device address of `scratch` on the current device `dev`; null on failure (status in *st)
static uint8_t* static_scratch_ptr(int dev, hipError_t* st) {
  *st = hipSuccess;
  if (dev < 0 || dev >= STATIC_MAX_DEVICES) { *st = hipErrorInvalidDevice; return nullptr; }
  std::lock_guard<std::mutex> lock(g_static_mu);
  if (!g_static_ptr[dev]) {
    void* p = nullptr;
    *st = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (*st != hipSuccess) return nullptr;
    g_static_ptr[dev] = (uint8_t*)p;
  }
  return g_static_ptr[dev];
}

// The fitted figures behind the split of a full batch between the three scheduling kernels, in one place.  They are
// microseconds of one wavefront on an MI355X, fitted to the per-wavefront clocks of configurations 2, 3 and 5
// (python -m rpeg_amd.engine.profile) and then to the step time of configuration 2 over a sweep of each figure;
// rpeg_engine_set_split_model replaces them (a measurement aid).  A wrong figure
// costs time, never a result: every kernel computes the same bits.
//   plan_a + plan_b x nodes                    what a plan costs k_plan (one plan per wavefront), beside the main kernel
//   quad_a + nodes x (quad_b + quad_c x pops)  a wavefront of k_quad (sixteen plans); pops = heap pops per dispatch,
//                                              as the main kernel measured them for the class
//   eff_beside_quad                            the part of the modelled room beside the main kernel that k_plan really
//                                              gets where k_quad takes its share of a compute unit too
//   quad_margin                                a class moves to k_quad only if it ends this much later in the main kernel
//   gain_threshold, gain_classes               a split by class size / by measured time must model this much earlier
struct SplitModel {
  double plan_a = 40.0, plan_b = 2.2;
  double quad_a = 40.0, quad_b = 1.6, quad_c = 0.45;
  double eff_beside_quad = 0.65;
  double quad_margin = 1.15;
  double gain_threshold = 0.97, gain_classes = 0.98;
};
constexpr int SPLIT_MODEL_FIELDS = 9;

// Staging of one small host-pointer evaluation: plans and class offsets in (pinned, then device), results out (pinned,
// written by the kernel itself), and which of the caller's plans went to the device.
struct HostLane {
  uint8_t *in = nullptr, *dev = nullptr, *out = nullptr;
  // `direct`: the kernel reads the plans from the pinned block itself (no copy ahead of the launch) and flags every
  // finished plan in the pinned result block, where the host polls for it instead of waiting for the launch to end:
  // for the steps of an annealing run, whose latency is what counts
  bool direct = false;
  uint8_t *in_dev = nullptr, *out_dev = nullptr;   // the pinned blocks as the device addresses them
  uint32_t tag = 0;
  size_t cap = 0;
  std::vector<uint32_t> idx;
  size_t n = 0, stride = 0;
  bool launched = false;
  void release() {
    if (in) { hipHostFree(in); hipFree(dev); hipHostFree(out); }
    in = dev = out = in_dev = out_dev = nullptr;
    cap = 0;
  }
};

struct rpeg_engine_s {
  rpeg_problem_t P;
  rpeg_problem_t* dP = nullptr;
  int device = 0;
  std::string err;
  // lowering classes
  std::unordered_map<uint64_t, uint32_t> class_off;  // signature -> byte offset in the pool
  std::vector<uint64_t> cls_sig;                     // class id -> signature / pool offset / node count
  std::vector<uint32_t> cls_off, cls_nodes, cls_slots;
  std::vector<uint32_t> cls_pops16;                  // learned, of the slowest full wavefront of the class in the main kernel:
                                                     // microseconds << 12 | heap pops per dispatch in sixteenths
  uint32_t* d_cstat = nullptr;                       // the device's copy, written by the main kernel
  uint32_t cstat_cap = 0;
  std::vector<uint8_t> cls_split;                    // where every class ran when that was last decided: 0 main kernel, 1 k_plan,
  uint64_t split_for_n = 0, split_at = 0;            // 2 k_quad, 255 not in that batch; the batch size and the call of that decision
  bool split_mass = false;
  uint32_t learn_calls = 0;                          // calls left after which the statistic is read back
  uint64_t batch_calls = 0;
  uint64_t* d_hkey = nullptr;                        // device table signature -> class id
  uint32_t* d_hval = nullptr;
  uint32_t* d_hoff = nullptr;                        // the same slots -> pool offset of the class blob
  uint32_t hcap = 0, tables_for = 0;                 // table capacity; class count the device tables reflect
  uint32_t ccap = 0;                                 // capacity of the per-class device arrays
  // per-class tables of a call, one block on each side: counters per (class, shard), which become the shards'
  // offsets, then first wavefront and plans per wavefront of every class
  uint32_t *d_ccount = nullptr, *h_ccount = nullptr;
  uint64_t count_clean = 0;                     // leading words of d_ccount that the last call left at zero,
  hipStream_t count_clean_on = nullptr;         // on this stream
  uint32_t* h_ccount_dev = nullptr;             // the same pinned buffer as the device addresses it
  uint32_t *h_tot = nullptr, *h_tot_dev = nullptr;   // pinned: per-class totals of a call, written by k_hand_counts
  uint32_t *h_sigflag = nullptr, *h_sigflag_dev = nullptr;   // pinned word: the tag of the call whose counters are in h_ccount
  uint32_t sig_tag = 0;
  uint32_t *d_cid = nullptr, *d_kidx = nullptr;   // per plan: class id, arrival index within the class
  std::vector<uint8_t> pool;
  uint8_t* d_pool = nullptr;
  size_t d_pool_cap = 0, d_pool_used = 0;
  uint32_t max_nodes = 1, max_slots = 1, max_cls_bytes = 16;
  bool lds_attr_set[5] = {false, false, false, false, false};
  // staging of the host-pointer path: plans and class offsets in (pinned, then device), results out (pinned,
  // written by the kernel itself)
  HostLane lane0;
  uint8_t* d_stage = nullptr;   // device copy of host tensors and results for larger host-pointer batches
  size_t d_stage_cap = 0;
  uint8_t* h_stage = nullptr;   // pinned mirror of the result region of d_stage
  size_t h_stage_cap = 0;
  uint8_t* d_trace = nullptr;   // rpeg_eval_trace: one plan's fields and header, then start / finish / dispatch index
  uint8_t* d_detail = nullptr;  // rpeg_plan_detail: one plan's fields and header, then slot durations and vertex-set peaks
  size_t d_trace_nodes = 0;
  SplitModel split_model;
  int sa_lanes = 3;     // rpeg_sa_run: groups of chains whose evaluations overlap the host's work on the others
  int lanes_busy = 0;   // evaluations submitted on lanes and not yet collected (their kernels read d_pool)
  uint64_t relearn_at = 0;                // the call that last asked for the measurements again
  uint32_t one_plan_waves_per_cu = 64;    // batches of at most this many plans per compute unit take one wavefront per plan
  uint32_t host_small_max = 1024;          // rpeg_eval_host: largest batch whose classes the host looks up itself
  int state_lanes = -1;   // -1: chosen per batch; 0: per-plan state in HBM; 8/16/32/64: in LDS, that many plans per wavefront; 1: one plan per wavefront (k_plan)
  bool prof_on = false;
  unsigned long long* d_prof = nullptr;
  uint64_t prof_waves = 0;
  // per-batch buffers
  size_t cap_n = 0, cap_perm = 0, cap_cls = 0;
  // Ready-list capacity of k_eval: learned from the longest list seen so far (running maxima kept by the
  // kernel, read back with the class counts of the next call); plans that outgrow it are flagged and redone
  // with the full capacity by a second launch.
  uint8_t* d_ovf = nullptr;
  uint32_t ready_cap = 32;      // ready-list entries per plan in the main kernel (rpeg_engine_set_ready_cap)
  uint32_t* d_need = nullptr;
  uint32_t need = 0;
  uint32_t max_v = RPEG_MAX_V;   // largest vertex count of the problem's structures
  hipStream_t s2 = nullptr;                     // second stream: single-plan wavefronts of a large batch run beside the others
  hipEvent_t ev_fork = nullptr, ev_join = nullptr;
  hipEvent_t ev_counts = nullptr;               // the statistic of a call has reached the host (the calls that read it)
  hipStream_t s3 = nullptr;                     // third stream: the four-lanes-per-plan wavefronts (k_quad)
  hipEvent_t ev_join3 = nullptr;
  hipEvent_t ev_sig = nullptr;                  // the signature kernel of a call is done (its class ids are there)
  bool layout_ahead = true;                     // prologue, layout and main kernel on k_quad's stream (see `ahead` in eval_batch_impl)
  int side_dev = 0;                             // device of the side streams
  uint32_t quad_share_pct = 25;                 // share of a full batch that k_quad takes (rpeg_engine_set_quad_share)
  bool quad_attr_set = false;
  int split_heavy = 1;                          // 0: the classes with the largest graphs stay in the main kernel
  uint64_t* d_sig = nullptr;
  uint64_t* h_sig = nullptr;
  uint32_t *d_perm = nullptr, *d_cls = nullptr, *h_cls = nullptr;   // lane -> plan; wavefront -> class blob
  uint8_t* d_ws = nullptr;
  // outputs of the prologue launches (rpeg_kernel_prologue.h), cap_n plans each: pair relations, penalty factor, gate
  // bits; the durations of the slot universe ([slot][plan]); and the universe itself
  uint64_t *d_aux_ovl = nullptr, *d_aux_dpne = nullptr, *d_aux_eq = nullptr;
  double* d_vm = nullptr;
  double* d_aux_pen = nullptr;
  uint8_t* d_aux_mask = nullptr;
  double* d_dur = nullptr;
  size_t dur_cap = 0;
  SlotDesc* d_uni = nullptr;
  uint32_t n_uni[RPEG_MAX_STRUCT] = {0, 0, 0}, max_uni = 0;
  uint32_t* d_queues = nullptr;                 // N_QUEUES task counters, cleared by k_scatter
  uint32_t* d_limit = nullptr;                  // count, then (plan, class offset) pairs: plans to redo without a bound on the ready set
  uint8_t* d_limit_ws = nullptr;                // state of the launch that redoes them
  size_t limit_ws_cap = 0;
  uint32_t limit_grid = 0;
  size_t ws_cap = 0;
  // timing / stats
  bool timing = false;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  double last_ms = -1.0;
  uint64_t stats[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  double host_us[4] = {0, 0, 0, 0};   // host time of the last laid-out rpeg_eval_batch call: rpeg_engine_host_us
  int n_cu = 256;
  uint8_t* static_ptr = nullptr;    // this device's copy of the file-scope scratch array (rpeg_eval_batch_static)
  uint32_t* h_static = nullptr;     // pinned: the counters of that array, read back after a call
  std::vector<uint32_t> cls_sorted, cls_pos;   // all classes by node count (largest first); place of a class among those of the batch
};

static int ensure_batch(rpeg_engine_t* e, size_t n) {
  if (n <= e->cap_n) return 0;
  size_t cap = std::max<size_t>(n, 4096);
  if (e->d_sig) {
    hipFree(e->d_sig); hipHostFree(e->h_sig); hipFree(e->d_cid); hipFree(e->d_kidx); hipFree(e->d_ovf); hipFree(e->d_limit);
    hipFree(e->d_aux_ovl); hipFree(e->d_aux_dpne); hipFree(e->d_aux_pen); hipFree(e->d_aux_mask); hipFree(e->d_dur);
    hipFree(e->d_aux_eq); hipFree(e->d_vm);
    e->d_dur = nullptr;
  }
  e->cap_n = 0;
  HIP_TRY(e, hipMalloc(&e->d_ovf, cap));
  HIP_TRY(e, hipMemset(e->d_ovf, 0, cap));   // flags are cleared again by the launch that consumes them
  if (!e->d_queues) {
    HIP_TRY(e, hipMalloc(&e->d_queues, N_QUEUES * 4));
    HIP_TRY(e, hipMemset(e->d_queues, 0, N_QUEUES * 4));
  }
  if (!e->d_need) {
    HIP_TRY(e, hipMalloc(&e->d_need, (KE_NEED_SHARDS + 1) * 4));
    HIP_TRY(e, hipMemset(e->d_need, 0, (KE_NEED_SHARDS + 1) * 4));
  } else {
    HIP_TRY(e, hipMemset(e->d_need + KE_NEED_SHARDS, 0, 4));   // the count of flagged plans belongs to the flags just replaced
  }
  HIP_TRY(e, hipMalloc(&e->d_sig, cap * 8));
  HIP_TRY(e, hipHostMalloc(&e->h_sig, cap * 8));
  HIP_TRY(e, hipMalloc(&e->d_cid, cap * 4));
  HIP_TRY(e, hipMalloc(&e->d_kidx, cap * 4));
  HIP_TRY(e, hipMalloc(&e->d_limit, (1 + 2 * cap) * 4));
  HIP_TRY(e, hipMemset(e->d_limit, 0, 4));
  HIP_TRY(e, hipMalloc(&e->d_aux_ovl, cap * 8));
  HIP_TRY(e, hipMalloc(&e->d_aux_dpne, cap * 8));
  HIP_TRY(e, hipMalloc(&e->d_aux_pen, cap * 8));
  HIP_TRY(e, hipMalloc(&e->d_aux_mask, cap));
  HIP_TRY(e, hipMalloc(&e->d_aux_eq, cap * 8));
  HIP_TRY(e, hipMalloc(&e->d_vm, cap * 8 * 4 * RPEG_MAX_V));
  HIP_TRY(e, hipMalloc(&e->d_dur, cap * 8 * (size_t)std::max<uint32_t>(e->max_uni, 1)));
  e->cap_n = cap;
  return 0;
}

// device copies of the class tables: signature -> class id, and room for the per-class counters
static int ensure_class_tables(rpeg_engine_t* e, hipStream_t s) {
  const uint32_t ncls = (uint32_t)e->cls_sig.size();
  if (e->d_hkey && e->tables_for == ncls) return 0;
  HIP_TRY(e, hipStreamSynchronize(s));
  uint32_t hcap = 1024;
  while (hcap < 4 * ncls) hcap *= 2;
  if (hcap != e->hcap) {
    if (e->d_hkey) { hipFree(e->d_hkey); hipFree(e->d_hval); hipFree(e->d_hoff); }
    e->d_hkey = nullptr; e->hcap = 0;
    HIP_TRY(e, hipMalloc(&e->d_hkey, (size_t)hcap * 8));
    HIP_TRY(e, hipMalloc(&e->d_hval, (size_t)hcap * 4));
    HIP_TRY(e, hipMalloc(&e->d_hoff, (size_t)hcap * 4));
    e->hcap = hcap;
  }
  std::vector<uint64_t> hk(hcap, SIG_INVALID);
  std::vector<uint32_t> hv(hcap, 0), ho(hcap, 0);
  for (uint32_t c = 0; c < ncls; ++c) {
    uint32_t slot = (uint32_t)sig_hash(e->cls_sig[c]) & (hcap - 1);
    while (hk[slot] != SIG_INVALID) slot = (slot + 1) & (hcap - 1);
    hk[slot] = e->cls_sig[c];
    hv[slot] = c;
    ho[slot] = e->cls_off[c];
  }
  HIP_TRY(e, hipMemcpy(e->d_hkey, hk.data(), (size_t)hcap * 8, hipMemcpyHostToDevice));
  HIP_TRY(e, hipMemcpy(e->d_hval, hv.data(), (size_t)hcap * 4, hipMemcpyHostToDevice));
  HIP_TRY(e, hipMemcpy(e->d_hoff, ho.data(), (size_t)hcap * 4, hipMemcpyHostToDevice));
  if (ncls + 1 > e->ccap) {
    const uint32_t cap = std::max<uint32_t>(2 * (ncls + 1), 4096);
    if (e->d_ccount) {
      hipFree(e->d_ccount);
      hipHostFree(e->h_ccount);
    }
    e->d_ccount = nullptr; e->ccap = 0;
    e->count_clean = 0;
    HIP_TRY(e, hipMalloc(&e->d_ccount, (4 * (size_t)cap + COUNT_SLOTS + 64) * 4));
    // (the signature kernel writes the counters here itself while the host polls: coherent, and mapped)
    HIP_TRY(e, hipHostMalloc(&e->h_ccount, (4 * (size_t)cap + COUNT_SLOTS + 64) * 4, hipHostMallocCoherent));
    e->h_ccount_dev = nullptr;
    HIP_TRY(e, hipHostGetDevicePointer((void**)&e->h_ccount_dev, e->h_ccount, 0));
    if (e->h_tot) hipHostFree(e->h_tot);
    e->h_tot = e->h_tot_dev = nullptr;
    HIP_TRY(e, hipHostMalloc(&e->h_tot, ((size_t)cap + 1 + KE_NEED_SHARDS) * 4, hipHostMallocCoherent));
    HIP_TRY(e, hipHostGetDevicePointer((void**)&e->h_tot_dev, e->h_tot, 0));
    if (!e->h_sigflag) {
      HIP_TRY(e, hipHostMalloc(&e->h_sigflag, 64, hipHostMallocCoherent));
      std::memset(e->h_sigflag, 0, 64);
      HIP_TRY(e, hipHostGetDevicePointer((void**)&e->h_sigflag_dev, e->h_sigflag, 0));
    }
    e->ccap = cap;
  }
  if (ncls > e->cstat_cap) {   // the per-class statistic keeps what it has learned
    const uint32_t cap = std::max<uint32_t>(2 * ncls, 4096);
    if (e->d_cstat) hipFree(e->d_cstat);
    e->d_cstat = nullptr; e->cstat_cap = 0;
    HIP_TRY(e, hipMalloc(&e->d_cstat, (size_t)cap * 4));
    HIP_TRY(e, hipMemset(e->d_cstat, 0, (size_t)cap * 4));
    HIP_TRY(e, hipMemcpy(e->d_cstat, e->cls_pops16.data(), (size_t)ncls * 4, hipMemcpyHostToDevice));
    e->cstat_cap = cap;
  }
  e->tables_for = ncls;
  return 0;
}

// permutation (one entry per lane, classes padded to wavefronts) and class offset per wavefront
static int ensure_perm(rpeg_engine_t* e, size_t lanes, size_t tasks) {
  if (lanes > e->cap_perm) {
    size_t cap = std::max<size_t>(lanes + lanes / 4, 8192);
    if (e->d_perm) hipFree(e->d_perm);
    e->d_perm = nullptr;
    e->cap_perm = 0;
    HIP_TRY(e, hipMalloc(&e->d_perm, cap * 4));
    e->cap_perm = cap;
  }
  if (tasks > e->cap_cls) {
    size_t cap = std::max<size_t>(tasks + tasks / 4, 1024);
    if (e->d_cls) { hipFree(e->d_cls); hipHostFree(e->h_cls); }
    e->d_cls = e->h_cls = nullptr;
    e->cap_cls = 0;
    HIP_TRY(e, hipMalloc(&e->d_cls, cap * 4));
    HIP_TRY(e, hipHostMalloc(&e->h_cls, cap * 4));
    e->cap_cls = cap;
  }
  return 0;
}

static int ensure_pool(rpeg_engine_t* e, hipStream_t s) {
  if (e->pool.size() > e->d_pool_cap) {
    size_t cap = std::max<size_t>(e->pool.size() * 2, 1 << 20);
    uint8_t* np = nullptr;
    HIP_TRY(e, hipMalloc(&np, cap));
    HIP_TRY(e, hipStreamSynchronize(s));
    if (e->lanes_busy > 0) HIP_TRY(e, hipDeviceSynchronize());   // kernels of other lanes still read the old pool
    if (e->d_pool) hipFree(e->d_pool);
    e->d_pool = np;
    e->d_pool_cap = cap;
    e->d_pool_used = 0;
  }
  if (e->pool.size() > e->d_pool_used) {
    HIP_TRY(e, hipMemcpyAsync(e->d_pool + e->d_pool_used, e->pool.data() + e->d_pool_used,
                              e->pool.size() - e->d_pool_used, hipMemcpyHostToDevice, s));
    // the host vector may reallocate on the next insertion: finish the copy first
    HIP_TRY(e, hipStreamSynchronize(s));
    e->d_pool_used = e->pool.size();
  }
  return 0;
}

// appends a lowered class to the engine's tables; returns its pool offset or -1
static int64_t class_append(rpeg_engine_t* e, uint64_t sig, const LoweredClass& lc) {
  const ClassHdr* h = (const ClassHdr*)lc.blob.data();
  e->max_nodes = std::max(e->max_nodes, h->n_nodes);
  e->max_slots = std::max(e->max_slots, h->n_slots);
  e->max_cls_bytes = std::max(e->max_cls_bytes, h->n_nodes * 8u + h->n_succ * 2u);
  if (e->pool.size() + lc.blob.size() >= (1ull << 31)) { e->err = "class pool exceeds 2 GiB"; return -1; }   // bit 31 of an offset is a flag
  uint32_t off = (uint32_t)e->pool.size();
  e->pool.insert(e->pool.end(), lc.blob.begin(), lc.blob.end());
  ((ClassHdr*)(e->pool.data() + off))->id = (uint32_t)e->cls_sig.size();
  e->class_off.emplace(sig, off);
  e->cls_sig.push_back(sig);
  e->cls_off.push_back(off);
  e->cls_nodes.push_back(h->n_nodes);
  e->cls_slots.push_back(h->n_slots);
  e->cls_pops16.push_back(0);
  e->learn_calls = 3;
  return off;
}

// returns the pool offset of the class of `sig`, lowering it on first sight; -1 on failure
static int64_t class_offset(rpeg_engine_t* e, uint64_t sig, bool* is_new) {
  auto it = e->class_off.find(sig);
  if (it != e->class_off.end()) return it->second;
  LoweredClass lc;
  try {
    lc = lower_class(e->P, sig);
  } catch (const std::exception& ex) {
    e->err = std::string("lowering failed: ") + ex.what();
    return -1;
  }
  if (is_new) *is_new = true;
  return class_append(e, sig, lc);
}

// lowers the classes of `sigs` that the engine does not hold yet, on up to eight host threads (lowering a
// class reads only the problem tables), and appends them in the order of `sigs`
static int lower_new_classes(rpeg_engine_t* e, const std::vector<uint64_t>& sigs, uint64_t* n_new) {
  std::vector<uint64_t> todo;
  {
    std::unordered_map<uint64_t, char> seen;
    for (uint64_t sg : sigs)
      if (!e->class_off.count(sg) && seen.emplace(sg, 1).second) todo.push_back(sg);
  }
  if (todo.empty()) return 0;
  std::vector<LoweredClass> lowered(todo.size());
  std::vector<std::string> errors(todo.size());
  const unsigned hw = std::max(1u, std::thread::hardware_concurrency());
  const size_t n_threads = std::min<size_t>({(size_t)8, (size_t)hw, (todo.size() + 15) / 16});
  auto work = [&](size_t t) {
    for (size_t i = t; i < todo.size(); i += n_threads) {
      try { lowered[i] = lower_class(e->P, todo[i]); } catch (const std::exception& ex) { errors[i] = ex.what(); if (errors[i].empty()) errors[i] = "error"; }
    }
  };
  if (n_threads <= 1) {
    work(0);
  } else {
    std::vector<std::thread> pool;
    for (size_t t = 0; t < n_threads; ++t) pool.emplace_back(work, t);
    for (auto& th : pool) th.join();
  }
  for (size_t i = 0; i < todo.size(); ++i) {
    if (!errors[i].empty()) { e->err = "lowering failed: " + errors[i]; return -5; }
    if (class_append(e, todo[i], lowered[i]) < 0) return -5;
  }
  *n_new += todo.size();
  return 0;
}

static int ensure_ws(rpeg_engine_t* e, size_t bytes, hipStream_t s) {
  if (bytes <= e->ws_cap) return 0;
  HIP_TRY(e, hipStreamSynchronize(s));
  if (e->d_ws) hipFree(e->d_ws);
  e->d_ws = nullptr;
  e->ws_cap = 0;
  HIP_TRY(e, hipMalloc(&e->d_ws, bytes));
  e->ws_cap = bytes;
  return 0;
}

// state of the launch that redoes flagged plans: as many wavefronts as 128 MiB hold, at most one per compute unit
static int ensure_limit_ws(rpeg_engine_t* e, hipStream_t s) {
  const size_t per_wave = limit_ws_bytes(e->max_nodes, e->max_slots);
  const uint32_t grid = (uint32_t)std::max<size_t>(1, std::min<size_t>((size_t)e->n_cu, ((size_t)128 << 20) / per_wave));
  if (per_wave * grid <= e->limit_ws_cap) { e->limit_grid = (uint32_t)std::min<size_t>(e->n_cu, e->limit_ws_cap / per_wave); return 0; }
  HIP_TRY(e, hipStreamSynchronize(s));
  if (e->d_limit_ws) hipFree(e->d_limit_ws);
  e->d_limit_ws = nullptr;
  e->limit_ws_cap = 0;
  HIP_TRY(e, hipMalloc(&e->d_limit_ws, per_wave * grid));
  e->limit_ws_cap = per_wave * grid;
  e->limit_grid = grid;
  return 0;
}

static int eval_batch_impl(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                           double* peak, double* score, uint8_t* mask, double* mass, void* stream);
static int eval_host_impl(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                          double* peak, double* score, uint8_t* mask, double* mass, void* stream);

extern "C" {

int rpeg_engine_create(const rpeg_problem_t* problem, rpeg_engine_t** out) {
  if (!problem || !out) return -1;
  *out = nullptr;
  if (problem->abi_version != RPEG_ABI_VERSION) return -3;
  if (problem->n_struct < 1 || problem->n_struct > RPEG_MAX_STRUCT || problem->n_split < 1 ||
      problem->n_split > RPEG_MAX_SPLIT || problem->K_eval < 1 || problem->transfer_both < 0 ||
      problem->transfer_both > 3)
    return -3;
  for (int s = 0; s < problem->n_struct; ++s) {
    const rpeg_struct_t& st = problem->st[s];
    if (st.n_vertex < 1 || st.n_vertex > RPEG_MAX_V || st.n_edge < 0 || st.n_edge > RPEG_MAX_E || st.n_pub < 0 ||
        st.n_pub > RPEG_MAX_PUB || st.n_pair < 0 || st.n_pair > RPEG_MAX_PAIR || st.n_rel < 0 || st.n_rel > RPEG_MAX_REL)
      return -3;
  }
  int count = 0;
  if (hipGetDeviceCount(&count) != hipSuccess || count < 1) return -4;  // no GPU: there is no CPU path
  rpeg_engine_t* e = new rpeg_engine_s();
  e->P = *problem;
  hipGetDevice(&e->device);
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, e->device) == hipSuccess) e->n_cu = prop.multiProcessorCount;
  e->max_v = 1;
  for (int q = 0; q < e->P.n_struct; ++q) e->max_v = std::max<uint32_t>(e->max_v, (uint32_t)e->P.st[q].n_vertex);

  {  // the device address of the static scratch array, once per device, with that device current
    hipError_t st;
    e->static_ptr = static_scratch_ptr(e->device, &st);
    if (!e->static_ptr || hipHostMalloc(&e->h_static, STATIC_COUNTER_BYTES) != hipSuccess) {
      delete e;
      return -2;
    }
  }
  {   // the slot universe of every structure, for the duration launch
    std::vector<SlotDesc> uni((size_t)RPEG_MAX_STRUCT * RPEG_MAX_UNIVERSE, SlotDesc{0, 0, 0, 0});
    for (int q = 0; q < e->P.n_struct; ++q) {
      const int nu = slot_universe(e->P, e->P.st[q], uni.data() + (size_t)q * RPEG_MAX_UNIVERSE);
      if (nu > RPEG_MAX_UNIVERSE) { delete e; return -3; }
      e->n_uni[q] = (uint32_t)nu;
      e->max_uni = std::max(e->max_uni, (uint32_t)nu);
    }
    if (hipMalloc(&e->d_uni, uni.size() * sizeof(SlotDesc)) != hipSuccess ||
        hipMemcpy(e->d_uni, uni.data(), uni.size() * sizeof(SlotDesc), hipMemcpyHostToDevice) != hipSuccess) {
      delete e;
      return -2;
    }
  }
  if (hipMalloc(&e->dP, sizeof(rpeg_problem_t)) != hipSuccess ||
      hipMemcpy(e->dP, problem, sizeof(rpeg_problem_t), hipMemcpyHostToDevice) != hipSuccess ||
      hipEventCreate(&e->ev0) != hipSuccess || hipEventCreate(&e->ev1) != hipSuccess) {
    delete e;
    return -2;
  }
  *out = e;
  return 0;
}

void rpeg_engine_destroy(rpeg_engine_t* e) {
  if (!e) return;
  hipDeviceSynchronize();
  if (e->dP) hipFree(e->dP);
  if (e->d_pool) hipFree(e->d_pool);
  if (e->d_sig) {
    hipFree(e->d_sig); hipHostFree(e->h_sig); hipFree(e->d_cid); hipFree(e->d_kidx); hipFree(e->d_ovf); hipFree(e->d_limit);
    hipFree(e->d_aux_ovl); hipFree(e->d_aux_dpne); hipFree(e->d_aux_pen); hipFree(e->d_aux_mask);
    hipFree(e->d_aux_eq); hipFree(e->d_vm);
  }
  if (e->d_limit_ws) hipFree(e->d_limit_ws);
  if (e->d_need) hipFree(e->d_need);
  if (e->d_queues) hipFree(e->d_queues);
  if (e->d_cstat) hipFree(e->d_cstat);
  if (e->d_hkey) { hipFree(e->d_hkey); hipFree(e->d_hval); hipFree(e->d_hoff); }
  if (e->h_static) hipHostFree(e->h_static);
  if (e->h_sigflag) hipHostFree(e->h_sigflag);
  if (e->h_tot) hipHostFree(e->h_tot);
  if (e->d_ccount) {
    hipFree(e->d_ccount);
    hipHostFree(e->h_ccount);
  }
  if (e->d_perm) hipFree(e->d_perm);
  if (e->d_dur) hipFree(e->d_dur);
  if (e->d_uni) hipFree(e->d_uni);
  if (e->d_cls) { hipFree(e->d_cls); hipHostFree(e->h_cls); }
  // (the side streams belong to the device, not to the engine: side_streams)
  if (e->s2) { hipStreamSynchronize(e->s2); hipEventDestroy(e->ev_fork); hipEventDestroy(e->ev_join); }
  if (e->s3) { hipStreamSynchronize(e->s3); hipEventDestroy(e->ev_join3); }
  if (e->ev_sig) hipEventDestroy(e->ev_sig);
  if (e->ev_counts) hipEventDestroy(e->ev_counts);
  e->lane0.release();
  if (e->d_stage) hipFree(e->d_stage);
  if (e->h_stage) hipHostFree(e->h_stage);
  if (e->d_trace) hipFree(e->d_trace);
  if (e->d_detail) hipFree(e->d_detail);
  if (e->d_ws) hipFree(e->d_ws);
  if (e->ev0) hipEventDestroy(e->ev0);
  if (e->ev1) hipEventDestroy(e->ev1);
  delete e;
}

const char* rpeg_last_error(const rpeg_engine_t* e) { return e ? e->err.c_str() : "null engine"; }

int rpeg_engine_set_timing(rpeg_engine_t* e, int32_t enabled) {
  if (!e) return -1;
  e->timing = enabled != 0;
  return 0;
}

double rpeg_engine_last_kernel_ms(const rpeg_engine_t* e) { return e ? e->last_ms : -1.0; }

// Phase clocks of the last batch (development aid): 8 counters of the 100 MHz wall clock per wavefront.
int rpeg_engine_profile(rpeg_engine_t* e, int32_t enable, unsigned long long* out, uint64_t cap_waves) {
  if (!e) return -1;
  e->prof_on = enable != 0;
  if (out && e->d_prof) {
    uint64_t nw = std::min<uint64_t>(cap_waves, e->prof_waves);
    hipDeviceSynchronize();
    hipMemcpy(out, e->d_prof, nw * 64, hipMemcpyDeviceToHost);
    return (int)nw;
  }
  return 0;
}

int rpeg_engine_set_state_lanes(rpeg_engine_t* e, int32_t lanes) {
  if (!e) return -1;
  if (lanes != -1 && lanes != 0 && lanes != 1 && lanes != 4 && lanes != 8 && lanes != 16 && lanes != 32 && lanes != 64) {
    e->err = "state lanes must be -1, 0, 1, 4, 8, 16, 32 or 64";
    return -1;
  }
  e->state_lanes = lanes;
  e->split_for_n = 0;
  return 0;
}

int rpeg_engine_set_split_model(rpeg_engine_t* e, const double* values, int32_t n) {
  if (!e || !values || n != SPLIT_MODEL_FIELDS) { if (e) e->err = "nine figures"; return -1; }
  for (int i = 0; i < n; ++i)
    if (!(values[i] >= 0.0)) { e->err = "the figures are non-negative"; return -1; }
  SplitModel& m = e->split_model;
  m.plan_a = values[0]; m.plan_b = values[1]; m.quad_a = values[2]; m.quad_b = values[3]; m.quad_c = values[4];
  m.eff_beside_quad = values[5]; m.quad_margin = values[6]; m.gain_threshold = values[7]; m.gain_classes = values[8];
  e->split_for_n = 0;
  return 0;
}

int rpeg_engine_set_side_layout(rpeg_engine_t* e, int32_t on) {
  if (!e) return -1;
  e->layout_ahead = on != 0;
  return 0;
}

int rpeg_engine_set_sa_groups(rpeg_engine_t* e, int32_t groups) {
  if (!e) return -1;
  if (groups < 1 || groups > 8) { e->err = "1 to 8 groups of chains"; return -1; }
  e->sa_lanes = groups;
  return 0;
}

int rpeg_engine_set_quad_share(rpeg_engine_t* e, int32_t percent) {
  if (!e) return -1;
  if (percent < 0 || percent > 100) { e->err = "the share is a percentage"; return -1; }
  e->quad_share_pct = (uint32_t)percent;
  e->split_for_n = 0;
  return 0;
}

int rpeg_engine_set_ready_cap(rpeg_engine_t* e, int32_t entries) {
  if (!e) return -1;
  if (entries != 8 && entries != 16 && entries != 24 && entries != 32) {
    e->err = "the ready-list capacity must be 8, 16, 24 or 32";
    return -1;
  }
  e->ready_cap = (uint32_t)entries;
  e->split_for_n = 0;
  return 0;
}

int rpeg_engine_reset_classes(rpeg_engine_t* e) {
  if (!e) return -1;
  hipDeviceSynchronize();
  e->class_off.clear();
  e->cls_sig.clear();
  e->cls_off.clear();
  e->cls_nodes.clear();
  e->cls_slots.clear();
  e->cls_pops16.clear();
  e->cls_split.clear();
  e->split_for_n = 0;
  if (e->d_cstat) { hipFree(e->d_cstat); e->d_cstat = nullptr; e->cstat_cap = 0; }
  e->cls_sorted.clear();
  e->tables_for = 0xFFFFFFFFu;
  e->pool.clear();
  e->d_pool_used = 0;
  return 0;
}

int rpeg_engine_stats(const rpeg_engine_t* e, uint64_t* out, int32_t n) {
  if (!e || !out) return -1;
  for (int i = 0; i < n && i < 8; ++i) out[i] = e->stats[i];
  return 0;
}

int rpeg_eval_batch(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                    double* peak, double* score, uint8_t* mask, void* stream) {
  return eval_batch_impl(e, n, plans, flags, makespan, peak, score, mask, nullptr, stream);
}

int rpeg_eval_batch_mass(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                         double* peak, double* score, uint8_t* mask, double* mass, void* stream) {
  return eval_batch_impl(e, n, plans, flags, makespan, peak, score, mask, mass, stream);
}

int rpeg_eval_host(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                   double* peak, double* score, uint8_t* mask, double* mass, void* stream) {
  return eval_host_impl(e, n, plans, flags, makespan, peak, score, mask, mass, stream);
}

}  // extern "C"

constexpr uint32_t TINY_CLASS = 16;   // classes of fewer plans go to the single-plan kernel


// When a step ends, for a batch of more than one round of wavefronts (microseconds).  The main kernel keeps r
// wavefronts on every compute unit and lasts max(its longest task, its work / (units x r)); k_plan runs beside it in
// the LDS and registers left (16 - 2r wavefronts of 128 registers), and what it has not done by then it does with
// the units to itself, sixteen wavefronts each.  What a plan costs k_plan: SplitModel.
struct DeepModel {
  double n_cu, lds_main, lds_plan;
  double eff = 1.0;   // the part of the modelled room beside the main kernel that k_plan really gets
  uint64_t r_max;
  SplitModel sm;
  double plan_cost(uint32_t plans, uint32_t nodes) const { return (double)plans * (sm.plan_a + sm.plan_b * (double)nodes); }
  double total(double w_main, double w_plan, double max_t, uint64_t r) const {
    const double t_main = std::max(max_t, w_main / (n_cu * (double)r));
    const double room = eff * std::max(0.0, std::min(16.0 - 2.0 * (double)r, std::floor((160.0 * 1024 - (double)r * lds_main) / lds_plan)));
    const double left = std::max(0.0, w_plan - t_main * n_cu * room);
    return t_main + left / (n_cu * 16.0);
  }
  double best(double w_main, double w_plan, double max_t, uint64_t* r_best) const {
    double b = 0.0;
    for (uint64_t r = r_max; r >= 1; --r) {
      const double t = total(w_main, w_plan, max_t, r);
      if (r == r_max || t < b) { b = t; if (r_best) *r_best = r; }
    }
    return b;
  }
};
static DeepModel deep_model(const rpeg_engine_t* e, uint32_t rcap) {
  DeepModel m;
  m.sm = e->split_model;
  m.n_cu = (double)e->n_cu;
  m.lds_main = (double)ke_lds_bytes((e->max_cls_bytes + 15u) & ~15u, rcap, 0, e->max_nodes, e->max_slots, e->max_v);
  m.lds_plan = (double)kp_lds_bytes(e->max_nodes, e->max_slots);
  m.r_max = std::max<uint64_t>(1, std::min<uint64_t>(8, (uint64_t)(160.0 * 1024 / m.lds_main)));
  return m;
}

// The two streams on which k_plan and k_quad run beside the main kernel, one pair per device for all engines of the
// process (never destroyed).  A process has few hardware queues (four by default): with a pair of side streams per
// engine, two engines that evaluate at the same time on two caller streams are six streams, several of which share
// a queue and then wait for each other's kernels; with one pair they are four.
static int side_streams(rpeg_engine_t* e, hipStream_t* plan_stream, hipStream_t* quad_stream) {
  static std::mutex mu;
  static hipStream_t pair[64][2] = {};
  int dev = 0;
  HIP_TRY(e, hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) { e->err = "device index out of range"; return -2; }
  std::lock_guard<std::mutex> lock(mu);
  for (int k = 0; k < 2; ++k)
    if (!pair[dev][k]) HIP_TRY(e, hipStreamCreateWithFlags(&pair[dev][k], hipStreamNonBlocking));
  if (plan_stream) *plan_stream = pair[dev][0];
  if (quad_stream) *quad_stream = pair[dev][1];
  return 0;
}

// The engine's handles on the two side streams and the events of its forks and joins.
static int ensure_side(rpeg_engine_t* e) {
  if (!e->s2) {
    if (int rc = side_streams(e, &e->s2, nullptr)) return rc;
    HIP_TRY(e, hipEventCreateWithFlags(&e->ev_fork, hipEventDisableTiming));
    HIP_TRY(e, hipEventCreateWithFlags(&e->ev_join, hipEventDisableTiming));
  }
  if (!e->s3) {
    if (int rc = side_streams(e, nullptr, &e->s3)) return rc;
    HIP_TRY(e, hipEventCreateWithFlags(&e->ev_join3, hipEventDisableTiming));
    HIP_TRY(e, hipEventCreateWithFlags(&e->ev_sig, hipEventDisableTiming));
    HIP_TRY(e, hipGetDevice(&e->side_dev));
  }
  return 0;
}

// Whether the side streams of the device are this engine's to plan with: it was the last engine that used them (what
// they still hold is then its own earlier call, which the caller's stream follows anyway), or they are idle.  When
// another engine of the process is in the middle of a call on them, work put there would wait for that call's kernels.
static bool side_claim(rpeg_engine_t* e) {
  static std::mutex mu;
  static const void* owner[64] = {};
  std::lock_guard<std::mutex> lock(mu);
  const void* last = owner[e->side_dev];
  owner[e->side_dev] = e;
  if (last == e || last == nullptr) return true;
  return hipStreamQuery(e->s2) == hipSuccess && hipStreamQuery(e->s3) == hipSuccess;
}

static int eval_batch_impl(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                           double* peak, double* score, uint8_t* mask, double* mass, void* stream) {
  if (!e || !plans) return -1;
  e->err.clear();
  e->last_ms = -1.0;
  if (n == 0) return 0;
  if (n >= (1ull << 32)) { e->err = "at most 2^32-1 plans per call"; return -1; }
  if (!plans->vert || !plans->head || plans->stride < n) { e->err = "bad plan tensors"; return -1; }
  hipStream_t s = (hipStream_t)stream;
  if (int rc = ensure_batch(e, n)) return rc;
  const unsigned blk = 256;
  const unsigned nblk = (unsigned)((n + blk - 1) / blk);
  // A batch that gets one wavefront per plan whatever its classes are needs no layout: every plan finds the pool
  // offset of its class through the table of the classes lowered so far, k_plan takes the plans in their own order,
  // and the host only learns afterwards whether a plan belonged to a class not lowered yet (then the call goes the
  // long way below and evaluates the batch again).  Two launches and one wait instead of a round trip between them.
  // Only for an engine of few classes or a batch that is resident at once with room to spare: with hundreds of
  // classes the plans in their own order make neighbouring wavefronts work on different classes, and k_plan ran
  // half as long again as on the sorted batch (config 2 with 8,192 plans: 0.28 against 0.19 ms; with 2,048 plans
  // 0.17 against 0.16 ms and the step 0.21 against 0.23 ms; config 4, 16 classes, 8,192 plans: the step 0.15 against
  // 0.18 ms).
  if ((e->state_lanes == 1 || (e->state_lanes == -1 && n <= (uint64_t)e->n_cu * e->one_plan_waves_per_cu)) && !e->prof_on &&
      !e->cls_sig.empty() && (e->cls_sig.size() <= DIRECT_MAX_CLASSES || n <= (uint64_t)e->n_cu * DIRECT_WAVES_PER_CU) && e->d_hkey && e->tables_for == (uint32_t)e->cls_sig.size() && e->d_pool &&
      e->d_pool_used == e->pool.size() && e->max_nodes <= (uint32_t)(WAVE * KP_MAX_NS) &&
      kp_lds_bytes(e->max_nodes, e->max_slots) <= 64 * 1024) {
    if (int rc = ensure_perm(e, 0, n)) return rc;
    uint32_t* const d_unknown = e->d_queues + (N_QUEUES - 1);
    hipLaunchKernelGGL(k_fill_u32, dim3(1), dim3(64), 0, s, d_unknown, (uint64_t)1, 0u);
    hipLaunchKernelGGL(k_class_direct, dim3((unsigned)((n + SIG_BLOCK - 1) / SIG_BLOCK)), dim3(SIG_BLOCK), 0, s, e->dP, n,
                       plans->vert, plans->head, plans->stride, makespan, peak, score, mask, mass, e->d_hkey, e->d_hoff,
                       e->hcap - 1, e->d_cls, d_unknown);
    HIP_TRY(e, hipGetLastError());
    EvalLaunch L;
    L.P = e->dP; L.vert = plans->vert; L.head = plans->head; L.stride = plans->stride;
    L.perm = nullptr; L.wave_cls = e->d_cls; L.pool = e->d_pool; L.ws = nullptr;
    L.n_waves = n; L.ws_nodes = e->max_nodes; L.ws_slots = e->max_slots;
    L.cls_bytes = 0; L.rcap = 0; L.max_v = e->max_v; L.ovf = nullptr; L.need = nullptr;
    L.flags = flags; L.makespan = makespan; L.peak = peak; L.score = score; L.mask = mask;
    L.mass = mass; L.prof = nullptr;
    const size_t lds = kp_lds_bytes(e->max_nodes, e->max_slots);
    if (e->timing) HIP_TRY(e, hipEventRecord(e->ev0, s));
    hipLaunchKernelGGL(k_plan, dim3((unsigned)std::min<uint64_t>(n, (uint64_t)e->n_cu * 32)), dim3(WAVE), lds, s, L);
    HIP_TRY(e, hipGetLastError());
    if (e->timing) HIP_TRY(e, hipEventRecord(e->ev1, s));
    HIP_TRY(e, hipMemcpyAsync(e->h_ccount, d_unknown, 4, hipMemcpyDeviceToHost, s));
    HIP_TRY(e, hipStreamSynchronize(s));
    if (e->h_ccount[0] == 0u) {
      e->stats[0] = e->cls_sig.size();   // (the classes the engine knows: which of them the batch holds was not counted)
      e->stats[1] = 0; e->stats[2] = n; e->stats[3] = lds; e->stats[4] = 0; e->stats[5] = 1; e->stats[6] = 0;
      e->stats[7] = 0;
      ++e->batch_calls;
      if (e->timing) {
        float ms = 0.f;
        HIP_TRY(e, hipEventElapsedTime(&ms, e->ev0, e->ev1));
        e->last_ms = ms;
      }
      return 0;
    }
  }
  // A batch small enough to get a wavefront per plan whatever its classes are (k_plan) leaves the cost model and the
  // memory model to that kernel, which spreads them over the lanes of a plan's wavefront: the prologue launches work a
  // plan per lane, and a few thousand plans are a few dozen wavefronts that take as long as a full grid would.
  const bool own_prologue = e->state_lanes == 1 || (e->state_lanes == -1 && n <= (uint64_t)e->n_cu * e->one_plan_waves_per_cu);
  bool prologue_done = false, peaks_deferred = false;
  // ahead: k_quad's stream becomes the main line of the call -- the cost-model launch goes there as soon as the class
  // ids are written (beside the hand-over of the counters to the host), the layout and the scatter follow it there
  // as soon as the host has them, and the main kernel follows those in order; the caller's stream carries k_quad
  // and joins at the end.  Only when no other engine of the process is using the side streams.
  bool ahead = false;
  // (whatever way the call ends, the caller's stream follows what went to k_quad's stream)
  struct AheadJoin {
    rpeg_engine_t* e; hipStream_t s; bool* ahead; bool joined = false;
    ~AheadJoin() {
      if (*ahead && !joined && e->s3 && e->ev_join3 && hipEventRecord(e->ev_join3, e->s3) == hipSuccess) hipStreamWaitEvent(s, e->ev_join3, 0);
    }
  } ahead_join{e, s, &ahead};
  PrologueLaunch G;
  // defer: only the cost-model launch now; the memory-model launch (k_peaks) goes out beside the scheduling kernels,
  // which need nothing of it, and k_finish applies its verdicts when all of them are done
  auto launch_prologue = [&](bool defer) -> int {
    G.P = e->dP; G.vert = plans->vert; G.head = plans->head; G.stride = plans->stride; G.n = n; G.cid = e->d_cid;
    G.uni = e->d_uni;
    for (int q = 0; q < RPEG_MAX_STRUCT; ++q) G.n_uni[q] = e->n_uni[q];
    G.max_uni = e->max_uni;
    G.max_v = e->max_v;
    G.dur = e->d_dur; G.dur_stride = e->cap_n;
    G.aux_ovl = e->d_aux_ovl; G.aux_eq = e->d_aux_eq; G.aux_dpne = e->d_aux_dpne; G.vm = e->d_vm;
    G.aux_pen = e->d_aux_pen; G.aux_mask = e->d_aux_mask;
    G.peak = peak;
    const unsigned pblk = (unsigned)((n + WAVE - 1) / WAVE);
    hipLaunchKernelGGL(k_prologue, dim3(pblk, KPRO_PARTS), dim3(WAVE), 0, ahead ? e->s3 : s, G);
    if (!defer) hipLaunchKernelGGL(k_peaks, dim3(pblk), dim3(WAVE), kpeaks_lds_bytes(e->max_v), s, G);
    HIP_TRY(e, hipGetLastError());
    prologue_done = true;
    peaks_deferred = defer;
    return 0;
  };
  const auto t_call = std::chrono::steady_clock::now();
  auto t_counts = t_call, t_waited = t_call;
  // classes of the batch: every plan looks its class id up on the device and counts itself; only the
  // per-class counts come back.  Plans of classes not lowered yet make the call take the slow round:
  // their signatures are read back, the classes are lowered on the host, the tables are rebuilt.
  uint64_t n_new = 0;
  uint32_t ncls = 0, shards = 1;
  for (int round = 0;; ++round) {
    if (int rc = ensure_class_tables(e, s)) return rc;
    ncls = (uint32_t)e->cls_sig.size();
    // (a counter that every block adds to takes the blocks one after the other, ~0.1 us each: no more than about
    // sixteen blocks per counter, and no more counters than that asks for -- all of them are cleared and summed)
    shards = MAX_SHARDS;
    while (shards > 1 && ((uint64_t)ncls * shards > COUNT_SLOTS || (uint64_t)shards * 8 * SIG_BLOCK >= n)) shards >>= 1;
    const uint64_t n_count = (uint64_t)ncls * shards + 1;
    // what earlier launches of the main kernel learned about the classes (pops per dispatch): read in the calls
    // that follow new classes, and now and then afterwards
    const bool read_stat = round == 0 && e->quad_share_pct && ncls && (e->learn_calls > 0 || (e->batch_calls & 63) == 0);
    // The counters go to the host through k_hand_counts; in the first round the host polls its flag instead of waiting
    // for the stream, unless a copy of the statistic has to be waited for anyway.
    const bool handed = round == 0 && !read_stat;
    const uint32_t tag = ++e->sig_tag ? e->sig_tag : ++e->sig_tag;
    if (round == 0 && !own_prologue) {
      if (int rc = ensure_side(e)) return rc;
      ahead = !e->prof_on && e->layout_ahead && side_claim(e);
    }
    if (round > 0 && ahead) HIP_TRY(e, hipStreamSynchronize(e->s3));   // (the cost-model launch reads the class ids)
    // (clear already where the launch that ended the engine's last call did it)
    if (e->count_clean < n_count || e->count_clean_on != s)
      hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)((n_count + blk - 1) / blk)), dim3(blk), 0, s, e->d_ccount, n_count, 0u);
    e->count_clean = 0;
    hipLaunchKernelGGL(k_signature, dim3((unsigned)((n + SIG_BLOCK - 1) / SIG_BLOCK)), dim3(SIG_BLOCK), 0, s, e->dP, n, plans->vert, plans->head, plans->stride,
                       e->d_sig, makespan, peak, score, mask, mass, e->d_hkey, e->d_hval, e->hcap - 1, e->d_cid,
                       e->d_kidx, e->d_ccount, ncls, shards);
    HIP_TRY(e, hipGetLastError());
    // Cost model, memory model and gates of every plan: they need the verdict of the gate (which plans to skip) and
    // nothing of the classes, so they run behind the signature kernel while the host waits for the counts (their
    // flag, not the stream) and lays the batch out.  On k_quad's stream the launch goes out first: it does not wait for
    // the hand-over of the counts, and the hand-over has a few microseconds to spare.
    if (round == 0 && ahead) {
      HIP_TRY(e, hipEventRecord(e->ev_sig, s));
      HIP_TRY(e, hipStreamWaitEvent(e->s3, e->ev_sig, 0));
      if (int rc = launch_prologue(true)) return rc;
    }
    hipLaunchKernelGGL(k_hand_counts, dim3(1), dim3(HAND_BLOCK), 0, s, e->d_ccount, e->d_need, ncls, shards, e->h_tot_dev, e->h_sigflag_dev, tag);
    HIP_TRY(e, hipGetLastError());
    if (read_stat) HIP_TRY(e, hipMemcpyAsync(e->cls_pops16.data(), e->d_cstat, (size_t)ncls * 4, hipMemcpyDeviceToHost, s));
    if (round == 0) {
      if (!handed) {   // (the copy of the statistic has to be waited for: an event, so that the wait leaves the launch below alone)
        if (!e->ev_counts) HIP_TRY(e, hipEventCreateWithFlags(&e->ev_counts, hipEventDisableTiming));
        HIP_TRY(e, hipEventRecord(e->ev_counts, s));
      }
      if (!own_prologue && !ahead)
        if (int rc = launch_prologue(true)) return rc;
      t_counts = std::chrono::steady_clock::now();
      bool seen = false;
      if (handed) {
        for (uint64_t spins = 0;; ++spins) {
          if (__atomic_load_n(e->h_sigflag, __ATOMIC_ACQUIRE) == tag) { seen = true; break; }
          // a launch that does not come to an end is the stream's to report
          if ((spins & 0xFFFFu) == 0xFFFFu && std::chrono::steady_clock::now() - t_counts > std::chrono::seconds(2)) break;
#if defined(__x86_64__) || defined(__i386__)
          __builtin_ia32_pause();
#endif
        }
      }
      if (!seen) {
        if (handed) HIP_TRY(e, hipStreamSynchronize(s));
        else HIP_TRY(e, hipEventSynchronize(e->ev_counts));
      }
      t_waited = std::chrono::steady_clock::now();
    } else {
      HIP_TRY(e, hipStreamSynchronize(s));
    }
    if (read_stat && e->learn_calls > 0) --e->learn_calls;
    for (int q = 0; q < KE_NEED_SHARDS; ++q) e->need = std::max(e->need, e->h_tot[ncls + 1 + q]);
    if (e->h_tot[ncls] == 0) break;
    if (round >= 2) { e->err = "class table did not converge"; return -5; }
    HIP_TRY(e, hipMemcpyAsync(e->h_sig, e->d_sig, n * 8, hipMemcpyDeviceToHost, s));
    HIP_TRY(e, hipStreamSynchronize(s));
    std::vector<uint64_t> sigs;
    uint64_t last_sig = SIG_INVALID;
    for (uint64_t i = 0; i < n; ++i) {
      const uint64_t sg = e->h_sig[i];
      if (sg == SIG_INVALID || sg == last_sig) continue;
      last_sig = sg;
      sigs.push_back(sg);
    }
    if (int rc = lower_new_classes(e, sigs, &n_new)) return rc;
  }
  ++e->batch_calls;
  std::vector<uint32_t> offs, counts, cids;   // the classes present in this batch
  for (uint32_t c = 0; c < ncls; ++c) {
    const uint32_t total = e->h_tot[c];
    if (total) { cids.push_back(c); offs.push_back(e->cls_off[c]); counts.push_back(total); }
  }
  // Plans per wavefront and where their scheduler state lives.  A full batch keeps 64 plans per wavefront
  // with the state in the HBM workspace; a batch too small to fill the chip that way is spread over more
  // wavefronts of fewer plans whose state fits in LDS, which shortens every scheduler step.
  int ls = e->state_lanes;
  bool one = false;   // one plan per wavefront (k_plan)
  const bool quad_all = ls == 4;   // every class in the four-lanes-per-plan kernel (k_quad)
  if (quad_all) {
    ls = 0;
    if (kq_lds_bytes((e->max_cls_bytes + 15u) & ~15u, e->max_nodes, e->max_slots, e->max_v, (uint32_t)KQ_PLANS, mass != nullptr) > 160 * 1024) {
      e->err = "per-plan state of this problem does not fit in LDS with sixteen plans per wavefront";
      return -8;
    }
  }
  {
    auto waves_for = [&](uint32_t per) { uint64_t t = 0; for (uint32_t c : counts) t += (c + per - 1) / per; return t; };
    auto fits = [&](int l) {
      return ke_lds_bytes((e->max_cls_bytes + 15u) & ~15u, 32, (uint32_t)l, e->max_nodes, e->max_slots, e->max_v) <= 160 * 1024;
    };
    const bool one_fits = e->max_nodes <= (uint32_t)(WAVE * KP_MAX_NS) && kp_lds_bytes(e->max_nodes, e->max_slots) <= 64 * 1024;
    if (ls < 0) {
      ls = 0;
      if (one_fits && waves_for(1) <= (uint64_t)e->n_cu * e->one_plan_waves_per_cu) {
        one = true;   // the batch does not fill the chip with a plan per lane: spread every plan over a wavefront
      } else if (waves_for(WAVE) < (uint64_t)e->n_cu * 2) {   // under two wavefronts per compute unit
        for (int l : {8, 16, 32, 64}) {              // fewest plans per wavefront that still gives each its own SIMD
          if (!fits(l)) break;
          ls = l;
          if (waves_for((uint32_t)l) <= (uint64_t)e->n_cu * 4) break;
        }
      }
    } else if (ls == 1) {
      if (!one_fits) { e->err = "a class of this problem has too many nodes for one plan per wavefront"; return -8; }
      one = true;
      ls = 0;
    } else if (ls > 0 && !fits(ls)) {
      e->err = "per-plan state of this problem does not fit in LDS with that many plans per wavefront";
      return -8;
    }
  }
  const uint32_t lpw = one ? 1u : ls ? (uint32_t)ls : (uint32_t)WAVE;   // plans per wavefront
  // every class starts on a wavefront boundary; the lanes left over are idle
  // classes with the largest graphs first: their wavefronts run longest and should not start last
  // (the order of all known classes is kept from call to call and only filtered here: a batch of config 3 meets
  // over ten thousand classes, and sorting them in every call took 0.4 ms)
  if (e->cls_sorted.size() != ncls) {
    e->cls_sorted.resize(ncls);
    for (uint32_t c = 0; c < ncls; ++c) e->cls_sorted[c] = c;
    std::stable_sort(e->cls_sorted.begin(), e->cls_sorted.end(), [&](uint32_t a, uint32_t b) { return e->cls_nodes[a] > e->cls_nodes[b]; });
  }
  e->cls_pos.assign(ncls, 0xFFFFFFFFu);
  for (size_t c = 0; c < counts.size(); ++c) e->cls_pos[cids[c]] = (uint32_t)c;
  std::vector<uint32_t> order;
  order.reserve(counts.size());
  for (uint32_t g : e->cls_sorted)
    if (e->cls_pos[g] != 0xFFFFFFFFu) order.push_back(e->cls_pos[g]);
  // first[c]: first wavefront of class c in launch order (first permutation entry for a class of
  // single-plan wavefronts, which follow the others in the permutation and in the task list)
  std::vector<uint32_t> first(counts.size(), 0), clpw(counts.size(), lpw);
  // ready-list capacity of the main kernel: the full list until the longest list of earlier launches is known
  const uint32_t rcap_main = e->need > 0 ? std::min(e->ready_cap, std::max(8u, (e->need + 2 + 7) & ~7u)) : e->ready_cap;
  std::vector<uint8_t> solo(counts.size(), 0), quad(counts.size(), quad_all ? 1 : 0);
  uint32_t quad_nodes = quad_all ? e->max_nodes : 0, quad_slots = quad_all ? e->max_slots : 0;
  // Where every class runs is decided from the class counts and what has been measured (below): on a batch of
  // thousands of classes that is 0.2 ms of host work.  The decision is kept per class for the next fifteen calls on
  // batches of about the same size (a class not seen then goes by the plain size rule), unless new measurements
  // are about to be read.
  const bool keep_split = !ls && !one && !quad_all && e->quad_share_pct && e->split_for_n && e->learn_calls == 0 &&
                          n * 4 >= e->split_for_n * 3 && n * 3 <= e->split_for_n * 4 && e->batch_calls - e->split_at < 16 &&
                          e->split_mass == (mass != nullptr);
  if (keep_split) {
    for (size_t c = 0; c < counts.size(); ++c) {
      const uint8_t a = cids[c] < e->cls_split.size() ? e->cls_split[cids[c]] : (uint8_t)255;
      if (a == 255) solo[c] = counts[c] < TINY_CLASS ? 1 : 0;
      else if (a == 1) solo[c] = 1;
      else if (a == 2) {
        quad[c] = 1;
        quad_nodes = std::max(quad_nodes, e->cls_nodes[cids[c]]);
        quad_slots = std::max(quad_slots, e->cls_slots[cids[c]]);
      }
    }
  } else if (!ls && !one && !quad_all && !order.empty()) {
    // The kernel ends with its slowest wavefront, and a wavefront is as slow as its slowest plan.  The
    // classes with the largest graphs (up to 15 % of the batch: beyond that the single-plan kernel would be
    // the one that ends last) are taken out of it, unless the batch is
    // many rounds of wavefronts deep anyway (then the sum of the work decides, not the slowest): their plans
    // get a wavefront each (k_plan, on a second stream, filling the registers and LDS the main kernel leaves
    // free; graphs of at least six tenths of the largest node count) or, where that kernel does not fit,
    // eight plans per wavefront (at least seven tenths).
    const uint32_t heavy_lpw = (uint32_t)KE_FEW;
    const bool one_fits = e->max_nodes <= (uint32_t)(WAVE * KP_MAX_NS) && kp_lds_bytes(e->max_nodes, e->max_slots) <= 64 * 1024;
    const bool split = e->split_heavy && one_fits;
    // node count from which a class counts as large: the smallest one, not under `floor` percent of the
    // largest, such that the large classes hold at most `share` percent of the batch
    // (eight percent when k_quad takes the dense classes: a plan costs k_plan four times the instructions)
    const uint64_t floor_pct = split ? 60ull : 70ull;
    uint64_t share_pct = split ? 15ull : 25ull;
    {
      uint64_t w64 = 0;
      for (uint32_t c : counts) w64 += (c + WAVE - 1) / WAVE;
      if (split && e->quad_share_pct && w64 <= (uint64_t)e->n_cu * 12) share_pct = 8;
    }
    const uint32_t top = e->cls_nodes[cids[order[0]]];
    uint64_t waves64 = 0;
    for (uint32_t c : counts) waves64 += (c + WAVE - 1) / WAVE;
    uint32_t cut = 0xFFFFFFFFu;   // classes of at least `cut` nodes are large
    uint64_t heavy_plans = 0;
    for (size_t k = 0; k < order.size();) {
      const uint32_t nodes = e->cls_nodes[cids[order[k]]];
      if (100ull * nodes < floor_pct * top) break;
      uint64_t group = 0;
      size_t k2 = k;
      for (; k2 < order.size() && e->cls_nodes[cids[order[k2]]] == nodes; ++k2) group += counts[order[k2]];
      if ((heavy_plans + group) * 100 > (uint64_t)n * share_pct) break;
      heavy_plans += group;
      cut = nodes;
      k = k2;
    }
    if (waves64 <= (uint64_t)e->n_cu * 16 && heavy_lpw >= 1 && heavy_lpw <= WAVE)
      for (size_t c = 0; c < counts.size(); ++c)
        if (e->cls_nodes[cids[c]] >= cut) {
          if (split) solo[c] = 1;
          else clpw[c] = heavy_lpw;
        }
    // A class with a handful of plans would occupy a wavefront of the main kernel with nearly all lanes idle
    // (on the seeded set of config 3, 46 % of the wavefronts carried 4 % of the plans): its plans get a
    // wavefront each as well.  Six wavefronts of the main kernel and sixteen of k_plan fit on a compute unit,
    // and a plan takes k_plan about half as long as a wavefront takes the main kernel: below six plans k_plan
    // is the cheaper place; the two kernels also run side by side (one waits on latencies, the other issues
    // vector instructions), and on config 3 any threshold between 8 and 32 plans gives the same step time.
    if (split)
      for (size_t c = 0; c < counts.size(); ++c)
        if (counts[c] < TINY_CLASS) solo[c] = 1;
    // Where the work decides (more wavefronts of either kernel than are resident at once) and the main kernel has
    // measured its classes, the threshold is chosen for the batch: of 4, 8, 12, 16 and 24 plans the one for which the
    // modelled end of the step (deep_model) is earliest.  A class not measured yet counts with the measured time per
    // node of the batch's other classes.  (Config 1 with 65,536 plans: 21,500 plans in classes of fewer than 16, the
    // main kernel half empty beside them; with 8 the kernels take 1.4 instead of 2.15 ms.  Config 3 keeps 16.)
    // (One pass over the classes: sums by class size below 24 plans, then the five thresholds from them.)
    if (split && e->quad_share_pct) {
      uint32_t best_th = TINY_CLASS;
      const DeepModel dm = deep_model(e, rcap_main);
      constexpr uint32_t TOP = 24;
      double t_sum = 0.0, nodes_sum = 0.0;
      uint64_t main_tasks = 0, solo_plans = 0;
      for (size_t c = 0; c < counts.size(); ++c) {
        const double t = (double)(e->cls_pops16[cids[c]] >> 12);
        if (t > 0.0) { t_sum += t; nodes_sum += (double)e->cls_nodes[cids[c]]; }
        if (solo[c]) solo_plans += counts[c];
        else main_tasks += (counts[c] + WAVE - 1) / WAVE;
      }
      if (t_sum > 0.0 && (main_tasks > (uint64_t)e->n_cu * dm.r_max || solo_plans > (uint64_t)e->n_cu * 32)) {
        const double per_node = t_sum / nodes_sum;
        double plan_by[TOP] = {}, main_by[TOP] = {}, max_by[TOP] = {};   // by class size: cost in k_plan, time in the main kernel
        double w_plan0 = 0.0, w_main0 = 0.0, max0 = 0.0;                  // the classes no threshold moves
        for (size_t c = 0; c < counts.size(); ++c) {
          const uint32_t nodes = e->cls_nodes[cids[c]];
          if (nodes >= cut) { w_plan0 += dm.plan_cost(counts[c], nodes); continue; }
          const double t0 = (double)(e->cls_pops16[cids[c]] >> 12), t = t0 > 0.0 ? t0 : per_node * (double)nodes;
          if (counts[c] >= TOP) {
            w_main0 += (double)((counts[c] + WAVE - 1) / WAVE) * t;
            max0 = std::max(max0, t);
          } else {
            plan_by[counts[c]] += dm.plan_cost(counts[c], nodes);
            main_by[counts[c]] += t;
            max_by[counts[c]] = std::max(max_by[counts[c]], t);
          }
        }
        double best_t = 0.0;
        for (uint32_t th : {TINY_CLASS, 4u, 8u, 12u, TOP}) {
          double w_main = w_main0, w_plan = w_plan0, max_t = max0;
          for (uint32_t k = 0; k < TOP; ++k) {
            if (k < th) w_plan += plan_by[k];
            else { w_main += main_by[k]; max_t = std::max(max_t, max_by[k]); }
          }
          const double t = dm.best(w_main, w_plan, max_t, nullptr);
          if (th == TINY_CLASS) best_t = t;
          else if (t < dm.sm.gain_threshold * best_t) { best_t = t; best_th = th; }
        }
      }
      if (best_th != TINY_CLASS)
        for (size_t c = 0; c < counts.size(); ++c)
          if (e->cls_nodes[cids[c]] < cut) solo[c] = counts[c] < best_th ? 1 : 0;
    }
    // The main kernel ends when its work is done, unless one wavefront alone runs longer than that (in a batch of a
    // single round of wavefronts it always does).  With the measured time of every class (its slowest wavefront on
    // earlier launches; a class not measured yet counts with the measured time per node of the others) the
    // longest classes are taken out, as many of them as make the modelled end of the step (deep_model) earliest.
    if (split && e->quad_share_pct) {
      DeepModel dm = deep_model(e, rcap_main);
      // (where k_quad is going to take its share of a compute unit's wavefront slots and LDS, k_plan gets through
      // about two thirds of what the model gives it beside the main kernel: measured on configs 2 and 5)
      if (waves64 <= (uint64_t)e->n_cu * 12) dm.eff = dm.sm.eff_beside_quad;
      double w_main = 0.0, w_plan = 0.0, t_sum = 0.0, nodes_sum = 0.0;
      std::vector<uint32_t> cand;
      for (uint32_t c = 0; c < counts.size(); ++c) {
        const double t = (double)(e->cls_pops16[cids[c]] >> 12);
        if (t > 0.0) { t_sum += t; nodes_sum += (double)e->cls_nodes[cids[c]]; }
      }
      const double per_node = nodes_sum > 0.0 ? t_sum / nodes_sum : 0.0;
      auto t_of = [&](uint32_t c) {
        const double t = (double)(e->cls_pops16[cids[c]] >> 12);
        return t > 0.0 ? t : per_node * (double)e->cls_nodes[cids[c]];
      };
      for (uint32_t c = 0; c < counts.size(); ++c) {
        if (solo[c]) { w_plan += dm.plan_cost(counts[c], e->cls_nodes[cids[c]]); continue; }
        w_main += (double)((counts[c] + WAVE - 1) / WAVE) * t_of(c);
        cand.push_back(c);
      }
      if (t_sum > 0.0 && !cand.empty()) {
        std::sort(cand.begin(), cand.end(), [&](uint32_t x, uint32_t y) { return t_of(x) > t_of(y); });
        // the modelled end with the k longest classes taken out, for every k: the best k wins (classes of nearly
        // equal time form plateaus, so one class at a time would stop at the first)
        double best_t = dm.best(w_main, w_plan, t_of(cand[0]), nullptr);
        size_t best_k = 0;
        double wm = w_main, wp = w_plan;
        for (size_t k = 0; k < cand.size(); ++k) {
          const uint32_t c = cand[k];
          wm -= (double)((counts[c] + WAVE - 1) / WAVE) * t_of(c);
          wp += dm.plan_cost(counts[c], e->cls_nodes[cids[c]]);
          const double t = dm.best(wm, wp, k + 1 < cand.size() ? t_of(cand[k + 1]) : 0.0, nullptr);
          if (t < dm.sm.gain_classes * best_t) { best_t = t; best_k = k + 1; }
        }
        for (size_t k = 0; k < best_k; ++k) solo[cand[k]] = 1;
      }
    }
    // Of what stays, the wavefronts that end last are those of dense graphs (long ready lists, keys that go stale
    // often).  The main kernel measures itself: per class, the time of its slowest wavefront on earlier launches and
    // the heap pops per dispatch it needed (cls_pops16).  What a wavefront of k_quad takes: SplitModel.  The classes
    // are taken in the order of their measured time while one still ends later by SplitModel::quad_margin
    // in the main kernel than the slowest chosen class ends in k_quad, up to `quad_share_pct`
    // percent of the batch.  Nothing is known before the first launch of a class: it stays in the main kernel then.
    if (split && e->quad_share_pct && waves64 <= (uint64_t)e->n_cu * 12) {
      auto t_main = [&](uint32_t c) { return (double)(e->cls_pops16[cids[c]] >> 12); };
      auto t_quad = [&](uint32_t c) {
        const double nd = e->cls_nodes[cids[c]], p = (e->cls_pops16[cids[c]] & 0xFFFu) / 16.0;
        return e->split_model.quad_a + nd * (e->split_model.quad_b + e->split_model.quad_c * p);
      };
      std::vector<uint32_t> cand;
      for (uint32_t c = 0; c < counts.size(); ++c)
        if (!solo[c] && e->cls_pops16[cids[c]]) cand.push_back(c);
      std::sort(cand.begin(), cand.end(), [&](uint32_t x, uint32_t y) { return t_main(x) > t_main(y); });
      // (k_quad's wavefronts have the LDS that the main kernel's wavefronts and a few of k_plan's leave on a compute
      // unit: beyond one round of them the time of a wavefront counts as many times as there are rounds)
      const size_t lds_main = ke_lds_bytes((e->max_cls_bytes + 15u) & ~15u, rcap_main, 0, e->max_nodes, e->max_slots, e->max_v);
      uint64_t main_tasks = 0;
      for (uint32_t c = 0; c < counts.size(); ++c)
        if (!solo[c]) main_tasks += (counts[c] + WAVE - 1) / WAVE;
      double slowest_quad = 0.0;
      uint64_t taken = 0, tasks = 0;
      for (uint32_t c : cand) {
        const uint32_t nodes = e->cls_nodes[cids[c]], slots = e->cls_slots[cids[c]];
        const size_t qlds = kq_lds_bytes((e->max_cls_bytes + 15u) & ~15u, std::max(quad_nodes, nodes), std::max(quad_slots, slots), e->max_v,
                                         (uint32_t)KQ_PLANS, mass != nullptr);
        if (qlds > 64 * 1024) continue;
        const uint64_t c_tasks = (counts[c] + KQ_PLANS - 1) / KQ_PLANS;
        const uint64_t main_left = main_tasks - std::min<uint64_t>(main_tasks, (counts[c] + WAVE - 1) / WAVE);
        const double lds_left = 144.0 * 1024 - (double)((main_left + e->n_cu - 1) / e->n_cu) * (double)lds_main;
        const double room = (double)e->n_cu * std::max(1.0, std::floor(lds_left / (double)qlds));
        const double tq = std::max(slowest_quad, t_quad(c));
        const double rounds = std::max(1.0, (double)(tasks + c_tasks) / room);
        if (t_main(c) <= e->split_model.quad_margin * tq * rounds) break;   // (a margin: beyond the classes that clearly end later, more wavefronts of k_quad cost more than they save)
        if ((taken + counts[c]) * 100 > (uint64_t)n * e->quad_share_pct) break;
        quad[c] = 1;
        taken += counts[c];
        tasks += c_tasks;
        main_tasks = main_left;
        slowest_quad = tq;
        quad_nodes = std::max(quad_nodes, nodes);
        quad_slots = std::max(quad_slots, slots);
      }
    }
    if (split && e->quad_share_pct) {   // kept for the next calls
      e->cls_split.assign(ncls, (uint8_t)255);
      for (size_t c = 0; c < counts.size(); ++c) e->cls_split[cids[c]] = solo[c] ? 1 : quad[c] ? 2 : 0;
      e->split_for_n = n; e->split_at = e->batch_calls; e->split_mass = mass != nullptr;
      // a class that runs in the main kernel for the first time is measured by this launch: read it in the next call
      // (at most once in eight calls, so that a class whose measurement never arrives cannot keep the read-back on)
      bool unmeasured = false;
      for (size_t c = 0; c < counts.size() && !unmeasured; ++c) unmeasured = !solo[c] && !quad[c] && (e->cls_pops16[cids[c]] >> 12) == 0;
      if (unmeasured && e->learn_calls == 0 && e->batch_calls - e->relearn_at >= 8) { e->learn_calls = 1; e->relearn_at = e->batch_calls; }
    }
  }
  uint32_t n_eval_waves = 0, n_quad_waves = 0, n_solo = 0;
  for (size_t k = 0; k < order.size(); ++k) {
    const uint32_t c = order[k];
    if (solo[c] || quad[c]) continue;
    first[c] = n_eval_waves;
    n_eval_waves += (counts[c] + clpw[c] - 1) / clpw[c];
  }
  for (size_t k = 0; k < order.size(); ++k) {   // the tasks of k_quad follow those of the main kernel
    const uint32_t c = order[k];
    if (!quad[c]) continue;
    clpw[c] = (uint32_t)(uint32_t)KQ_PLANS;
    first[c] = n_eval_waves + n_quad_waves;
    n_quad_waves += (counts[c] + clpw[c] - 1) / clpw[c];
  }
  const uint32_t n_lane_waves = n_eval_waves + n_quad_waves;
  const uint32_t pstride = one ? 1u : (uint32_t)WAVE;
  const uint64_t n_sorted = (uint64_t)n_lane_waves * pstride;   // permutation entries of the main kernel and k_quad
  for (size_t k = 0; k < order.size(); ++k) {
    const uint32_t c = order[k];
    if (!solo[c]) continue;
    first[c] = (uint32_t)n_sorted + n_solo;
    clpw[c] = 1u | (1u << 16);
    n_solo += counts[c];
  }
  e->stats[0] = counts.size();
  e->stats[1] = n_new;
  e->stats[6] = 0;
  if (n_sorted + n_solo == 0) return 0;
  if (int rc = ensure_perm(e, n_sorted + n_solo, (size_t)n_lane_waves + n_solo)) return rc;
  // the per-class tables of the layout: on the device behind the shard offsets (which k_hand_counts left there), from
  // a sixteen-byte boundary on
  const size_t tab0 = ((size_t)ncls * shards + 1 + 3) & ~size_t(3);
  uint32_t* const h_cfirst = e->h_ccount + tab0;
  uint32_t* const h_clpw = h_cfirst + ncls;
  uint32_t* const h_coff = h_clpw + ncls;
  const uint32_t* const d_cfirst = e->d_ccount + tab0;
  const uint32_t* const d_clpw = d_cfirst + ncls;
  const uint32_t* const d_coff = d_clpw + ncls;
  // tasks of one plan get their class from the scatter kernel, not from the host: with one plan per wavefront
  // throughout that is every task of the launch, otherwise the tasks of the classes taken out of the main kernel
  const uint32_t n_host_tasks = one ? 0u : n_lane_waves;
  // their class offsets ride behind the per-class tables when the block has room, else in a copy of their own
  const size_t block_words = tab0 + 3 * (size_t)ncls;
  const bool tasks_in_block = block_words + n_host_tasks <= 4 * (size_t)e->ccap + COUNT_SLOTS;
  uint32_t* const h_tasks = tasks_in_block ? e->h_ccount + block_words : e->h_cls;
  for (size_t c = 0; c < counts.size(); ++c) {
    h_cfirst[cids[c]] = first[c];
    h_clpw[cids[c]] = one ? (1u | (1u << 16)) : clpw[c];
    h_coff[cids[c]] = offs[c];
  }
  // wavefronts of few plans keep their scheduler state in LDS when that needs no more LDS than the ready
  // lists of a full wavefront do
  // Ready-list capacity: the full 32 entries until the longest list of earlier launches is known, then a
  // short list (less LDS, more wavefronts per compute unit); plans that outgrow it are redone below.
  const uint32_t rcap_full = e->ready_cap;
  const bool short_list = !ls && !one && rcap_main < rcap_full;
  const uint32_t rcap = short_list ? rcap_main : rcap_full;
  const bool few_in_lds = !ls && !one &&
      ke_lds_bytes(0, rcap, KE_FEW, e->max_nodes, e->max_slots, e->max_v) <= ke_lds_bytes(0, rcap, 0, e->max_nodes, e->max_slots, e->max_v);
  for (size_t k = 0; k < order.size(); ++k) {
    const uint32_t c = order[k];
    if (solo[c] || one) {
      continue;
    } else {
      // (never for a task of k_quad, whose eight plans of eight lanes each are not that layout)
      const uint32_t flag = !quad[c] && few_in_lds && clpw[c] == (uint32_t)KE_FEW ? KE_CLS_LDS : 0u;
      const uint32_t nw = (counts[c] + clpw[c] - 1) / clpw[c];
      for (uint32_t t = 0; t < nw; ++t) h_tasks[first[c] + t] = offs[c] | flag;
    }
  }
  if (int rc = ensure_pool(e, s)) return rc;
  // (with `ahead`, the layout goes up and the plans are dealt to their tasks on k_quad's stream, right behind the
  // cost-model launch; the host has seen the counts, so all that the upload and the scatter read or overwrite is at
  // rest)
  if (ahead && (one || !prologue_done || !peaks_deferred)) {   // (not the call that was foreseen: back to the caller's stream)
    HIP_TRY(e, hipStreamSynchronize(e->s3));
    ahead = false;
  }
  const hipStream_t sl = ahead ? e->s3 : s;
  const uint64_t n_idle = !one ? n_sorted : 0;   // with one plan per wavefront every entry is written by the scatter
  if (e->h_ccount_dev && (tasks_in_block || !n_host_tasks)) {
    const uint64_t n_quads = (block_words - tab0 + (tasks_in_block ? n_host_tasks : 0u) + 3) / 4;
    const uint64_t threads = std::max<uint64_t>(n_quads, n_idle);
    hipLaunchKernelGGL(k_upload_fill, dim3((unsigned)((threads + blk - 1) / blk)), dim3(blk), 0, sl, (const uint4*)(e->h_ccount_dev + tab0),
                       (uint4*)(e->d_ccount + tab0), n_quads, e->d_perm, n_idle, IDLE_LANE);
  } else {
    HIP_TRY(e, hipMemcpyAsync(e->d_ccount + tab0, e->h_ccount + tab0, (block_words - tab0 + (tasks_in_block ? n_host_tasks : 0u)) * 4, hipMemcpyHostToDevice, sl));
    if (n_host_tasks && !tasks_in_block) HIP_TRY(e, hipMemcpyAsync(e->d_cls, e->h_cls, (size_t)n_host_tasks * 4, hipMemcpyHostToDevice, sl));
    if (n_idle)
      hipLaunchKernelGGL(k_fill_u32, dim3((unsigned)((n_idle + blk - 1) / blk)), dim3(blk), 0, sl, e->d_perm, n_idle, IDLE_LANE);
  }
  const auto t_laid = std::chrono::steady_clock::now();
  hipLaunchKernelGGL(k_scatter, dim3(nblk), dim3(blk), 0, sl, n, e->d_cid, e->d_kidx, d_cfirst, d_clpw, e->d_ccount, shards, e->d_perm, pstride,
                     d_coff, e->d_cls + n_host_tasks, one ? 0u : (uint32_t)n_sorted, e->d_queues, e->d_limit);
  HIP_TRY(e, hipGetLastError());

  const uint64_t n_waves = n_eval_waves;
  // The main kernel with the state in the workspace is launched with as many wavefronts as can be resident (LDS, and
  // two per SIMD by registers), which take the wave tasks from a counter as they become free: the tasks are in the
  // order of their graphs' sizes, so the longest start first and the rest fills in behind them, and the wavefronts
  // keep their place on the chip while k_plan's smaller ones run beside them.
  const bool queued = !ls && !one;
  uint64_t resident_per_cu = 0;
  if (queued) {
    const size_t lds_main = ke_lds_bytes((e->max_cls_bytes + 15u) & ~15u, rcap, 0, e->max_nodes, e->max_slots, e->max_v);
    const uint64_t r_max = std::max<uint64_t>(1, std::min<uint64_t>(8, 160 * 1024 / lds_main));
    resident_per_cu = r_max;
    // More than one round of wavefronts with work for k_plan beside them: the main kernel leaves k_plan room
    // (deep_model: the number of its wavefronts per compute unit for which both kernels are done soonest).
    const DeepModel dm = deep_model(e, rcap);
    double w_main = 0.0, w_plan = 0.0, max_t = 0.0;
    bool known = true;
    for (size_t c = 0; c < counts.size(); ++c) {
      if (solo[c]) w_plan += dm.plan_cost(counts[c], e->cls_nodes[cids[c]]);
      else if (!quad[c]) {
        const double t = (double)(e->cls_pops16[cids[c]] >> 12);
        if (t == 0.0) known = false;
        w_main += (double)((counts[c] + clpw[c] - 1) / clpw[c]) * t;
        max_t = std::max(max_t, t);
      }
    }
    if (known && n_solo && n_waves > (uint64_t)e->n_cu * r_max) dm.best(w_main, w_plan, max_t, &resident_per_cu);
  }
  const unsigned grid = (unsigned)std::min<uint64_t>(std::max<uint64_t>(n_waves, 1), (uint64_t)e->n_cu * (one ? 32 : queued ? resident_per_cu : 16));
  const size_t wsb = ls || one ? 0 : ke_ws_bytes(e->max_nodes, e->max_slots);
  if (!ls && !one && n_waves)
    if (int rc = ensure_ws(e, wsb * grid, s)) return rc;
  EvalLaunch L;
  L.P = e->dP; L.vert = plans->vert; L.head = plans->head; L.stride = plans->stride;
  L.perm = e->d_perm; L.wave_cls = tasks_in_block && !one ? e->d_ccount + block_words : e->d_cls; L.pool = e->d_pool; L.ws = e->d_ws;
  L.n_waves = n_waves; L.ws_nodes = e->max_nodes; L.ws_slots = e->max_slots;
  L.cls_bytes = (e->max_cls_bytes + 15u) & ~15u;
  // ready-list capacity (a multiple of the scan's batch of 8); classes with more than 4095 nodes or
  // tie-break keys above 15 cannot be packed into a ready entry
  if (e->max_nodes > 4095) { e->err = "class with more than 4095 nodes"; return -8; }
  L.rcap = rcap;
  L.max_v = e->max_v;
  // Overflow flags are written only by a launch that a fix-up launch follows (the short list): with the full list
  // an overflow is final (RPEG_MASK_LIMIT), and a flag left standing would be redone by a later call's fix-up.
  L.ovf = short_list ? e->d_ovf : nullptr;
  L.need = !ls && !one ? e->d_need : nullptr;
  L.cstat = !ls && !one && e->quad_share_pct ? e->d_cstat : nullptr;
  L.queue = queued ? e->d_queues : nullptr;
  L.flags = flags; L.makespan = makespan; L.peak = peak; L.score = score; L.mask = mask;
  L.mass = mass;
  L.prof = nullptr;
  if (!prologue_done && !one)   // (the classes lowered in this call changed what was foreseen for the batch)
    if (int rc = launch_prologue(false)) return rc;
  if (prologue_done) {
    L.dur = e->d_dur; L.aux_ovl = e->d_aux_ovl; L.aux_dpne = e->d_aux_dpne;
    if (!peaks_deferred) { L.aux_pen = e->d_aux_pen; L.aux_mask = e->d_aux_mask; }
    L.dur_stride = e->cap_n;
  }
  const bool bounded = !one;   // some kernel of this call holds a bounded ready set
  if (bounded) {
    if (int rc = ensure_limit_ws(e, s)) return rc;
    L.limit = e->d_limit;
  }
  if (e->prof_on) {
    if (e->d_prof) hipFree(e->d_prof);
    HIP_TRY(e, hipMalloc(&e->d_prof, (n_waves + n_quad_waves + n_solo) * 64));
    HIP_TRY(e, hipMemsetAsync(e->d_prof, 0, (n_waves + n_quad_waves + n_solo) * 64, s));
    e->prof_waves = n_waves + n_quad_waves + n_solo;
    L.prof = e->d_prof;
  }
  const size_t lds = one ? kp_lds_bytes(e->max_nodes, e->max_slots)
                   : ke_lds_bytes(L.cls_bytes, L.rcap, (uint32_t)ls, e->max_nodes, e->max_slots, e->max_v);
  if (lds > 160 * 1024) { e->err = "class tables exceed the LDS"; return -8; }
  const void* kfn = ls == 0 ? (const void*)k_eval<0> : ls == 8 ? (const void*)k_eval<8> : ls == 16 ? (const void*)k_eval<16>
                  : ls == 32 ? (const void*)k_eval<32> : (const void*)k_eval<64>;
  const int ki = ls == 0 ? 0 : ls == 8 ? 1 : ls == 16 ? 2 : ls == 32 ? 3 : 4;
  if (!one && lds > 64 * 1024 && !e->lds_attr_set[ki]) {
    HIP_TRY(e, hipFuncSetAttribute(kfn, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    e->lds_attr_set[ki] = true;
  }
  e->stats[2] = n_waves + n_quad_waves + n_solo;
  e->stats[7] = n_quad_waves;
  e->stats[3] = lds;
  e->stats[4] = wsb * grid;
  e->stats[5] = one ? 1u : (uint64_t)ls;
  e->stats[6] = n_solo;
  // The main kernel is submitted first: it needs 26 KB of LDS per wavefront, and once single-plan wavefronts
  // fill a compute unit its wavefronts only fit in as those retire.
  // The memory-model launch, where it was deferred: on k_quad's stream when that kernel has nothing to do in this call
  // (the launch then runs beside all scheduling kernels), else behind the main kernel, where it runs beside the tails
  // of the two other kernels.
  // With the layout ahead on k_quad's stream, that stream and the caller's change places until the join: the main
  // kernel follows the scatter in order (it starts first, as it must: the kernels of the two other streams see the
  // fork event a few microseconds later), and k_quad follows the cost-model launch on the caller's stream.
  const bool peaks_aside = peaks_deferred && !n_quad_waves;
  const hipStream_t sm = ahead ? e->s3 : s;    // the main kernel and what follows it
  hipStream_t sq = ahead ? s : e->s3;          // k_quad, or the memory-model launch in its place
  if (ahead) {
    HIP_TRY(e, hipEventRecord(e->ev_fork, e->s3));   // (cost-model launch, layout and scatter are done)
  } else if (n_solo || n_quad_waves || peaks_aside) {
    if (int rc = ensure_side(e)) return rc;
    sq = e->s3;
    HIP_TRY(e, hipEventRecord(e->ev_fork, s));
    if (e->timing) HIP_TRY(e, hipEventRecord(e->ev0, s));
  } else if (e->timing) {
    HIP_TRY(e, hipEventRecord(e->ev0, s));
  }
  auto launch_quad = [&]() -> int {   // the four-lanes-per-plan wavefronts, beside the main kernel
    if (!n_quad_waves) return 0;
    EvalLaunch Q = L;
    Q.perm = e->d_perm + (uint64_t)n_eval_waves * WAVE;
    Q.wave_cls = L.wave_cls + n_eval_waves;
    Q.n_waves = n_quad_waves;
    Q.ws_nodes = quad_nodes; Q.ws_slots = quad_slots;
    Q.ovf = nullptr; Q.need = nullptr; Q.cstat = nullptr; Q.queue = nullptr;   // (a plan that outgrows the 32 entries is flagged in Q.limit)
    if (L.prof) Q.prof = L.prof + n_waves * 8;
    const size_t qlds = kq_lds_bytes(L.cls_bytes, quad_nodes, quad_slots, e->max_v, (uint32_t)KQ_PLANS, mass != nullptr);
    if (qlds > 64 * 1024 && !e->quad_attr_set) {
      HIP_TRY(e, hipFuncSetAttribute((const void*)k_quad, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
      e->quad_attr_set = true;
    }
    hipLaunchKernelGGL(k_quad, dim3((unsigned)std::min<uint64_t>(n_quad_waves, (uint64_t)e->n_cu * 16)), dim3(WAVE), qlds, sq, Q);
    HIP_TRY(e, hipGetLastError());
    return 0;
  };
  auto launch_main = [&]() {
    if (n_waves == 0) {
    } else if (one) hipLaunchKernelGGL(k_plan, dim3(grid), dim3(WAVE), lds, sm, L);
    else switch (ls) {
      case 0: hipLaunchKernelGGL(k_eval<0>, dim3(grid), dim3(WAVE), lds, sm, L); break;
      case 8: hipLaunchKernelGGL(k_eval<8>, dim3(grid), dim3(WAVE), lds, sm, L); break;
      case 16: hipLaunchKernelGGL(k_eval<16>, dim3(grid), dim3(WAVE), lds, sm, L); break;
      case 32: hipLaunchKernelGGL(k_eval<32>, dim3(grid), dim3(WAVE), lds, sm, L); break;
      default: hipLaunchKernelGGL(k_eval<64>, dim3(grid), dim3(WAVE), lds, sm, L); break;
    }
    return hipGetLastError();
  };
  // (The main kernel first also when k_plan has only a handful of tasks, which then wait until wavefronts of the main
  // kernel retire: with those few in front the step was 30 us longer on config 4.)
  HIP_TRY(e, launch_main());
  // (the three launches back to back: every call between them delays the start of the later kernels)
  const bool side_q = n_quad_waves || peaks_aside;
  if (ahead) {
    HIP_TRY(e, hipStreamWaitEvent(s, e->ev_fork, 0));
    if (e->timing) HIP_TRY(e, hipEventRecord(e->ev0, s));
  } else if (side_q) {
    HIP_TRY(e, hipStreamWaitEvent(e->s3, e->ev_fork, 0));
  }
  // (k_quad second: measured against k_quad first, 0.50 against 0.52-0.53 ms on config 2, and against k_quad last,
  // 0.59 ms; its wavefronts need the most LDS after the main kernel's)
  if (int rc = launch_quad()) return rc;
  if (n_solo) {   // the single-plan wavefronts, beside the main kernel
    HIP_TRY(e, hipStreamWaitEvent(e->s2, e->ev_fork, 0));
    EvalLaunch S = L;
    S.queue = nullptr;
    S.perm = e->d_perm + n_sorted;
    S.wave_cls = e->d_cls + n_host_tasks;
    S.n_waves = n_solo;
    if (L.prof) S.prof = L.prof + (n_waves + n_quad_waves) * 8;
    hipLaunchKernelGGL(k_plan, dim3((unsigned)std::min<uint64_t>(n_solo, (uint64_t)e->n_cu * 32)), dim3(WAVE),
                       kp_lds_bytes(e->max_nodes, e->max_slots), e->s2, S);
    HIP_TRY(e, hipGetLastError());
  }
  if (peaks_deferred) {
    const unsigned pblk = (unsigned)((n + WAVE - 1) / WAVE);
    hipLaunchKernelGGL(k_peaks, dim3(pblk), dim3(WAVE), kpeaks_lds_bytes(e->max_v), peaks_aside ? sq : sm, G);
    HIP_TRY(e, hipGetLastError());
  }
  if (n_solo) HIP_TRY(e, hipEventRecord(e->ev_join, e->s2));
  // (after the submission of k_plan, which is the longer of the two kernels and should not wait for this one)
  if (short_list && n_waves) {   // the plans whose ready list outgrew the short one, with the full one
    EvalLaunch F = L;
    F.queue = nullptr;
    F.rcap = rcap_full;
    F.flags = flags | KE_FIXUP;
    const size_t lds_full = ke_lds_bytes(F.cls_bytes, F.rcap, 0, e->max_nodes, e->max_slots, e->max_v);
    if (lds_full > 160 * 1024) { e->err = "class tables exceed the LDS"; return -8; }
    if (lds_full > 64 * 1024 && !e->lds_attr_set[0]) {
      HIP_TRY(e, hipFuncSetAttribute((const void*)k_eval<0>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
      e->lds_attr_set[0] = true;
    }
    // a small grid: the launch almost always finds the count of flagged plans at zero and ends at once
    hipLaunchKernelGGL(k_eval<0>, dim3(std::min<unsigned>(grid, (unsigned)e->n_cu * 2u)), dim3(WAVE), lds_full, sm, F);
    HIP_TRY(e, hipGetLastError());
  }
  if (ahead || side_q) {   // whatever ran on k_quad's stream
    HIP_TRY(e, hipEventRecord(e->ev_join3, e->s3));
    HIP_TRY(e, hipStreamWaitEvent(s, e->ev_join3, 0));
    ahead_join.joined = true;
  }
  if (n_solo) HIP_TRY(e, hipStreamWaitEvent(s, e->ev_join, 0));
  if (peaks_deferred) {   // (before k_eval_limit, whose plans get their final outputs from that kernel itself)
    // (the layout tables in the counters' buffer have been read by now: the counters of the next call are cleared here)
    const uint32_t zero_n = (uint32_t)std::min<size_t>(std::max<size_t>((size_t)COUNT_SLOTS, ncls) + 1, 4 * (size_t)e->ccap + COUNT_SLOTS);
    hipLaunchKernelGGL(k_finish, dim3(nblk), dim3(blk), 0, s, n, e->d_cid, e->d_aux_pen, e->d_aux_mask, flags, score, mask, e->d_ccount, zero_n);
    HIP_TRY(e, hipGetLastError());
    e->count_clean = zero_n;
    e->count_clean_on = s;
  }
  if (bounded) {   // the plans flagged by the kernels above, without a bound on the ready set (ends at once when there is none)
    EvalLaunch U = L;
    U.queue = nullptr;
    hipLaunchKernelGGL(k_eval_limit, dim3(e->limit_grid), dim3(WAVE), 0, s, U, e->d_limit_ws);
    HIP_TRY(e, hipGetLastError());
  }
  {
    const auto t_end = std::chrono::steady_clock::now();
    auto us = [](std::chrono::steady_clock::time_point a, std::chrono::steady_clock::time_point b) {
      return std::chrono::duration<double, std::micro>(b - a).count();
    };
    e->host_us[0] = us(t_call, t_counts);    // gate and signature launch, copies of the counts, prologue launch
    e->host_us[1] = us(t_counts, t_waited);  // the wait for the counts
    e->host_us[2] = us(t_waited, t_laid);    // layout of the batch and the split between the kernels, tables up
    e->host_us[3] = us(t_laid, t_end);       // scatter, fork, the scheduling launches, join, the launches that end the call
  }
  if (e->timing) {
    HIP_TRY(e, hipEventRecord(e->ev1, s));
    HIP_TRY(e, hipEventSynchronize(e->ev1));
    float ms = 0.f;
    HIP_TRY(e, hipEventElapsedTime(&ms, e->ev0, e->ev1));
    e->last_ms = ms;
  }
  return 0;
}

extern "C" {

int rpeg_engine_host_us(const rpeg_engine_t* e, double* out, int32_t n) {
  if (!e || !out) return -1;
  for (int i = 0; i < n && i < 4; ++i) out[i] = e->host_us[i];
  return 0;
}

// rpeg_eval_batch for callers that cannot allocate: every intermediate of the call lives in the file-scope
// scratch array of this device, and the call makes no hipMalloc / hipFree.  One plan per wavefront (k_plan).
int rpeg_eval_batch_static(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                           double* peak, double* score, uint8_t* mask, void* stream) {
  if (!e || !plans) return -1;
  e->err.clear();
  e->last_ms = -1.0;
  if (n == 0) return 0;
  if (n > (uint64_t)RPEG_STATIC_MAX_PLANS) {
    e->err = "rpeg_eval_batch_static takes at most " + std::to_string(RPEG_STATIC_MAX_PLANS) + " plans per call, got " +
             std::to_string(n);
    return -9;
  }
  if (!plans->vert || !plans->head || plans->stride < n) { e->err = "bad plan tensors"; return -1; }
  if (!e->d_hkey || e->tables_for != (uint32_t)e->cls_sig.size() || e->d_pool_used != e->pool.size() || !e->d_pool) {
    e->err = "the engine's class tables are not on the device: evaluate a batch with these classes through rpeg_eval_batch first";
    return -10;
  }
  if (e->max_nodes > (uint32_t)(WAVE * KP_MAX_NS) || kp_lds_bytes(e->max_nodes, e->max_slots) > 64 * 1024) {
    e->err = "a class of this problem has too many nodes for one plan per wavefront";
    return -8;
  }
  hipStream_t s = (hipStream_t)stream;
  uint32_t* const d_cls = (uint32_t*)e->static_ptr;
  uint32_t* const d_counters = (uint32_t*)(e->static_ptr + STATIC_CLS_BYTES);
  // the array keeps what the last call left: the counters start at zero (a fill kernel, not a memset node: a caller
  // may capture these launches into a HIP graph), the task list is rewritten for all n plans
  hipLaunchKernelGGL(k_fill_u32, dim3(1), dim3(64), 0, s, d_counters, (uint64_t)(STATIC_COUNTER_BYTES / 4), 0u);
  hipLaunchKernelGGL(k_class_direct, dim3((unsigned)((n + SIG_BLOCK - 1) / SIG_BLOCK)), dim3(SIG_BLOCK), 0, s, e->dP, n,
                     plans->vert, plans->head, plans->stride, makespan, peak, score, mask, (double*)nullptr, e->d_hkey, e->d_hoff,
                     e->hcap - 1, d_cls, d_counters);
  HIP_TRY(e, hipGetLastError());
  EvalLaunch L;
  L.P = e->dP; L.vert = plans->vert; L.head = plans->head; L.stride = plans->stride;
  L.perm = nullptr; L.wave_cls = d_cls; L.pool = e->d_pool; L.ws = nullptr;
  L.n_waves = n; L.ws_nodes = e->max_nodes; L.ws_slots = e->max_slots;
  L.cls_bytes = 0; L.rcap = 0; L.max_v = e->max_v; L.ovf = nullptr; L.need = nullptr;
  L.flags = flags & RPEG_GATE_STALE; L.makespan = makespan; L.peak = peak; L.score = score; L.mask = mask;
  L.mass = nullptr; L.prof = nullptr;
  const size_t lds = kp_lds_bytes(e->max_nodes, e->max_slots);
  hipLaunchKernelGGL(k_plan, dim3((unsigned)std::min<uint64_t>(n, (uint64_t)e->n_cu * 32)), dim3(WAVE), lds, s, L);
  HIP_TRY(e, hipGetLastError());
  e->stats[0] = 0; e->stats[1] = 0; e->stats[2] = n; e->stats[3] = lds; e->stats[4] = 0; e->stats[5] = 1; e->stats[6] = 0;
  e->stats[7] = 0;
  // With RPEG_NO_WAIT the call ends here: three launches on the caller's stream, no copy and no wait (what a
  // capturing stream accepts).  Plans of classes the engine has not met are then told by their mask alone.
  if (flags & RPEG_NO_WAIT) return 0;
  HIP_TRY(e, hipMemcpyAsync(e->h_static, d_counters, 4, hipMemcpyDeviceToHost, s));
  HIP_TRY(e, hipStreamSynchronize(s));
  if (e->h_static[0] != 0u) {
    e->err = std::to_string(e->h_static[0]) + " plans belong to lowering classes the engine has not met: evaluate them through "
             "rpeg_eval_batch once (their outputs are NaN, their mask has RPEG_MASK_ERROR)";
    return -11;
  }
  return 0;
}

int rpeg_op_time_batch(rpeg_engine_t* e, uint64_t n, int32_t structure, int32_t vertex, const int16_t* strat,
                       uint64_t stride, double* time, double* peak, void* stream) {
  if (!e || !strat) return -1;
  e->err.clear();
  if (structure < 0 || structure >= e->P.n_struct || vertex < 0 || vertex >= e->P.st[structure].n_vertex || stride < n) {
    e->err = "bad structure/vertex/stride";
    return -1;
  }
  if (n == 0) return 0;
  const unsigned blk = 256;
  hipLaunchKernelGGL(k_op_time, dim3((unsigned)((n + blk - 1) / blk)), dim3(blk), 0, (hipStream_t)stream, e->dP, n,
                     structure, vertex, strat, stride, time, peak);
  HIP_TRY(e, hipGetLastError());
  return 0;
}

int rpeg_eval_trace(rpeg_engine_t* e, const int16_t* vert_fields, const uint8_t* head4, double* start, double* finish,
                    int32_t* dispatch_index, int32_t* node_kind, int32_t* node_vertex, int32_t* node_step, int32_t* node_sub, int32_t* node_src,
                    int32_t* edges, int32_t* n_edges, int32_t cap, uint8_t* node_reserved) {
  if (!e || !vert_fields || !head4 || !start || !finish) return -1;
  e->err.clear();
  PlanHead h = load_head(head4, 1, 0);
  VPlan a[RPEG_MAX_V];
  std::memset(a, 0, sizeof a);
  if (h.structure >= e->P.n_struct) { e->err = "bad structure"; return -1; }
  for (int v = 0; v < e->P.st[h.structure].n_vertex; ++v) load_vertex(vert_fields, 1, 0, v, &a[v]);
  if (!plan_valid(e->P, h, a)) { e->err = "plan violates the integer validity rules"; return -6; }
  const uint64_t sg = plan_signature(e->P, h.structure, h.split, h.tau0, h.tau1, a);
  LoweredClass lc;
  try { lc = lower_class(e->P, sg); } catch (const std::exception& ex) { e->err = ex.what(); return -5; }
  const int n = (int)lc.nodes.size();
  if (n > cap || (edges && (int)lc.edges.size() > cap)) { e->err = "trace arrays too small"; return -7; }
  int64_t off = class_offset(e, sg, nullptr);
  if (off < 0) return -5;
  hipStream_t s = nullptr;
  // This call works on the null stream and reuses the engine's task, lane and state buffers.  A batched call
  // returns without waiting for its stream, and a stream created as non-blocking does not order itself against
  // the null stream: wait for everything the device still runs before those buffers are written.
  HIP_TRY(e, hipDeviceSynchronize());
  if (int rc = ensure_pool(e, s)) return rc;
  if (int rc = ensure_perm(e, WAVE, 1)) return rc;
  if (int rc = ensure_ws(e, wave_ws_bytes(e->max_nodes, e->max_slots), s)) return rc;
  constexpr size_t IN_BYTES = 256;   // fields (120 B) and header (4 B) of the plan, padded
  if (!e->d_trace || (size_t)n > e->d_trace_nodes) {
    if (e->d_trace) hipFree(e->d_trace);
    e->d_trace = nullptr;
    e->d_trace_nodes = std::max<size_t>(512, (size_t)n * 2);
    HIP_TRY(e, hipMalloc(&e->d_trace, IN_BYTES + e->d_trace_nodes * 20));
  }
  int16_t* d_vert = (int16_t*)e->d_trace;
  uint8_t* d_head = e->d_trace + RPEG_MAX_V * RPEG_FIELDS * 2;
  double* d_tr = (double*)(e->d_trace + IN_BYTES);
  HIP_TRY(e, hipMemcpy(d_vert, vert_fields, RPEG_MAX_V * RPEG_FIELDS * 2, hipMemcpyHostToDevice));
  HIP_TRY(e, hipMemcpy(d_head, head4, 4, hipMemcpyHostToDevice));
  uint32_t lanes[WAVE];
  for (int l = 0; l < WAVE; ++l) lanes[l] = l == 0 ? 0u : IDLE_LANE;
  const uint32_t o32 = (uint32_t)off;
  HIP_TRY(e, hipMemcpy(e->d_perm, lanes, sizeof lanes, hipMemcpyHostToDevice));
  HIP_TRY(e, hipMemcpy(e->d_cls, &o32, 4, hipMemcpyHostToDevice));
  hipLaunchKernelGGL(k_eval_generic, dim3(1), dim3(WAVE), 0, s, e->dP, (uint64_t)WAVE, d_vert, d_head,
                     (uint64_t)1, e->d_perm, e->d_cls, e->d_pool, e->d_ws, e->max_nodes, e->max_slots, 0u,
                     (double*)nullptr, (double*)nullptr, (double*)nullptr, (uint8_t*)nullptr, d_tr, d_tr + n,
                     (int32_t*)(d_tr + 2 * (size_t)n));
  HIP_TRY(e, hipGetLastError());
  HIP_TRY(e, hipMemcpy(start, d_tr, (size_t)n * 8, hipMemcpyDeviceToHost));
  HIP_TRY(e, hipMemcpy(finish, d_tr + n, (size_t)n * 8, hipMemcpyDeviceToHost));
  if (dispatch_index) HIP_TRY(e, hipMemcpy(dispatch_index, d_tr + 2 * (size_t)n, (size_t)n * 4, hipMemcpyDeviceToHost));
  for (int i = 0; i < n; ++i) {
    if (node_kind) node_kind[i] = lc.nodes[i].kind;
    if (node_vertex) node_vertex[i] = lc.nodes[i].kind == 0 ? lc.nodes[i].vertex : lc.nodes[i].a1;
    if (node_step) node_step[i] = lc.nodes[i].step;
    if (node_sub) node_sub[i] = lc.nodes[i].sub;
    if (node_src) node_src[i] = lc.nodes[i].kind == 0 ? lc.nodes[i].vertex : lc.nodes[i].a0;
  }
  if (node_reserved) {   // the vertices whose allocations the scheduler reserves for the node
    const ClassView cv = class_view(e->pool.data() + off);
    const uint64_t dpne = plan_masks(a, e->P.st[h.structure].n_vertex).dpne;
    for (int i = 0; i < n; ++i) node_reserved[i] = (uint8_t)blocked_mask(cv.node[i], dpne);
  }
  if (edges)
    for (size_t j = 0; j < lc.edges.size(); ++j) { edges[2 * j] = lc.edges[j].first; edges[2 * j + 1] = lc.edges[j].second; }
  if (n_edges) *n_edges = (int32_t)lc.edges.size();
  return n;
}

// lower() of ONE plan on the host (integer work only, no engine and no GPU needed): the plan's class signature
// and the class lowering the engine itself uses.
int rpeg_lower_plan(const rpeg_problem_t* problem, const int16_t* vert_fields, const uint8_t* head4, int32_t* node_kind,
                    int32_t* node_vertex, int32_t* node_step, int32_t* node_sub, int32_t* node_src, int64_t* node_payload,
                    int32_t* node_ref, int32_t* edges, int32_t* n_edges, int32_t cap) {
  if (!problem || !vert_fields || !head4) return -1;
  if (problem->abi_version != RPEG_ABI_VERSION) return -3;
  const PlanHead h = load_head(head4, 1, 0);
  if (h.structure < 0 || h.structure >= problem->n_struct || h.split < 0 || h.split >= problem->n_split || h.tau0 > 3 || h.tau1 > 3)
    return -1;
  const rpeg_struct_t& st = problem->st[h.structure];
  VPlan a[RPEG_MAX_V];
  std::memset(a, 0, sizeof a);
  for (int v = 0; v < st.n_vertex; ++v) load_vertex(vert_fields, 1, 0, v, &a[v]);
  const uint64_t sg = plan_signature(*problem, h.structure, h.split, h.tau0, h.tau1, a);
  LoweredClass lc;
  try { lc = lower_class(*problem, sg); } catch (const std::exception&) { return -5; }
  const int n = (int)lc.nodes.size();
  if (n > cap || (edges && (int)lc.edges.size() > cap)) return -7;
  const ClassView cv = class_view(lc.blob.data());
  for (int i = 0; i < n; ++i) {
    const LoweredNode& nd = lc.nodes[i];
    const SlotDesc sd = cv.slot[nd.slot];
    if (node_kind) node_kind[i] = nd.kind;
    if (node_vertex) node_vertex[i] = nd.kind == 0 ? nd.vertex : nd.a1;
    if (node_step) node_step[i] = nd.step;
    if (node_sub) node_sub[i] = nd.sub;
    if (node_src) node_src[i] = nd.kind == 0 ? nd.vertex : nd.a0;
    int64_t payload = 0;
    int32_t ref = -1;
    if (sd.type == SLOT_COMM_DATA) {
      payload = sd.q == 0xFF ? st.edge[sd.a].full_bytes : st.edge[sd.a].sub_bytes[h.split][sd.q];
      ref = sd.a;
    } else if (sd.type == SLOT_COMM_PUB) {
      const rpeg_pub_t& pb = st.pub[sd.a];
      payload = pub_payload(*problem, a[pb.src], a[pb.dst], pb.model);
      ref = 16 + pb.model;
    } else if (sd.type == SLOT_RESHARD) {
      payload = problem->model[sd.b].n_params * problem->model[sd.b].sb;
      ref = 16 + sd.b;
    }
    if (node_payload) node_payload[i] = payload;
    if (node_ref) node_ref[i] = ref;
  }
  if (edges)
    for (size_t j = 0; j < lc.edges.size(); ++j) { edges[2 * j] = lc.edges[j].first; edges[2 * j + 1] = lc.edges[j].second; }
  if (n_edges) *n_edges = (int32_t)lc.edges.size();
  return n;
}

int rpeg_plan_detail(rpeg_engine_t* e, const int16_t* vert_fields, const uint8_t* head4, double* node_time,
                     int64_t* node_payload, int32_t* node_ref, int32_t cap, double* set_peak) {
  if (!e || !vert_fields || !head4) return -1;
  e->err.clear();
  PlanHead h = load_head(head4, 1, 0);
  VPlan a[RPEG_MAX_V];
  std::memset(a, 0, sizeof a);
  if (h.structure >= e->P.n_struct) { e->err = "bad structure"; return -1; }
  const rpeg_struct_t& st = e->P.st[h.structure];
  for (int v = 0; v < st.n_vertex; ++v) load_vertex(vert_fields, 1, 0, v, &a[v]);
  if (!plan_valid(e->P, h, a)) { e->err = "plan violates the integer validity rules"; return -6; }
  const uint64_t sg = plan_signature(e->P, h.structure, h.split, h.tau0, h.tau1, a);
  LoweredClass lc;
  try { lc = lower_class(e->P, sg); } catch (const std::exception& ex) { e->err = ex.what(); return -5; }
  const int n = (int)lc.nodes.size();
  if ((node_time || node_payload || node_ref) && n > cap) { e->err = "node arrays too small"; return -7; }
  const int64_t off = class_offset(e, sg, nullptr);
  if (off < 0) return -5;
  hipStream_t s = nullptr;
  HIP_TRY(e, hipDeviceSynchronize());   // (null stream, shared buffers: as rpeg_eval_trace)
  if (int rc = ensure_pool(e, s)) return rc;
  constexpr size_t IN_BYTES = 256, SLOTS = 256;
  if (!e->d_detail) HIP_TRY(e, hipMalloc(&e->d_detail, IN_BYTES + (SLOTS + WAVE) * 8));
  int16_t* d_vert = (int16_t*)e->d_detail;
  uint8_t* d_head = e->d_detail + RPEG_MAX_V * RPEG_FIELDS * 2;
  double* d_out = (double*)(e->d_detail + IN_BYTES);
  HIP_TRY(e, hipMemcpy(d_vert, vert_fields, RPEG_MAX_V * RPEG_FIELDS * 2, hipMemcpyHostToDevice));
  HIP_TRY(e, hipMemcpy(d_head, head4, 4, hipMemcpyHostToDevice));
  hipLaunchKernelGGL(k_plan_detail, dim3(1), dim3(WAVE), 0, s, e->dP, d_vert, d_head, e->d_pool + off, d_out, d_out + SLOTS);
  HIP_TRY(e, hipGetLastError());
  double out[SLOTS + WAVE];
  HIP_TRY(e, hipMemcpy(out, d_out, sizeof out, hipMemcpyDeviceToHost));
  const ClassView cv = class_view(e->pool.data() + off);
  for (int i = 0; i < n; ++i) {
    const LoweredNode& nd = lc.nodes[i];
    const SlotDesc sd = cv.slot[nd.slot];
    if (node_time) node_time[i] = out[nd.slot];
    int64_t payload = 0;
    int32_t ref = -1;
    if (sd.type == SLOT_COMM_DATA) {
      payload = sd.q == 0xFF ? st.edge[sd.a].full_bytes : st.edge[sd.a].sub_bytes[h.split][sd.q];
      ref = sd.a;
    } else if (sd.type == SLOT_COMM_PUB) {
      const rpeg_pub_t& pb = st.pub[sd.a];
      payload = pub_payload(e->P, a[pb.src], a[pb.dst], pb.model);
      ref = 16 + pb.model;
    } else if (sd.type == SLOT_RESHARD) {
      payload = e->P.model[sd.b].n_params * e->P.model[sd.b].sb;
      ref = 16 + sd.b;
    }
    if (node_payload) node_payload[i] = payload;
    if (node_ref) node_ref[i] = ref;
  }
  if (set_peak) std::memcpy(set_peak, out + SLOTS, WAVE * 8);
  return n;
}

int rpeg_eval_trace_metrics(rpeg_engine_t* e, const int16_t* vert_fields, const uint8_t* head4, double* utilization,
                            int32_t* n_active) {
  if (!e || !vert_fields || !head4) return -1;
  const int cap = 4096;
  std::vector<double> start(cap), finish(cap);
  std::vector<int32_t> order(cap), kind(cap), vertex(cap), src(cap);
  std::vector<uint8_t> reserved(cap);
  const int n = rpeg_eval_trace(e, vert_fields, head4, start.data(), finish.data(), order.data(), kind.data(),
                                vertex.data(), nullptr, nullptr, src.data(), nullptr, nullptr, cap, reserved.data());
  if (n < 0) return n;
  const int N = e->P.N, G = e->P.G;
  const int nv = e->P.st[head4[0]].n_vertex;
  auto field = [&](int v, int f) { return (int)vert_fields[v * RPEG_FIELDS + f]; };
  auto same_box = [&](int u, int v) {
    for (int f = 4; f < 10; ++f) if (field(u, f) != field(v, f)) return false;
    return true;
  };
  auto for_devices = [&](int v, auto&& fn) {   // rack-major, as the reference enumerates an allocation
    for (int r = field(v, 4); r < field(v, 4) + field(v, 7); ++r)
      for (int q = field(v, 5); q < field(v, 5) + field(v, 8); ++q)
        for (int g = field(v, 6); g < field(v, 6) + field(v, 9); ++g) fn((r * N + q) * G + g);
  };
  if (n_active) {   // devices inside any allocation of any node: every vertex has operator nodes
    std::vector<char> seen((size_t)e->P.R * N * G, 0);
    int cnt = 0;
    for (int v = 0; v < nv; ++v) for_devices(v, [&](int d) { if (!seen[d]) { seen[d] = 1; ++cnt; } });
    *n_active = cnt;
  }
  if (!utilization) return 0;
  double ms = 0.0;
  for (int i = 0; i < n; ++i) ms = i == 0 ? finish[0] : std::max(ms, finish[i]);
  *utilization = 0.0;
  if (n == 0 || ms <= 0) return 0;
  std::vector<int> by_dispatch(n);
  for (int i = 0; i < n; ++i) by_dispatch[i] = i;
  std::stable_sort(by_dispatch.begin(), by_dispatch.end(), [&](int x, int y) { return order[x] < order[y]; });
  std::vector<int> slot((size_t)e->P.R * N * G, -1);           // device -> position in first-touch order
  std::vector<std::vector<std::pair<double, double>>> spans;
  for (int i : by_dispatch) {
    int owners[2], no = 0;
    if (kind[i] == 0) owners[no++] = vertex[i];
    else { owners[no++] = src[i]; owners[no++] = vertex[i]; }
    int used[2], nu = 0;
    for (int k = 0; k < no; ++k) {
      if (!((reserved[i] >> owners[k]) & 1)) continue;
      if (nu == 1 && same_box(used[0], owners[k])) continue;   // identical allocations once
      used[nu++] = owners[k];
    }
    for (int k = 0; k < nu; ++k)
      for_devices(used[k], [&](int d) {
        if (slot[d] < 0) { slot[d] = (int)spans.size(); spans.emplace_back(); }
        spans[slot[d]].emplace_back(start[i], finish[i]);
      });
  }
  if (spans.empty()) return 0;
  double total = 0.0;
  for (auto& sp : spans) {
    std::sort(sp.begin(), sp.end());
    double merged = 0.0, cs = 0.0, ce = 0.0;
    bool open = false;
    for (const auto& se : sp) {
      if (!open || se.first > ce) {
        if (open) merged += ce - cs;
        cs = se.first; ce = se.second; open = true;
      } else {
        ce = std::max(ce, se.second);
      }
    }
    if (open) merged += ce - cs;
    total += merged / ms;
  }
  *utilization = total / (double)spans.size();
  return 0;
}

}  // extern "C"

// Evaluates the candidates of a simulated-annealing step on the GPU: plans are staged through pinned
// host memory into structure-of-arrays device tensors, scored by the batch kernel (with critical-chain
// masses) and read back in one synchronisation.
namespace {

constexpr size_t HS_IN_BYTES = (size_t)RPEG_MAX_V * RPEG_FIELDS * 2 + 4 + 4;   // per plan: fields, header, class offset
constexpr size_t HS_OUT_BYTES = 3 * 8 + (size_t)RPEG_MAX_V * 8 + 8 + 8 + 8;    // makespan, peak, score, mass, utilisation, mask (padded), done flag (padded)

int ensure_host_stage(rpeg_engine_t* e, HostLane& ln, size_t n, hipStream_t s) {
  if (n <= ln.cap) return 0;
  HIP_TRY(e, hipStreamSynchronize(s));
  ln.release();
  const size_t cap = (std::max<size_t>(n + n / 2, 1024) + 63) & ~size_t(63);
  HIP_TRY(e, hipHostMalloc(&ln.in, HS_IN_BYTES * cap));
  HIP_TRY(e, hipMalloc(&ln.dev, HS_IN_BYTES * cap));
  HIP_TRY(e, hipHostMalloc(&ln.out, HS_OUT_BYTES * cap, hipHostMallocCoherent));   // (the host reads it while a launch runs)
  std::memset(ln.out, 0, HS_OUT_BYTES * cap);
  HIP_TRY(e, hipHostGetDevicePointer((void**)&ln.in_dev, ln.in, 0));
  HIP_TRY(e, hipHostGetDevicePointer((void**)&ln.out_dev, ln.out, 0));
  ln.cap = cap;
  return 0;
}

// Plans in host memory, results to host memory, for a batch small enough for one plan per wavefront: the
// host computes the class of every plan itself (validity gate, signature, table lookup: ~100 ns per plan),
// so the call is one copy to the device, one launch of k_plan, whose first lanes write the results straight
// into pinned host memory, and one wait.  get(i, head, a) yields plan i.  The work comes in two halves so that a
// caller with several lanes (staging buffers and a stream each) can keep one evaluation running while it prepares
// the next: host_small_submit stages and launches, host_small_collect waits and hands the results out.  Submit
// returns 1 when the batch is not eligible (a class too large for k_plan); the caller then takes the device path.
template <class GET>
int host_small_submit(rpeg_engine_t* e, HostLane& ln, uint64_t n, GET get, uint32_t flags, bool want_mass, bool want_util,
                      hipStream_t s) {
  ln.n = n; ln.launched = false; ln.idx.clear();
  if (n == 0) return 0;
  const size_t stride = ((size_t)n + 63) & ~size_t(63);
  ln.stride = stride;
  if (int rc = ensure_host_stage(e, ln, stride, s)) return rc;
  int16_t* in_vert = (int16_t*)ln.in;
  uint8_t* in_head = ln.in + (size_t)RPEG_MAX_V * RPEG_FIELDS * 2 * stride;
  uint32_t* in_cls = (uint32_t*)(in_head + 4 * stride);
  uint64_t n_new = 0;
  for (uint64_t i = 0; i < n; ++i) {
    PlanHead h;
    VPlan a[RPEG_MAX_V];
    get(i, h, a);
    const int nv = (h.structure >= 0 && h.structure < e->P.n_struct) ? e->P.st[h.structure].n_vertex : 0;
    if (nv == 0 || !plan_valid(e->P, h, a)) continue;
    bool is_new = false;
    const int64_t off = class_offset(e, plan_signature(e->P, h.structure, h.split, h.tau0, h.tau1, a), &is_new);
    if (off < 0) return -5;
    n_new += is_new ? 1 : 0;
    const size_t j = ln.idx.size();
    ln.idx.push_back((uint32_t)i);
    for (int v = 0; v < nv; ++v) {
      int16_t* p = in_vert + (size_t)v * RPEG_FIELDS * stride + j;
      p[0 * stride] = (int16_t)a[v].dp; p[1 * stride] = (int16_t)a[v].pp; p[2 * stride] = (int16_t)a[v].tp; p[3 * stride] = (int16_t)a[v].mb;
      p[4 * stride] = (int16_t)a[v].o[0]; p[5 * stride] = (int16_t)a[v].o[1]; p[6 * stride] = (int16_t)a[v].o[2];
      p[7 * stride] = (int16_t)a[v].e[0]; p[8 * stride] = (int16_t)a[v].e[1]; p[9 * stride] = (int16_t)a[v].e[2];
    }
    in_head[0 * stride + j] = (uint8_t)h.structure; in_head[1 * stride + j] = (uint8_t)h.split;
    in_head[2 * stride + j] = (uint8_t)h.tau0; in_head[3 * stride + j] = (uint8_t)h.tau1;
    in_cls[j] = (uint32_t)off;
  }
  const size_t m = ln.idx.size();
  e->stats[0] = 0; e->stats[1] = n_new; e->stats[2] = m; e->stats[3] = 0; e->stats[4] = 0; e->stats[5] = 1; e->stats[6] = 0;
  if (m == 0) return 0;
  if (e->max_nodes > (uint32_t)(WAVE * KP_MAX_NS) || kp_lds_bytes(e->max_nodes, e->max_slots) > 64 * 1024) return 1;
  if (int rc = ensure_pool(e, s)) return rc;
  if (!ln.direct) HIP_TRY(e, hipMemcpyAsync(ln.dev, ln.in, HS_IN_BYTES * stride, hipMemcpyHostToDevice, s));
  const uint8_t* d_in = ln.direct ? ln.in_dev : ln.dev;
  double* o_makespan = (double*)ln.out_dev;
  double* o_peak = o_makespan + stride;
  double* o_score = o_peak + stride;
  double* o_mass = o_score + stride;
  double* o_util = o_mass + (size_t)RPEG_MAX_V * stride;
  uint8_t* o_mask = (uint8_t*)(o_util + stride);
  EvalLaunch L;
  L.P = e->dP;
  L.vert = (const int16_t*)d_in;
  L.head = d_in + (size_t)RPEG_MAX_V * RPEG_FIELDS * 2 * stride;
  L.stride = stride;
  L.perm = nullptr;
  L.wave_cls = (const uint32_t*)(L.head + 4 * stride);
  L.pool = e->d_pool; L.ws = nullptr;
  L.n_waves = m; L.ws_nodes = e->max_nodes; L.ws_slots = e->max_slots;
  L.cls_bytes = 0; L.rcap = 0; L.max_v = e->max_v; L.ovf = nullptr; L.need = nullptr;
  L.flags = flags; L.makespan = o_makespan; L.peak = o_peak; L.score = o_score; L.mask = o_mask;
  L.mass = want_mass ? o_mass : nullptr;
  L.util = want_util ? o_util : nullptr;
  L.prof = nullptr;
  if (e->prof_on) {   // phase clocks of this launch's wavefronts, read with rpeg_engine_profile
    if (e->prof_waves < m) {
      HIP_TRY(e, hipStreamSynchronize(s));
      if (e->d_prof) hipFree(e->d_prof);
      e->d_prof = nullptr;
      HIP_TRY(e, hipMalloc(&e->d_prof, m * 64));
    }
    HIP_TRY(e, hipMemsetAsync(e->d_prof, 0, m * 64, s));
    e->prof_waves = m;
    L.prof = e->d_prof;
  }
  if (ln.direct) {
    if (++ln.tag == 0) ++ln.tag;
    L.done = (uint32_t*)(o_mask + stride);
    L.done_tag = ln.tag;
  }
  const size_t lds = kp_lds_bytes(e->max_nodes, e->max_slots);
  const unsigned grid = (unsigned)std::min<uint64_t>(m, (uint64_t)e->n_cu * 32);
  e->stats[3] = lds;
  if (e->timing) HIP_TRY(e, hipEventRecord(e->ev0, s));
  hipLaunchKernelGGL(k_plan, dim3(grid), dim3(WAVE), lds, s, L);
  HIP_TRY(e, hipGetLastError());
  if (e->timing) HIP_TRY(e, hipEventRecord(e->ev1, s));
  ln.launched = true;
  ++e->lanes_busy;
  return 0;
}

// Output arrays may be null; plans the validity gate refuses read NaN and a zero mask.
int host_small_collect(rpeg_engine_t* e, HostLane& ln, double* makespan, double* peak, double* score, uint8_t* mask,
                       double* mass, double* util, hipStream_t s) {
  const size_t n = ln.n, m = ln.idx.size(), stride = ln.stride;
  if (ln.launched) {
    ln.launched = false;
    --e->lanes_busy;
    bool seen = false;
    if (ln.direct) {
      // the flags of all plans, in pinned memory: a plan's results are there once its flag is
      const uint32_t* done = (const uint32_t*)(ln.out + (3 * 8 + (size_t)RPEG_MAX_V * 8 + 8) * stride + stride);
      const auto t0 = std::chrono::steady_clock::now();
      size_t j = 0;
      for (uint64_t spins = 0;; ++spins) {
        while (j < m && __atomic_load_n(&done[j], __ATOMIC_ACQUIRE) == ln.tag) ++j;
        if (j == m) { seen = true; break; }
        // a launch that does not come to an end is the stream's to report
        if ((spins & 0xFFFFu) == 0xFFFFu && std::chrono::steady_clock::now() - t0 > std::chrono::seconds(2)) break;
#if defined(__x86_64__) || defined(__i386__)
        __builtin_ia32_pause();
#endif
      }
    }
    if (!seen) HIP_TRY(e, hipStreamSynchronize(s));
    if (e->timing && !seen) {
      float ms = 0.f;
      HIP_TRY(e, hipEventElapsedTime(&ms, e->ev0, e->ev1));
      e->last_ms = ms;
    }
  }
  if (m < n) {
    const double nan = __builtin_nan("");
    for (size_t i = 0; i < n; ++i) {
      if (makespan) makespan[i] = nan;
      if (peak) peak[i] = nan;
      if (score) score[i] = nan;
      if (mask) mask[i] = 0;
      if (mass)
        for (int x = 0; x < RPEG_MAX_V; ++x) mass[i * RPEG_MAX_V + x] = nan;
      if (util) util[i] = nan;
    }
  }
  if (m == 0) return 0;
  const double* o_makespan = (const double*)ln.out;
  const double* o_peak = o_makespan + stride;
  const double* o_score = o_peak + stride;
  const double* o_mass = o_score + stride;
  const double* o_util = o_mass + (size_t)RPEG_MAX_V * stride;
  const uint8_t* o_mask = (const uint8_t*)(o_util + stride);
  for (size_t j = 0; j < m; ++j) {
    const uint32_t i = ln.idx[j];
    if (makespan) makespan[i] = o_makespan[j];
    if (peak) peak[i] = o_peak[j];
    if (score) score[i] = o_score[j];
    if (mask) mask[i] = o_mask[j];
    if (mass)
      for (int x = 0; x < RPEG_MAX_V; ++x) mass[(size_t)i * RPEG_MAX_V + x] = o_mass[j * RPEG_MAX_V + x];
    if (util) util[i] = o_util[j];
  }
  return 0;
}

template <class GET>
int eval_host_small(rpeg_engine_t* e, uint64_t n, GET get, uint32_t flags, double* makespan, double* peak, double* score,
                    uint8_t* mask, double* mass, hipStream_t s, double* util = nullptr) {
  e->last_ms = -1.0;
  const int rc = host_small_submit(e, e->lane0, n, get, flags, mass != nullptr, util != nullptr, s);
  if (rc != 0) return rc;
  return host_small_collect(e, e->lane0, makespan, peak, score, mask, mass, util, s);
}

}  // namespace

// rpeg_eval_host: plans and results in host memory.  Small batches go through eval_host_small; larger ones
// (or problems whose classes are too large for it) are copied to the device and take the batch path.
static int eval_host_impl(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                          double* peak, double* score, uint8_t* mask, double* mass, void* stream) {
  if (!e || !plans) return -1;
  e->err.clear();
  e->last_ms = -1.0;
  if (n == 0) return 0;
  if (n >= (1ull << 32)) { e->err = "at most 2^32-1 plans per call"; return -1; }
  if (!plans->vert || !plans->head || plans->stride < n) { e->err = "bad plan tensors"; return -1; }
  hipStream_t s = (hipStream_t)stream;
  const int16_t* vert = plans->vert;
  const uint8_t* head = plans->head;
  const uint64_t stride = plans->stride;
  if ((e->state_lanes == -1 || e->state_lanes == 1) && n <= (uint64_t)e->host_small_max) {
    auto get = [&](uint64_t i, PlanHead& h, VPlan (&a)[RPEG_MAX_V]) {
      h = load_head(head, stride, i);
      const int nv = (h.structure >= 0 && h.structure < e->P.n_struct) ? e->P.st[h.structure].n_vertex : 0;
      for (int v = 0; v < nv; ++v) load_vertex(vert, stride, i, v, &a[v]);
    };
    const int rc = eval_host_small(e, n, get, flags, makespan, peak, score, mask, mass, s);
    if (rc <= 0) return rc;
  }
  // device path: stage the tensors and the results in device memory for this call
  const size_t V = (size_t)RPEG_MAX_V * RPEG_FIELDS;
  const size_t b_vert = V * 2 * n, b_head = 4 * n, b_f64 = 8 * n;
  const size_t o_head = (b_vert + 255) & ~size_t(255), o_mk = (o_head + b_head + 255) & ~size_t(255), o_pk = o_mk + b_f64,
               o_sc = o_pk + b_f64, o_ms = o_sc + b_f64, o_mask = o_ms + (mass ? b_f64 * RPEG_MAX_V : 0), total = o_mask + n;
  if (total > e->d_stage_cap) {   // grow-only staging block, kept by the engine
    HIP_TRY(e, hipStreamSynchronize(s));
    if (e->d_stage) hipFree(e->d_stage);
    e->d_stage = nullptr;
    e->d_stage_cap = 0;
    HIP_TRY(e, hipMalloc(&e->d_stage, total + total / 4));
    e->d_stage_cap = total + total / 4;
  }
  uint8_t* d = e->d_stage;
  int rc = 0;
  auto fail = [&](hipError_t st, const char* what) { e->err = std::string(what) + ": " + hipGetErrorString(st); rc = -2; };
  // results come back in one copy into a pinned mirror of the output region
  const size_t b_out = total - o_mk;
  if (b_out > e->h_stage_cap) {
    HIP_TRY(e, hipStreamSynchronize(s));
    if (e->h_stage) hipHostFree(e->h_stage);
    e->h_stage = nullptr;
    e->h_stage_cap = 0;
    HIP_TRY(e, hipHostMalloc(&e->h_stage, b_out + b_out / 4));
    e->h_stage_cap = b_out + b_out / 4;
  }
  hipError_t st = stride == n ? hipMemcpyAsync(d, vert, b_vert, hipMemcpyHostToDevice, s)
                              : hipMemcpy2DAsync(d, n * 2, vert, stride * 2, n * 2, V, hipMemcpyHostToDevice, s);
  if (st != hipSuccess) fail(st, "hipMemcpyAsync");
  if (!rc) {
    st = stride == n ? hipMemcpyAsync(d + o_head, head, b_head, hipMemcpyHostToDevice, s)
                     : hipMemcpy2DAsync(d + o_head, n, head, stride, n, 4, hipMemcpyHostToDevice, s);
    if (st != hipSuccess) fail(st, "hipMemcpyAsync");
  }
  if (!rc) {
    rpeg_plan_soa_t soa{(const int16_t*)d, d + o_head, n};
    rc = eval_batch_impl(e, n, &soa, flags, (double*)(d + o_mk), (double*)(d + o_pk), (double*)(d + o_sc), d + o_mask,
                         mass ? (double*)(d + o_ms) : nullptr, stream);
  }
  const double last_ms = e->last_ms;
  if (!rc && (st = hipMemcpyAsync(e->h_stage, d + o_mk, b_out, hipMemcpyDeviceToHost, s)) != hipSuccess) fail(st, "hipMemcpyAsync");
  const hipError_t sy = hipStreamSynchronize(s);
  if (!rc && sy != hipSuccess) fail(sy, "hipStreamSynchronize");
  if (!rc) {
    const uint8_t* h = e->h_stage - o_mk;   // same offsets as in the device block
    if (makespan) std::memcpy(makespan, h + o_mk, b_f64);
    if (peak) std::memcpy(peak, h + o_pk, b_f64);
    if (score) std::memcpy(score, h + o_sc, b_f64);
    if (mass) std::memcpy(mass, h + o_ms, b_f64 * RPEG_MAX_V);
    if (mask) std::memcpy(mask, h + o_mask, n);
  }
  e->last_ms = last_ms;
  return rc;
}

namespace {
struct GpuSaBackend : SaBackend {
  rpeg_engine_t* e;
  hipStream_t s;
  int cap = 0;
  uint8_t head_of[256][4] = {};
  int16_t *h_vert = nullptr, *d_vert = nullptr;
  uint8_t *h_head = nullptr, *d_head = nullptr, *h_mask = nullptr, *d_mask = nullptr;
  double *h_score = nullptr, *d_score = nullptr, *h_mass = nullptr, *d_mass = nullptr, *h_util = nullptr;
  double eval_s = 0.0;
  long n_launch = 0, n_plans = 0;
  int rc_alloc = 0;
  // lanes of submit() / collect(): staging buffers and a stream each, so that the evaluation of one group of chains
  // runs while the host merges and proposes for another
  struct Lane {
    HostLane st;
    hipStream_t s = nullptr;
    bool deferred = false;     // the batch is not one for k_plan: evaluated in collect()
    int n = 0;
    const SaPlan* plans = nullptr;
    const uint8_t* variant = nullptr;
  };
  std::vector<Lane> lane;

  GpuSaBackend(rpeg_engine_t* eng, hipStream_t st, int capacity, int n_lanes = 1) : e(eng), s(st), cap(capacity) {
    lane.resize((size_t)std::max(1, n_lanes));
    for (Lane& l : lane) {
      l.st.direct = true;
      if (hipStreamCreateWithFlags(&l.s, hipStreamNonBlocking) != hipSuccess) { rc_alloc = -2; e->err = "hipStreamCreate failed"; l.s = nullptr; }
    }
    const size_t V = RPEG_MAX_V * RPEG_FIELDS;
    bool ok = hipHostMalloc(&h_vert, V * cap * 2) == hipSuccess && hipMalloc(&d_vert, V * cap * 2) == hipSuccess &&
              hipHostMalloc(&h_head, 4 * (size_t)cap) == hipSuccess && hipMalloc(&d_head, 4 * (size_t)cap) == hipSuccess &&
              hipHostMalloc(&h_mask, cap) == hipSuccess && hipMalloc(&d_mask, cap) == hipSuccess &&
              hipHostMalloc(&h_score, 8 * (size_t)cap) == hipSuccess && hipMalloc(&d_score, 8 * (size_t)cap) == hipSuccess &&
              hipHostMalloc(&h_mass, 8 * (size_t)cap * RPEG_MAX_V) == hipSuccess &&
              hipMalloc(&d_mass, 8 * (size_t)cap * RPEG_MAX_V) == hipSuccess &&
              hipHostMalloc(&h_util, 8 * (size_t)cap) == hipSuccess;
    if (!ok) { rc_alloc = -2; e->err = "out of memory for the annealing buffers"; }
    else std::memset(h_vert, 0, V * cap * 2);
  }
  ~GpuSaBackend() override {
    hipStreamSynchronize(s);
    for (Lane& l : lane) {
      if (l.st.launched) { --e->lanes_busy; l.st.launched = false; }
      if (l.s) { hipStreamSynchronize(l.s); hipStreamDestroy(l.s); }
      l.st.release();
    }
    if (h_vert) hipHostFree(h_vert);
    if (d_vert) hipFree(d_vert);
    if (h_head) hipHostFree(h_head);
    if (d_head) hipFree(d_head);
    if (h_mask) hipHostFree(h_mask);
    if (d_mask) hipFree(d_mask);
    if (h_score) hipHostFree(h_score);
    if (d_score) hipFree(d_score);
    if (h_mass) hipHostFree(h_mass);
    if (d_mass) hipFree(d_mass);
    if (h_util) hipHostFree(h_util);
  }

  int utilization(const SaPlan& plan, uint8_t variant, double* out) override {
    return rpeg_eval_trace_metrics(e, &plan.f[0][0], head_of[variant], out, nullptr);
  }

  int evaluate(int n, const SaPlan* plans, const uint8_t* variant, SaEval* out) override { return evaluate(n, plans, variant, out, false); }

  int lanes() const override { return (int)lane.size(); }

  int submit(int li, int n, const SaPlan* plans, const uint8_t* variant) override {
    Lane& l = lane[(size_t)li];
    l.n = n; l.plans = plans; l.variant = variant; l.deferred = false;
    if (n > cap) { e->err = "annealing batch exceeds its buffers"; return -1; }
    const auto t0 = std::chrono::steady_clock::now();
    auto get = [&](uint64_t i, PlanHead& h, VPlan (&a)[RPEG_MAX_V]) {
      const uint8_t* hd = head_of[variant[i]];
      h.structure = hd[0]; h.split = hd[1]; h.tau0 = hd[2]; h.tau1 = hd[3];
      const int nv = e->P.st[hd[0]].n_vertex;
      for (int v = 0; v < nv; ++v) {
        const int16_t* f = plans[i].f[v];
        a[v].dp = f[0]; a[v].pp = f[1]; a[v].tp = f[2]; a[v].mb = f[3];
        a[v].o[0] = f[4]; a[v].o[1] = f[5]; a[v].o[2] = f[6];
        a[v].e[0] = f[7]; a[v].e[1] = f[8]; a[v].e[2] = f[9];
      }
    };
    const int rc = host_small_submit(e, l.st, (uint64_t)n, get, 0u, true, false, l.s);
    eval_s += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    if (rc == 1) { l.deferred = true; return 0; }
    return rc;
  }

  int collect(int li, SaEval* out) override {
    Lane& l = lane[(size_t)li];
    if (l.deferred) { l.deferred = false; return evaluate(l.n, l.plans, l.variant, out, false); }
    if (l.n == 0) return 0;
    const auto t0 = std::chrono::steady_clock::now();
    if (int rc = host_small_collect(e, l.st, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, l.s)) return rc;
    const size_t n = l.st.n, m = l.st.idx.size(), stride = l.st.stride;
    if (m < n) {
      const double nan = __builtin_nan("");
      for (size_t i = 0; i < n; ++i) {
        out[i].score = nan;
        out[i].mask = 0;
        for (int x = 0; x < RPEG_MAX_V; ++x) out[i].mass[x] = nan;
      }
    }
    const double* o_score = (const double*)l.st.out + 2 * stride;
    const double* o_mass = o_score + stride;
    const uint8_t* o_mask = (const uint8_t*)(o_mass + (size_t)RPEG_MAX_V * stride + stride);
    for (size_t j = 0; j < m; ++j) {
      SaEval& o = out[l.st.idx[j]];
      o.score = o_score[j];
      o.mask = o_mask[j];
      for (int x = 0; x < RPEG_MAX_V; ++x) o.mass[x] = o_mass[j * RPEG_MAX_V + x];
    }
    eval_s += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    ++n_launch;
    n_plans += l.n;
    return 0;
  }

  // with_util: Trace.utilization() of every plan from the same launch (out[i].util); 1 when this batch cannot
  // take that path (the caller then asks per plan)
  int evaluate(int n, const SaPlan* plans, const uint8_t* variant, SaEval* out, bool with_util) override {
    if (n > cap) { e->err = "annealing batch exceeds its buffers"; return -1; }
    {  // a step's proposals are a small batch: one copy, one launch (eval_host_small)
      const auto t0 = std::chrono::steady_clock::now();
      auto get = [&](uint64_t i, PlanHead& h, VPlan (&a)[RPEG_MAX_V]) {
        const uint8_t* hd = head_of[variant[i]];
        h.structure = hd[0]; h.split = hd[1]; h.tau0 = hd[2]; h.tau1 = hd[3];
        const int nv = e->P.st[hd[0]].n_vertex;
        for (int v = 0; v < nv; ++v) {
          const int16_t* f = plans[i].f[v];
          a[v].dp = f[0]; a[v].pp = f[1]; a[v].tp = f[2]; a[v].mb = f[3];
          a[v].o[0] = f[4]; a[v].o[1] = f[5]; a[v].o[2] = f[6];
          a[v].e[0] = f[7]; a[v].e[1] = f[8]; a[v].e[2] = f[9];
        }
      };
      const int rc = eval_host_small(e, (uint64_t)n, get, 0u, nullptr, nullptr, h_score, h_mask, h_mass, s,
                                     with_util ? h_util : nullptr);
      if (rc < 0) return rc;
      if (rc == 0) {
        for (int i = 0; i < n; ++i) {
          out[i].score = h_score[i];
          out[i].mask = h_mask[i];
          for (int x = 0; x < RPEG_MAX_V; ++x) out[i].mass[x] = h_mass[(size_t)i * RPEG_MAX_V + x];
          if (with_util) out[i].util = h_util[i];
        }
        eval_s += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
        ++n_launch;
        n_plans += n;
        return 0;
      }
    }
    if (with_util) return 1;   // the staged path has no utilisation output
    const auto t0 = std::chrono::steady_clock::now();
    const size_t V = RPEG_MAX_V * RPEG_FIELDS;
    for (int i = 0; i < n; ++i) {
      const int16_t* f = &plans[i].f[0][0];
      for (size_t x = 0; x < V; ++x) h_vert[x * cap + i] = f[x];
      for (int x = 0; x < 4; ++x) h_head[(size_t)x * cap + i] = head_of[variant[i]][x];
    }
    // rows are `cap` apart: copy the used prefix of every row in one strided copy
    HIP_TRY(e, hipMemcpy2DAsync(d_vert, (size_t)cap * 2, h_vert, (size_t)cap * 2, (size_t)n * 2, V, hipMemcpyHostToDevice, s));
    HIP_TRY(e, hipMemcpy2DAsync(d_head, cap, h_head, cap, n, 4, hipMemcpyHostToDevice, s));
    rpeg_plan_soa_t soa{d_vert, d_head, (uint64_t)cap};
    if (int rc = eval_batch_impl(e, (uint64_t)n, &soa, 0u, nullptr, nullptr, d_score, d_mask, d_mass, s)) return rc;
    HIP_TRY(e, hipMemcpyAsync(h_score, d_score, 8 * (size_t)n, hipMemcpyDeviceToHost, s));
    HIP_TRY(e, hipMemcpyAsync(h_mask, d_mask, n, hipMemcpyDeviceToHost, s));
    HIP_TRY(e, hipMemcpyAsync(h_mass, d_mass, 8 * (size_t)n * RPEG_MAX_V, hipMemcpyDeviceToHost, s));
    HIP_TRY(e, hipStreamSynchronize(s));
    for (int i = 0; i < n; ++i) {
      out[i].score = h_score[i];
      out[i].mask = h_mask[i];
      for (int x = 0; x < RPEG_MAX_V; ++x) out[i].mass[x] = h_mass[(size_t)i * RPEG_MAX_V + x];
    }
    eval_s += std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    ++n_launch;
    n_plans += n;
    return 0;
  }
};
}  // namespace

extern "C" {

int rpeg_eval_host_util(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                        double* peak, double* score, uint8_t* mask, double* utilization, void* stream) {
  if (!e || !plans || !utilization) return -1;
  e->err.clear();
  e->last_ms = -1.0;
  if (n == 0) return 0;
  if (n >= (1ull << 32)) { e->err = "at most 2^32-1 plans per call"; return -1; }
  if (!plans->vert || !plans->head || plans->stride < n) { e->err = "bad plan tensors"; return -1; }
  const int16_t* vert = plans->vert;
  const uint8_t* head = plans->head;
  const uint64_t stride = plans->stride;
  // one launch of a plan per wavefront for every `host_small_max` plans
  const uint64_t piece = std::max<uint64_t>(1, e->host_small_max);
  bool too_large = false;
  for (uint64_t a = 0; a < n && !too_large; a += piece) {
    const uint64_t m = std::min(piece, n - a);
    auto get = [&](uint64_t i, PlanHead& h, VPlan (&pl)[RPEG_MAX_V]) {
      h = load_head(head, stride, a + i);
      const int nv = (h.structure >= 0 && h.structure < e->P.n_struct) ? e->P.st[h.structure].n_vertex : 0;
      for (int v = 0; v < nv; ++v) load_vertex(vert, stride, a + i, v, &pl[v]);
    };
    const int rc = eval_host_small(e, m, get, flags, makespan ? makespan + a : nullptr, peak ? peak + a : nullptr,
                                   score ? score + a : nullptr, mask ? mask + a : nullptr, nullptr, (hipStream_t)stream,
                                   utilization + a);
    if (rc == 1) too_large = true;
    else if (rc) return rc;
  }
  if (!too_large) return 0;
  // A class of this problem has more nodes than a wavefront holds: the batch takes the path of rpeg_eval_host and
  // every plan is traced on its own for its utilisation (rpeg_eval_trace_metrics).
  std::vector<uint8_t> own_mask;
  if (!mask) { own_mask.resize(n); mask = own_mask.data(); }
  if (int rc = eval_host_impl(e, n, plans, flags, makespan, peak, score, mask, nullptr, stream)) return rc;
  for (uint64_t i = 0; i < n; ++i) {
    utilization[i] = __builtin_nan("");
    if (!(mask[i] & RPEG_MASK_VALID) || (mask[i] & RPEG_MASK_ERROR)) continue;
    int16_t f[RPEG_MAX_V * RPEG_FIELDS] = {};
    uint8_t h4[4];
    for (int x = 0; x < RPEG_MAX_V * RPEG_FIELDS; ++x) f[x] = vert[(uint64_t)x * stride + i];
    for (int x = 0; x < 4; ++x) h4[x] = head[(uint64_t)x * stride + i];
    if (int rc = rpeg_eval_trace_metrics(e, f, h4, &utilization[i], nullptr)) return rc;
  }
  return 0;
}

int rpeg_sa_run(rpeg_engine_t* e, const rpeg_sa_params_t* prm, const int16_t* base_plan, rpeg_sa_result_t* res,
                void* stream) {
  if (!e || !prm || !res) return -1;
  e->err.clear();
  if (prm->structure < 0 || prm->structure >= e->P.n_struct || prm->split < 0 || prm->split >= e->P.n_split ||
      prm->n_variants < 1 || prm->n_variants > 8 || prm->n_chains < 1 || prm->n_steps < 0 || prm->K_x < 1 ||
      prm->K_x > 16 || prm->restart_attempts < 1 || prm->T_max < 0 || !(prm->T_init > 0.0)) {
    e->err = "bad annealing parameters";
    return -1;
  }
  SaContext cx;
  cx.init(e->P, prm->structure);
  for (int v = 0; v < cx.nv; ++v) {
    if (prm->dir_n[v] < 0 || (prm->dir_n[v] > 0 && !prm->dir[v])) { e->err = "bad candidate directory"; return -1; }
    if (const char* msg = cx.set_directory(v, prm->dir[v], prm->dir_n[v])) { e->err = msg; return -1; }
  }
  SaSettings st;
  sa_settings_from(*prm, &st);
  const int cap = prm->n_chains * std::max(prm->K_x, prm->restart_attempts);
  // chains in groups of at least 8, at most `sa_lanes` groups
  GpuSaBackend be(e, (hipStream_t)stream, cap, std::max(1, std::min(e->sa_lanes, prm->n_chains / 8)));
  if (be.rc_alloc) return be.rc_alloc;
  for (int k = 0; k < prm->n_variants; ++k) {
    be.head_of[k][0] = (uint8_t)prm->structure; be.head_of[k][1] = (uint8_t)prm->split;
    be.head_of[k][2] = prm->tau[k][0]; be.head_of[k][3] = prm->tau[k][1];
  }
  SaRun run(cx, st, be);
  SaPlan base;
  if (base_plan) std::memcpy(&base, base_plan, sizeof base);
  const bool was_timing = e->timing;
  e->timing = false;
  const int rc = run.run(base_plan ? &base : nullptr);
  e->timing = was_timing;
  if (rc) return rc;
  sa_run_result(run, res);
  res->eval_s = be.eval_s;
  res->n_launch = be.n_launch;
  res->n_plans = be.n_plans;
  return 0;
}

int rpeg_sa_optimize_families(rpeg_engine_t* e, int32_t n_families, const rpeg_sa_family_t* families,
                              const uint8_t base_tau[2], int32_t E_max, int32_t E_struct, int32_t R_max,
                              uint64_t stream_a, uint64_t stream_b, uint64_t stream_c, const int16_t* base_plan,
                              rpeg_sa_serial_result_t* res, void* stream) {
  if (!e || !families || !base_tau || !res || !base_plan || n_families < 1 || !families[0].params) return -1;
  e->err.clear();
  const rpeg_sa_params_t* prm = families[0].params;
  if (prm->K_x < 1 || prm->K_x > 16 || prm->T_max < 0 || !(prm->T_init > 0.0) || E_max < 1 || E_struct < 1 || R_max < 1) {
    e->err = "bad annealing parameters";
    return -1;
  }
  GpuSaBackend be(e, (hipStream_t)stream, std::max(prm->K_x, 16));
  if (be.rc_alloc) return be.rc_alloc;
  SaFamilySetup setup;
  if (const char* msg = setup.init(e->P, n_families, families, base_tau, be.head_of)) { e->err = msg; return -1; }
  SaSettings st;
  sa_settings_from(*prm, &st);
  SaSerial run(setup.fam, st, be, E_max, E_struct, R_max, prm->seed, stream_a, stream_b, stream_c);
  SaPlan base;
  std::memcpy(&base, base_plan, sizeof base);
  const auto t0 = std::chrono::steady_clock::now();
  const bool was_timing = e->timing;
  e->timing = false;
  const int rc = run.run(base, setup.base_variant);
  e->timing = was_timing;
  if (rc) return rc;
  sa_serial_result(run, res);
  res->wall_s = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
  return 0;
}

int rpeg_sa_optimize(rpeg_engine_t* e, const rpeg_sa_params_t* prm, int32_t E_max, int32_t E_struct, int32_t R_max,
                     uint64_t stream_a, uint64_t stream_b, uint64_t stream_c, const int16_t* base_plan,
                     rpeg_sa_serial_result_t* res, void* stream) {
  if (!e || !prm) return -1;
  const rpeg_sa_family_t one{prm, 1.0, 0, prm->structure};
  return rpeg_sa_optimize_families(e, 1, &one, prm->tau[0], E_max, E_struct, R_max, stream_a, stream_b, stream_c,
                                   base_plan, res, stream);
}

int rpeg_sa_propose(rpeg_engine_t* e, const rpeg_sa_params_t* prm, int32_t what, uint64_t stream_a, uint64_t stream_b,
                    uint64_t stream_c, const int16_t* plan, const double* mass, double T, int32_t vertex, int32_t r_lo,
                    int32_t r_hi, int16_t* out, int64_t* draws, int32_t* fallback) {
  if (!e || !prm || !out || what < 0 || what > 2) return -1;
  e->err.clear();
  if (prm->structure < 0 || prm->structure >= e->P.n_struct || prm->K_x < 1 || prm->K_x > 16 || !(prm->T_init > 0.0) ||
      prm->T_max < 0 || (what < 2 && !plan) || (what == 0 && !mass)) {
    e->err = "bad proposal parameters";
    return -1;
  }
  SaContext cx;
  cx.init(e->P, prm->structure);
  cx.fixed_mb = prm->fixed_mb != 0;
  cx.uniform_vertex = prm->uniform_vertex != 0;
  for (int v = 0; v < cx.nv; ++v) {
    if (prm->dir_n[v] < 0 || (prm->dir_n[v] > 0 && !prm->dir[v])) { e->err = "bad candidate directory"; return -1; }
    if (const char* msg = cx.set_directory(v, prm->dir[v], prm->dir_n[v])) { e->err = msg; return -1; }
  }
  if (what == 2 && (vertex < 0 || vertex >= cx.nv || r_lo < 0 || r_hi > cx.R || r_lo >= r_hi)) {
    e->err = "bad vertex or rack range";
    return -1;
  }
  if (what == 0)
    for (int v = 0; v < cx.nv; ++v)
      if (prm->dir_n[v] == 0) { e->err = "empty candidate table"; return -1; }   // the reference's move_gen raises on one
  SaRng rng(prm->seed, stream_a, stream_b, stream_c);
  if (draws) rng.k = (uint64_t)*draws;
  SaPlan cur;
  if (plan) std::memcpy(&cur, plan, sizeof cur);
  int n = 0, fb = 0;
  if (what == 0) {
    std::vector<SaPlan> o(prm->K_x);
    n = sa_move_gen(rng, cx, cur, mass, prm->K_x, prm->T_max, T, prm->T_init, o.data(), &fb);
    std::memcpy(out, o.data(), sizeof(SaPlan) * n);
  } else if (what == 1) {
    SaPlan o;
    n = sa_move_pair(rng, cx, cur, &o) ? 1 : 0;
    if (n) std::memcpy(out, &o, sizeof o);
  } else {
    n = sa_sample_region(rng, cx, vertex, r_lo, r_hi, out) ? 1 : 0;
  }
  if (draws) *draws = (int64_t)rng.k;
  if (fallback) *fallback = fb;
  return n;
}

int rpeg_device_exp(rpeg_engine_t* e, uint64_t n, const double* x, double* y, void* stream) {
  if (!e || !x || !y) return -1;
  if (n == 0) return 0;
  hipLaunchKernelGGL(k_exp, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, (hipStream_t)stream, n, x, y);
  HIP_TRY(e, hipGetLastError());
  return 0;
}

}  // extern "C"
