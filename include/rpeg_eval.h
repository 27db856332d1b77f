/*
 * rpeg_eval.h - C ABI of the MI355X batched plan evaluator.
 *
 * The reference (spcl/RPEG) is pure Python and has no FFI; its drop-in boundary is the Python
 * call `search.evaluate._eval_worker / evaluate_cached` (RPEG/search/evaluate.py:329-442), which
 * the simulated-annealing driver maps over the K_x candidates of one step
 * (RPEG/search/optimizer.py:793-798).  This library replaces that map by one batched call on the
 * GPU.  All entry points use plain pointers and sizes; plan tensors and outputs are DEVICE
 * pointers (structure-of-arrays, see rpeg_plan_soa_t), everything else is host memory.
 *
 * Status codes: 0 ok, negative = error (text via rpeg_last_error).
 */
#ifndef RPEG_EVAL_H
#define RPEG_EVAL_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define RPEG_ABI_VERSION 4

#define RPEG_MAX_V 6       /* template vertices per structure                */
#define RPEG_MAX_E 9       /* within-step data edges                          */
#define RPEG_MAX_PUB 2     /* publication edges                               */
#define RPEG_MAX_PAIR 4    /* consecutive same-model vertex pairs             */
#define RPEG_MAX_REL 13    /* vertex pairs whose relation decides the lowering */
#define RPEG_MAX_PH 6      /* generation phases (quantiles)                   */
#define RPEG_MAX_SPLIT 7   /* split variants: 0 = unsplit, j = quantiles[j-1:] */
#define RPEG_MAX_MODEL 5
#define RPEG_MAX_STRUCT 3
#define RPEG_FIELDS 10     /* per-vertex plan fields: dp pp tp mb o_r o_n o_g e_r e_n e_g */

enum { RPEG_ROLE_GEN = 0, RPEG_ROLE_INF = 1, RPEG_ROLE_TRAIN = 2 };
enum { RPEG_MODEL_ACTOR = 0, RPEG_MODEL_CRITIC = 1, RPEG_MODEL_REFERENCE = 2, RPEG_MODEL_REWARD = 3,
       RPEG_MODEL_AC_SHARE = 4 };

/* need flags of a relation pair */
enum { RPEG_NEED_DISJ = 1, RPEG_NEED_PI = 2 };

/* mask bits written per plan */
enum {
  RPEG_MASK_VALID = 1,     /* integer validity rules of is_valid (evaluate.py:172-196) hold   */
  RPEG_MASK_STALE_OK = 2,  /* stale_publication_layout_valid (evaluate.py:115-140)            */
  RPEG_MASK_MEM_OK = 4,    /* no device peak above capacity (memory.py:864-887)               */
  RPEG_MASK_ERROR = 8,     /* the reference would raise (division by zero, cycle) or an engine
                              limit was hit; the numeric outputs of this plan are NaN           */
  RPEG_MASK_LIMIT = 16     /* set with RPEG_MASK_ERROR when the cause is a limit of this engine: the
                              reference would have evaluated the plan.  No evaluation path sets it
                              for a graph within the stated bounds (4,095 lowered nodes per plan):
                              a plan whose ready set outgrows what a kernel holds -- 31 or 32 entries
                              in the plan-per-lane and four-lanes-per-plan kernels -- is redone by
                              the launch that ends the call with a ready list of one entry per
                              node, as the reference's heap has no capacity
                              (RPEG/schedule/scheduler.py:423-546)                                */
};

/* eval flags */
enum {
  RPEG_GATE_STALE = 1,     /* score := 0 when the stale-layout rule fails (evaluate_cached, :372-374);
                              without it the score is what _eval_worker returns (:406-442)      */
  RPEG_NO_WAIT = 2         /* rpeg_eval_batch_static only: enqueue the launches and return, without the
                              copy and the wait that report plans of unknown classes            */
};

/* hardware parameter indices (RPEG/model/hardware.py:17-68, in field order) */
enum {
  RPEG_HW_FLOPS = 0, RPEG_HW_MEM, RPEG_HW_BW,
  RPEG_HW_A_COLL_G, RPEG_HW_B_COLL_G, RPEG_HW_A_COLL_N, RPEG_HW_B_COLL_N, RPEG_HW_A_COLL_R, RPEG_HW_B_COLL_R,
  RPEG_HW_A_P2P_G, RPEG_HW_B_P2P_G, RPEG_HW_A_P2P_N, RPEG_HW_B_P2P_N, RPEG_HW_A_P2P_R, RPEG_HW_B_P2P_R,
  RPEG_HW_M_HALF, RPEG_HW_K_HALF, RPEG_HW_DECODE_EFF, RPEG_HW_NG_CONST, RPEG_HW_NG_SCALE, RPEG_HW_NG_BCAL,
  RPEG_HW_SCALE_GEN, RPEG_HW_SCALE_INF, RPEG_HW_SCALE_TRAIN, RPEG_HW_ACT_OVERHEAD, RPEG_HW_W_COMM_SCALE,
  RPEG_HW_RESHARD_SCALE, RPEG_HW_COUNT
};

typedef struct rpeg_model_s {
  int32_t L, d, d_ff, V, sb, kind;
  int64_t w_layer;        /* 4 d^2 + 2 d d_ff                                        */
  int64_t params_formula; /* L*w_layer + V*d (cost.py:188)                           */
  int64_t n_params;       /* ModelSuite.n_params (models.py:51-82): lowering payloads */
} rpeg_model_t;

/* plan-independent constants of one operator-node variant, evaluated on the host with exact
   Python integer/float semantics (cost.py:481-535, lower.py:288-327) */
typedef struct rpeg_opconst_s {
  double W;          /* float(_work_cost(node))                                  */
  double W_prefill;  /* float(prefill work) for generation nodes with a prefill   */
  double avg_past;   /* generation: S + t_start + steps/2, or S + T/2 unsplit     */
  int32_t n_eff;     /* _effective_batch(node)                                    */
  int32_t steps;     /* decode steps of a generation node                         */
  int32_t prefill;   /* generation node includes the prefill                      */
  int32_t sub;       /* 1: quantile sub-node, 0: unsplit node                     */
} rpeg_opconst_t;

typedef struct rpeg_vertex_s {
  int32_t role, model, topo_idx, tau_slot; /* topo_idx: rank of the id among sorted ids (scheduler.py:385-397) */
  rpeg_opconst_t unsplit;
  rpeg_opconst_t sub[RPEG_MAX_SPLIT][RPEG_MAX_PH];
} rpeg_vertex_t;

typedef struct rpeg_edge_s {
  int32_t src, dst, is_weight, gen_inf;
  int64_t full_bytes;                              /* container bytes                   */
  int64_t sub_bytes[RPEG_MAX_SPLIT][RPEG_MAX_PH];  /* max(1,int(full*n_seq/BK)), lower.py:562-563 */
} rpeg_edge_t;

typedef struct rpeg_pub_s { int32_t src, dst, model, tau_slot; } rpeg_pub_t;
typedef struct rpeg_pair_s { int32_t u, v, model, tau_slot, reach, pad; } rpeg_pair_t;
typedef struct rpeg_rel_s { int32_t u, v, flags, pad; } rpeg_rel_t;

typedef struct rpeg_struct_s {
  int32_t n_vertex, n_edge, n_pub, n_pair, n_rel, n_tau;
  rpeg_vertex_t vertex[RPEG_MAX_V];
  rpeg_edge_t edge[RPEG_MAX_E];
  rpeg_pub_t pub[RPEG_MAX_PUB];
  rpeg_pair_t pair[RPEG_MAX_PAIR];     /* within_step_priors over the LIFO topological order (lower.py:135-220) */
  rpeg_rel_t rel[RPEG_MAX_REL];
  uint8_t reach[RPEG_MAX_V][RPEG_MAX_V];  /* transitive closure of data edges (lower.py:170-193) */
  uint8_t trainable[RPEG_MAX_MODEL + 3];      /* RPEG.trainable: what lowering sees (lower.py:626-793)          */
  uint8_t mem_trainable[RPEG_MAX_MODEL + 3];  /* NodeMemoryModel.trainable: what the memory model sees
                                                 (memory.py:647-790).  evaluate_cached builds it from the template
                                                 (evaluate.py:378-385) and then the two agree; optimize() hands
                                                 is_valid the memory model of its BASE configuration
                                                 (optimizer.py:449-458), which for the AC-share template is another
                                                 set: that view of a template is a structure of its own           */
} rpeg_struct_t;

typedef struct rpeg_phase_s { int32_t n_active, n_seqs, steps, t_start, prefill, pad; } rpeg_phase_t;

typedef struct rpeg_problem_s {
  int32_t abi_version;
  int32_t n_struct, n_split, K_eval;
  int32_t R, N, G;
  int32_t B, K, S, T;
  int32_t optimizer_stage, ckpt, max_groups;
  int32_t n_phase[RPEG_MAX_SPLIT];
  int32_t transfer_both;  /* TransferResourcePolicy (core/types.py:128-200): bit 0 set when weight transfers
                             reserve both endpoints, bit 1 when activation transfers do; 0 = the default  */
  rpeg_phase_t phase[RPEG_MAX_SPLIT][RPEG_MAX_PH];
  double hw[RPEG_HW_COUNT];
  double cap;             /* (1 - eps_rt) * memory_per_gpu (memory.py:291-298)          */
  double group_overhead;  /* worker_overhead_bytes + semantic_activation_cache_bytes      */
  double score_num;       /* float(K_eval * B*K*(S+T)) (evaluate.py:288, trace.py:40-51)  */
  rpeg_model_t model[RPEG_MAX_MODEL];
  rpeg_struct_t st[RPEG_MAX_STRUCT];
} rpeg_problem_t;

/* Candidate plans, structure of arrays, DEVICE memory.
   vert[(slot*RPEG_FIELDS + f) * stride + i]  field f of vertex slot `slot` of plan i
   head[h * stride + i]                       h = 0 structure, 1 split index, 2 tau slot 0, 3 tau slot 1 */
typedef struct rpeg_plan_soa_s {
  const int16_t* vert;
  const uint8_t* head;
  uint64_t stride;
} rpeg_plan_soa_t;

typedef struct rpeg_engine_s rpeg_engine_t;

/* Creates an engine for one problem on the current HIP device.  Replaces the per-call construction
   of NodeCostModel / NodeMemoryModel / template graph in evaluate() (evaluate.py:261-287). */
int rpeg_engine_create(const rpeg_problem_t* problem, rpeg_engine_t** out);
void rpeg_engine_destroy(rpeg_engine_t* e);
const char* rpeg_last_error(const rpeg_engine_t* e);

/* Evaluates n plans: the batched form of Pool.map(_eval_worker, ...) (optimizer.py:793-798).
   makespan: Trace.makespan() (trace.py:31-38); peak: largest per-device peak in bytes
   (memory.py:608-841); score: throughput times the soft OOM penalty (evaluate.py:288, 396-401);
   mask: RPEG_MASK_* bits.  All four are device arrays of n elements; any may be NULL.
   `stream` is a hipStream_t (NULL = default stream).  The call waits for the host once, for the per-class totals
   of the batch (a few microseconds behind the kernel that writes the class ids), and again only where it must read
   back the list of new lowering classes; the evaluation kernels are left running on `stream`.  Successive calls on
   one engine use one stream, or the caller orders them. */
int rpeg_eval_batch(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags,
                    double* makespan, double* peak, double* score, uint8_t* mask, void* stream);

/* rpeg_eval_batch for callers that cannot allocate device memory.  It has no counterpart in the reference; it
   is there for callers that may not call hipMalloc: code under HIP graph capture, tight serving loops, harnesses
   that forbid allocation.  Same arguments, same results bit for bit.  Every intermediate of the call (the
   per-plan task list of the single-plan-per-wavefront kernel and a block of counters) lives in a file-scope
   device array of RPEG_STATIC_MAX_PLANS * 4 + 256 bytes that each GPU the library runs on holds until the
   process ends; the call makes no hipMalloc, hipFree or other allocating call.
     - n above RPEG_STATIC_MAX_PLANS is rejected with status -9.
     - The lowering classes of the plans must be on the device already, i.e. an earlier rpeg_eval_batch call
       of this engine has met them: status -10 when the engine's class tables are not on the device (no such
       call yet, or classes added since by rpeg_eval_host / rpeg_eval_trace), status -11 when plans of the
       batch belong to classes the engine has not met (those plans get NaN outputs and RPEG_MASK_ERROR, the
       others their results).  Problems with a class above 384 nodes are rejected with status -8.
     - All engines on one GPU share that GPU's array and it keeps the last call's contents; the call resets
       what must start at zero.  Calls that overlap on one GPU (two host threads, two streams) race.
   Without RPEG_NO_WAIT in `flags` the call returns after the results are in place: it copies one counter back and
   waits for the stream, which is how it knows of status -11.  With RPEG_NO_WAIT it only enqueues its three kernel
   launches on `stream` (a fill kernel, the class lookup, the evaluation) and returns 0: no copy, no wait and no
   memset node, so that the call may stand inside a HIP stream capture and the captured graph be replayed on the
   same buffers.  Plans of classes the engine has not met are then recognisable only by their outputs: NaN and
   RPEG_MASK_VALID | RPEG_MASK_ERROR in the mask. */
#define RPEG_STATIC_MAX_PLANS 32768
int rpeg_eval_batch_static(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags,
                           double* makespan, double* peak, double* score, uint8_t* mask, void* stream);

/* rpeg_eval_batch plus the critical-chain mass of every plan: what move_gen derives from (trace,
   lowered) of the current plan to bias its choice of vertex (_critical_chain and _critical_mass,
   RPEG/search/moves.py:590-642).  mass[i*RPEG_MAX_V + v] = summed finish - start of the operator nodes
   of vertex v on the chain that follows, from the first node of largest finish time backwards, the
   first predecessor of largest finish time; summed from the sink backwards (the reference sums in the
   iteration order of a set of string-hashed nodes, which differs between processes).  Device array of
   n*RPEG_MAX_V doubles. */
int rpeg_eval_batch_mass(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags,
                         double* makespan, double* peak, double* score, uint8_t* mask, double* mass, void* stream);

/* rpeg_eval_batch_mass for plans and results in HOST memory (any of the result pointers may be null).  This
   is what one step of the reference's search hands to its evaluation pool: a handful of candidate
   configurations held by the host (RPEG/search/optimizer.py:793-798, the `map` over `_eval_worker`; and
   every single call of evaluate / evaluate_cached, RPEG/search/evaluate.py:235-403).  For a batch of at most
   32 plans per compute unit the host computes the lowering class of each plan itself and the call is one
   copy to the device, one launch (one plan per wavefront) whose results land in pinned host memory, and one
   wait; larger batches are staged through device memory and take the path of rpeg_eval_batch.  Returns when
   the results are in place. */
int rpeg_eval_host(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                   double* peak, double* score, uint8_t* mask, double* mass, void* stream);

/* rpeg_eval_host with Trace.utilization() (RPEG/schedule/trace.py:53-101) of every plan as a further output,
   computed in the same launch from the schedule the kernel has just built: the mean over the devices that any
   node reserved of busy time / makespan, summed in the order in which the reference's trace first meets the
   devices, hence equal to the reference's number bit for bit (NaN for a plan with RPEG_MASK_ERROR or an
   invalid one).  This is the second factor of the utilisation objective of optimize() and polish()
   (RPEG/search/optimizer.py:461-486, 1021-1044), which then costs no launch of its own.  Any number of plans: one
   launch of a plan per wavefront for every 1,024 of them.  A problem with a class above 384 nodes does not fit that
   kernel: its batch takes the path of rpeg_eval_host and every plan is then traced on its own, as by
   rpeg_eval_trace_metrics (the same numbers, one launch per plan). */
int rpeg_eval_host_util(rpeg_engine_t* e, uint64_t n, const rpeg_plan_soa_t* plans, uint32_t flags, double* makespan,
                        double* peak, double* score, uint8_t* mask, double* utilization, void* stream);

/* Single-node durations and isolated peaks: the batched form of the candidate-directory loop
   (RPEG/search/moves.py:532-549): for strategy i, time = NodeCostModel.time(mock node) and
   peak = NodeMemoryModel.peak_bytes(mock node) of vertex `vertex` of structure `structure` placed at
   origin (0,0,0).  strat[(f)*stride + i], f = dp pp tp mb r_ext n_ext g_ext (int16, device). */
int rpeg_op_time_batch(rpeg_engine_t* e, uint64_t n, int32_t structure, int32_t vertex,
                       const int16_t* strat, uint64_t stride, double* time, double* peak, void* stream);

/* Start/finish time of every lowered node of ONE plan and the lowered graph itself (host arrays of
   capacity cap nodes / cap edges), in the reference's node and edge order: what evaluate() returns
   as (trace, lowered) (evaluate.py:290) and move_gen reads (moves.py:590-619).  vert_fields is one
   plan's RPEG_MAX_V*RPEG_FIELDS int16 values (stride 1), head4 its 4 header bytes.  node_kind:
   0 operator, 1 COMM, 2 RESHARD; node_vertex: the operator's vertex, or a transfer's destination
   vertex; node_src: a transfer's source vertex; node_sub: quantile phase or -1; edges: (src,dst)
   node index pairs; dispatch_index (may be NULL): position of the node in the scheduler's dispatch order,
   the insertion order of the reference's Trace.start (scheduler.py:517-518); node_reserved (may be NULL):
   bit v set when the scheduler reserves the allocation of vertex v for the node
   (RPEG/passes/transfer_resources.py:18-148, Trace.reserved_allocations).  Returns the node count, or a
   negative status. */
int rpeg_eval_trace(rpeg_engine_t* e, const int16_t* vert_fields, const uint8_t* head4,
                    double* start, double* finish, int32_t* dispatch_index, int32_t* node_kind, int32_t* node_vertex,
                    int32_t* node_step, int32_t* node_sub, int32_t* node_src, int32_t* edges,
                    int32_t* n_edges, int32_t cap, uint8_t* node_reserved);

/* Trace.utilization() and Trace.n_active() of ONE plan (RPEG/schedule/trace.py:53-118): the plan is traced on
   the GPU as by rpeg_eval_trace, then the busy intervals are merged device by device on the host in the
   insertion order of the reference's dictionaries (nodes in dispatch order, a node's reserved allocations
   source first, devices rack-major), so the sum has the reference's rounding.  Either output may be NULL.
   The metric steers optimize() when max_throughput_loss > 0 (optimizer.py:461-486). */
int rpeg_eval_trace_metrics(rpeg_engine_t* e, const int16_t* vert_fields, const uint8_t* head4,
                            double* utilization, int32_t* n_active);

/* lower() of ONE plan (RPEG/passes/unroll.py:85-152 and RPEG/passes/lower.py:330-851), on the host: the lowered
   graph in the reference's node order (the insertion order of its `nodes` dict) and edge order (the append order
   of its `edges` list), as rpeg_eval_trace returns it, without evaluating anything.  Integer work only: it needs
   no engine and no GPU, and reads of `problem` only the structure tables, K_eval, the generation phases and the
   model parameter counts -- not the hardware record, the device space or the memory policy, which lower() is not
   given either (the plan is not checked against is_valid, as the reference's lower() does not check it).
   node_payload / node_ref as for rpeg_plan_detail.  Any output may be NULL.  Returns the node count; -7 when
   `cap` (nodes, and edges) is too small; -5 when the class cannot be lowered. */
int rpeg_lower_plan(const rpeg_problem_t* problem, const int16_t* vert_fields, const uint8_t* head4, int32_t* node_kind,
                    int32_t* node_vertex, int32_t* node_step, int32_t* node_sub, int32_t* node_src, int64_t* node_payload,
                    int32_t* node_ref, int32_t* edges, int32_t* n_edges, int32_t cap);

/* Per-node and per-device quantities of ONE plan, for the host objects behind the reference's own names
   (NodeCostModel.time(node), RPEG/model/cost.py:66-88; _device_peaks / mem_worst_violation / mem_feasible,
   RPEG/model/memory.py:608-887; ExecNode.payload_in_bytes and .label, RPEG/passes/lower.py:396-403, 523-567,
   711-724).  The plan is given as for rpeg_eval_trace; nodes are in the reference's node order.
     node_time[i]     NodeCostModel.time of node i (NaN where the reference would raise ZeroDivisionError)
     node_payload[i]  payload_in_bytes of a COMM / RESHARD node, 0 for an operator node
     node_ref[i]      what the node's label names: the index of the template's data edge (the container of that
                      edge) for an activation transfer, 16 + model for a weight transfer or reshard ("W_<model>"),
                      -1 for an operator node
     set_peak[M]      64 doubles: for a non-empty set M of template vertices (bit v = vertex v) whose allocations
                      all intersect, the peak in bytes of a device that lies in the allocations of exactly the
                      vertices of M (every such device has the same peak: _device_peaks groups the operator nodes
                      by device, memory.py:626-636); 0 for any other M.  Which devices exist, and in which order
                      the reference's dictionary holds them, is integer geometry the caller does.
   Any output may be NULL.  Returns the node count, or a negative status (-6: the plan breaks an integer rule of
   is_valid; -7: cap too small). */
int rpeg_plan_detail(rpeg_engine_t* e, const int16_t* vert_fields, const uint8_t* head4, double* node_time,
                     int64_t* node_payload, int32_t* node_ref, int32_t cap, double* set_peak);

/* Batched simulated annealing: n_chains independent Metropolis-Hastings chains of n_steps steps.  One
   step of a chain is one iteration of the inner loop of optimize() (RPEG/search/optimizer.py:702-930):
   with probability alpha_pair*min(1,T/T_init) a donor/receiver proposal (multi_move_pair,
   moves.py:845-950), else up to K_x single-vertex proposals (move_gen, moves.py:645-825); the
   candidates of ALL chains are evaluated in one rpeg_eval_batch_mass launch (the reference maps
   _eval_worker over one chain's candidates, optimizer.py:793-798); best of K, one acceptance test,
   restart from the chain's best elite plan at T_warm after stag_window consecutive rejections
   (optimizer.py:632-694, 932-936).  Draws come from a counter-based generator keyed by (seed, chain,
   step), not from MT19937.  Chain c uses staleness variant c % n_variants.  Host memory throughout. */
typedef struct rpeg_sa_params_s {
  int32_t n_chains, n_steps, K_x, T_max, K_elite, stag_window, restart_attempts;
  int32_t gate_candidates;    /* 1: apply the stale-layout gate to candidates too (evaluate_cached);
                                 0: as _eval_worker, which the reference uses for candidates        */
  int32_t geometric_cooling;  /* OptimizerConfig.geometric_cooling (optimizer.py:77)                 */
  int32_t structure, split, n_variants;
  uint8_t tau[8][2];          /* staleness of the (up to 2) trainable models per variant             */
  double T_init, T_warm, T_min, T_cool, alpha_pair, score_eps;
  uint64_t seed;
  int32_t dir_n[RPEG_MAX_V];  /* candidate directory (moves.py:464-551): entries per vertex ...      */
  const int16_t* dir[RPEG_MAX_V]; /* ... rows of dp pp tp r_ext n_ext mb, ascending by time          */
  double max_throughput_loss; /* rpeg_sa_optimize*: > 0 ranks by throughput x Trace.utilization() above the
                                 floor (1 - loss) x best throughput so far, and by throughput x 1e-12 below
                                 it (optimizer.py:461-486); every evaluated plan is then traced once more
                                 for its utilisation (rpeg_eval_trace_metrics).  rpeg_sa_run ignores it  */
  /* the ablation switches of OptimizerConfig (RPEG/search/optimizer.py:83-88, 404-410) */
  int32_t fixed_mb;           /* moves.py:155-156, 182-188: one micro-batch count per (dp, pp) wherever strategies
                                 are drawn (the candidate directory must be built under the same rule)           */
  int32_t uniform_vertex;     /* moves.py:157-158, 688: move_gen draws its vertex uniformly                       */
  int32_t hard_oom;           /* evaluate.py:392, 437: a plan that does not fit scores 0 instead of the soft penalty */
  int32_t timed;              /* bit 0: deadline_s holds; bit 1: deadline_struct_s holds                          */
  /* rpeg_sa_optimize*: OptimizerConfig.deadline and .deadline_per_struct (optimizer.py:78-82) as readings of the
     run's clock.  That clock is `clock` (seconds, any origin; tests drive it) or, when `clock` is null, the
     steady clock counted from the start of the call, so that the two fields are then seconds from the start.
     Once the clock reads deadline_s or more the search ends whatever the budgets: the clock is read before
     every iteration and after every evaluated batch, and the conditions are tested in the reference's order
     (deadline, E_max, the setting's share, E_struct; :703-720, 848-865).  With a deadline the time left is
     split evenly among the structural settings still to come, whatever deadline_struct_s says (:571-579);
     without one, deadline_struct_s bounds every setting alike.  rpeg_sa_run ignores these. */
  double deadline_s;
  double deadline_struct_s;
  double (*clock)(void* ctx);
  void* clock_ctx;
} rpeg_sa_params_t;

typedef struct rpeg_sa_result_s {   /* per-chain arrays of n_chains elements, any may be NULL */
  int16_t* best_plan;      /* [RPEG_MAX_V*RPEG_FIELDS] per chain: best feasible plan, else best plan   */
  double* best_score;
  int32_t* best_step;      /* step at which it was first seen (-1: the start plan)                    */
  double* best_time;       /* seconds from the start of the run until then                            */
  uint8_t* best_feasible;  /* 1 when best_* describe a memory-feasible plan                           */
  int16_t* cur_plan;
  double* cur_score;
  int32_t* restarts;
  int64_t* n_eval;
  uint8_t* dead;           /* chain stopped: no valid restart found                                   */
  uint8_t* log;            /* [n_chains][n_steps]: kind (0 single, 1 pair) | candidates << 1 |
                              verdict << 4 (0 none, 1 rejected, 2 accepted) | restart << 6            */
  double wall_s, eval_s;   /* whole run / time inside the batched evaluations                         */
  int64_t n_launch, n_plans;
} rpeg_sa_result_t;

int rpeg_sa_run(rpeg_engine_t* e, const rpeg_sa_params_t* params, const int16_t* base_plan,
                rpeg_sa_result_t* result, void* stream);

/* optimize() as the reference runs it (RPEG/search/optimizer.py:365-946), for the structure of
   `params`: the staleness variants one after the other, each a sequence of restarts of one chain on the
   continuous random stream (params->seed, stream_a, stream_b, stream_c); evaluation cache (hits cost no
   budget and are merged before fresh results, :775-861); budgets E_max / E_struct in cache misses; elites
   shared by the variants; warm restarts (:640-663).  The K_x candidates of an iteration are one batched
   evaluation (the reference maps _eval_worker over them, :793-798).  Variant 0 must be the staleness of
   the base configuration.  n_chains, n_steps, restart_attempts and gate_candidates of `params` are not
   used.  With the same generator the reference's optimize() evaluates the same plans in the same order
   and returns the same plan. */
typedef struct rpeg_sa_serial_result_s {
  int16_t best_plan[RPEG_MAX_V * RPEG_FIELDS];  /* best feasible plan, else best plan (optimizer.py:946)  */
  int32_t best_variant, best_feasible;
  double best_score;
  int64_t E;                 /* evaluations counted against the budget (cache misses)                   */
  int64_t n_draws;           /* random words consumed                                                    */
  int64_t n_uncounted;       /* evaluations made for is_valid only (no budget, no cache)                 */
  int16_t* eval_log;         /* optional: every plan evaluated as a cache miss, in order, eval_log_cap   */
  uint8_t* eval_log_variant; /*   rows of RPEG_MAX_V*RPEG_FIELDS values / their staleness variants       */
  int64_t eval_log_cap, n_eval_log;
  double wall_s;
  int32_t best_family;       /* family of best_plan (0 from rpeg_sa_optimize)                            */
  int32_t timed_out;         /* 1: the search ended at its wall-clock deadline                           */
  double* eval_log_score;    /* optional, eval_log_cap entries each: what the run's cache holds for the   */
  uint8_t* eval_log_feasible;/*   logged plan -- score and feasibility as evaluate_cached stores them for a */
  double* eval_log_util;     /*   current plan (stale-layout gate applied) or as the merge of fresh         */
                             /*   candidates stores them (optimizer.py:838), and Trace.utilization() when   */
                             /*   the utilisation objective is on; a caller can carry them into its own     */
                             /*   EvalCache, which polish() reads next (RPEG/pipeline.py:1549-1560)         */
} rpeg_sa_serial_result_t;

int rpeg_sa_optimize(rpeg_engine_t* e, const rpeg_sa_params_t* params, int32_t E_max, int32_t E_struct,
                     int32_t R_max, uint64_t stream_a, uint64_t stream_b, uint64_t stream_c,
                     const int16_t* base_plan, rpeg_sa_serial_result_t* result, void* stream);

/* The same loop over several structural families, one after the other, as optimize() walks
   Iter_inter_model_candidates (RPEG/search/inter_model.py:68-121, optimizer.py:541-628): the separate
   template with its staleness variants, then the AC-share template with its own.  (The intra-stage-fusion
   settings in between are not entered: that pass does not run upstream.)  A family is a template
   (params->structure), its staleness variants in the order they are walked (params->tau) and its candidate
   directory (params->dir); the annealing settings are those of family 0.  `base_plan` is a plan of family
   0's template with staleness `base_tau`; a family of another template starts from a random valid plan
   and is skipped when 50 draws find none (optimizer.py:596-626).
     score_scale      multiplies every score of the family before it is compared (1 - lambda_ac for
                      AC-share, optimizer.py:132-145); elites keep raw scores
     elite_family     families with the same number share their elites (optimizer.py:500-515)
     valid_structure  structure whose memory verdict is_valid() uses for this family's plans: the
                      reference checks restarts against the memory model of the base configuration
                      (optimizer.py:449-458, 596-616, 640-663), see rpeg_struct_t.mem_trainable; equal to
                      params->structure when the two models agree
   result->best_variant counts within result->best_family; eval_log_variant holds family * 8 + variant,
   and 255 for the base configuration when its staleness is not among family 0's variants. */
typedef struct rpeg_sa_family_s {
  const rpeg_sa_params_t* params;
  double score_scale;
  int32_t elite_family, valid_structure;
} rpeg_sa_family_t;

int rpeg_sa_optimize_families(rpeg_engine_t* e, int32_t n_families, const rpeg_sa_family_t* families,
                              const uint8_t base_tau[2], int32_t E_max, int32_t E_struct, int32_t R_max,
                              uint64_t stream_a, uint64_t stream_b, uint64_t stream_c, const int16_t* base_plan,
                              rpeg_sa_serial_result_t* result, void* stream);

/* One draw of the proposal kernels that the annealing loops run, for callers that drive the loop themselves
   (host arithmetic only, no launch).  what = 0: move_gen (RPEG/search/moves.py:645-826) for the plan `plan` with
   critical-chain masses `mass` (RPEG_MAX_V doubles, rpeg_eval_batch_mass) at temperature T: up to K_x plans of
   RPEG_MAX_V*RPEG_FIELDS values each into `out`; *fallback = 1 when the current strategy was not in the
   directory (moves.py:554-587).  what = 1: multi_move_pair (moves.py:845-1010): one plan or none.  what = 2:
   sample_expl_in_region (moves.py:202-296) for vertex `vertex` on racks [r_lo, r_hi): RPEG_FIELDS values or none.
   The draws are words *draws+1, ... of the stream (prm->seed, stream_a, stream_b, stream_c); *draws is advanced
   by the words used, so that successive calls continue one stream.  Of `prm` the structure, K_x, T_max, T_init,
   the directory and the ablation switches are read.  Returns the number of plans (rows) written, negative on
   bad arguments. */
int rpeg_sa_propose(rpeg_engine_t* e, const rpeg_sa_params_t* prm, int32_t what, uint64_t stream_a, uint64_t stream_b,
                    uint64_t stream_c, const int16_t* plan, const double* mass, double T, int32_t vertex, int32_t r_lo,
                    int32_t r_hi, int16_t* out, int64_t* draws, int32_t* fallback);

/* Counters of the last rpeg_eval_batch call: [0] lowering classes in the batch (the classes the engine knows
   when a small batch needed no layout on the host and was not counted by class), [1] classes lowered
   by this call, [2] wave tasks, [3] dynamic LDS bytes of the evaluation kernel, [4] workspace bytes,
   [5] plans per wavefront with LDS-resident state (0: state in the HBM workspace; 1: one plan per
   wavefront), [6] plans of a large batch that ran one per wavefront beside the main kernel (included
   in [2]), [7] wave tasks of the four-lanes-per-plan kernel (included in [2]). */
int rpeg_engine_stats(const rpeg_engine_t* e, uint64_t* out, int32_t n);

/* Host time of the last rpeg_eval_batch call that laid its batch out, in microseconds of the steady clock: [0] from
   the call to the end of the launches up to the wait (signature kernel, cost-model launch, hand-over of the class
   totals), [1] the wait for the class totals, [2] the layout of the batch and the split between the kernels,
   [3] tables up, scatter, fork, the scheduling launches, join and the launches that end the call.  A measurement aid with
   no counterpart in the reference. */
int rpeg_engine_host_us(const rpeg_engine_t* e, double* out, int32_t n);

/* Where the evaluation kernel keeps the scheduler state of a plan (ready time, rank and remaining
   in-degree per node, duration per slot).  lanes = 0: in an HBM workspace, 64 plans per wavefront (the
   throughput layout).  lanes = 8, 16, 32 or 64: in LDS, that many plans per wavefront (the latency
   layout: a batch too small to fill the chip finishes sooner); fails at the next call when the state
   of the problem's largest class does not fit.  lanes = 1: one plan per wavefront, its nodes spread
   over the lanes (the layout of lowest latency, for batches of a few thousand plans at most; classes of
   up to 384 nodes).  lanes = 4: four lanes per plan, sixteen plans per wavefront, the ready entries (at most 32
   at once; a plan with more is redone by the launch that ends the call) in the registers of the four lanes (the
   layout for dense graphs, whose plan-per-lane wavefronts end last).
   lanes = -1 (default): chosen per batch from its size.
   Results do not depend on the setting. */
int rpeg_engine_set_state_lanes(rpeg_engine_t* e, int32_t lanes);

/* The nine fitted figures by which a full batch is split between the three scheduling kernels (microseconds of a
   wavefront on an MI355X): cost of a plan in the one-plan-per-wavefront kernel a + b x nodes (40, 2.2); of a wavefront
   of the four-lanes-per-plan kernel a + nodes x (b + c x heap pops per dispatch) (40, 1.6, 0.45); the share of the
   modelled room that the former really gets beside the latter (0.65); how much later a class must end in the main
   kernel to move to the four-lanes-per-plan kernel (1.15); the modelled gain that a split by class size (0.97) and by
   measured time (0.98) must reach.  A measurement aid: the figures decide where a plan is evaluated, never what
   the result is.  No counterpart in the reference. */
int rpeg_engine_set_split_model(rpeg_engine_t* e, const double* values, int32_t n);

/* rpeg_sa_run deals its chains to `groups` groups (1..8, default 2; never fewer than 8 chains per group) that take
   their steps in turn, each with a stream and staging buffers of its own: while the proposals of one group are being
   evaluated, the host merges the results of another and draws its next proposals.  A chain's draws are keyed by
   (seed, chain, step) and its decisions depend on its own evaluations only, so the result of a run does not depend
   on the number of groups (the reference steps its chains one after the other, optimizer.py:683-786; it has no
   counterpart of this setting). */
int rpeg_engine_set_sa_groups(rpeg_engine_t* e, int32_t groups);

/* on = 1 (default): in a full batched call the cost-model launch, the layout of the batch and the main scheduling
   kernel follow each other on the device's second side stream, from the moment the class ids are written, while the
   caller's stream hands the class totals to the host -- unless another engine of the process is in the middle of a
   call on the side streams.  on = 0: all of it on the caller's stream.  A measurement aid: results do not depend on
   it.  No counterpart in the reference. */
int rpeg_engine_set_side_layout(rpeg_engine_t* e, int32_t on);

/* With lanes = -1 and a batch that fills the chip in one round of wavefronts: the largest share of the batch's
   plans, in percent, that the four-lanes-per-plan kernel may take on a stream of its own (default 25; 0: none).
   Which classes it takes is learned: the main kernel records, per class, how long its slowest wavefront ran and how
   many heap pops per dispatch it needed, and from the second call on the classes that would end last there (dense
   graphs) are moved.  Results do not depend on the setting.  No reference counterpart (a tuning knob). */
int rpeg_engine_set_quad_share(rpeg_engine_t* e, int32_t percent);

/* Ready-list entries per plan in the main kernel: 8, 16, 24 or 32 (default).  A plan with that many nodes
   ready at once is redone, without a bound, by the launch that ends the call (one plan per lane, its state and
   ready list in HBM: slow, and rare -- the longest list seen on the shipped problems is 24).  Fewer entries take
   less LDS per wavefront.  The kernel that runs one plan per wavefront (small batches) keeps its ready set in
   registers and has no such bound.  Results do not depend on the setting.  No reference counterpart: tests use
   it to reach the redo path. */
int rpeg_engine_set_ready_cap(rpeg_engine_t* e, int32_t entries);

/* Forgets every lowered class, so that the next rpeg_eval_batch lowers all the classes of its batch
   again (used to measure a cold call). */
int rpeg_engine_reset_classes(rpeg_engine_t* e);

/* Kernel time of the dominant kernel in the last rpeg_eval_batch call, measured with HIP events on
   the launch stream (milliseconds); negative when timing was not enabled. */
int rpeg_engine_set_timing(rpeg_engine_t* e, int32_t enabled);
double rpeg_engine_last_kernel_ms(const rpeg_engine_t* e);

/* Development aid: per-wavefront phase clocks of the evaluation kernel.  enable != 0 makes the following
   rpeg_eval_batch calls record, per wavefront, seven stamps of the 100 MHz wall clock (start; after the
   plan load; durations; memory model; ranks; scheduling; outputs) and in the eighth word the node count
   << 32 | heap pops; with `out` non-NULL the stamps of the last call (8 words per wavefront, at most
   cap_waves wavefronts) are copied to host memory and their number is returned. */
int rpeg_engine_profile(rpeg_engine_t* e, int32_t enable, unsigned long long* out, uint64_t cap_waves);

/* exp() as the host C library of an FMA-capable x86-64 computes it, evaluated on the device for n
   inputs; exported for the parity test of the OOM penalty. */
int rpeg_device_exp(rpeg_engine_t* e, uint64_t n, const double* x, double* y, void* stream);

#ifdef __cplusplus
}
#endif
#endif
