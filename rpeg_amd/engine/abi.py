"""ctypes mirror of include/rpeg_eval.h (struct layouts and constants of the C ABI)."""

import ctypes as C

ABI_VERSION = 4
MAX_V, MAX_E, MAX_PUB, MAX_PAIR, MAX_REL, MAX_PH, MAX_SPLIT, MAX_MODEL, MAX_STRUCT = 6, 9, 2, 4, 13, 6, 7, 5, 3
FIELDS = 10
ROLE = {"GEN": 0, "INF": 1, "TRAIN": 2}
MODEL = {"Pi": 0, "V": 1, "Ref": 2, "R": 3, "AC": 4}
NEED_DISJ, NEED_PI = 1, 2
MASK_VALID, MASK_STALE_OK, MASK_MEM_OK, MASK_ERROR, MASK_LIMIT = 1, 2, 4, 8, 16
GATE_STALE = 1
NO_WAIT = 2
STATIC_MAX_PLANS = 32768
HW_FIELDS = (
    "flops_per_gpu", "memory_per_gpu", "memory_bandwidth",
    "alpha_coll_g", "beta_coll_g", "alpha_coll_n", "beta_coll_n", "alpha_coll_r", "beta_coll_r",
    "alpha_p2p_g", "beta_p2p_g", "alpha_p2p_n", "beta_p2p_n", "alpha_p2p_r", "beta_p2p_r",
    "gemm_m_half", "gemm_k_half", "decode_bw_eff", "non_gemm_constant", "non_gemm_scaling", "non_gemm_batch_cal",
    "op_generation_scale", "op_inference_scale", "op_training_scale", "activation_comm_overhead_s",
    "weight_comm_scale", "reshard_scale")


class ModelT(C.Structure):
    _fields_ = [("L", C.c_int32), ("d", C.c_int32), ("d_ff", C.c_int32), ("V", C.c_int32), ("sb", C.c_int32),
                ("kind", C.c_int32), ("w_layer", C.c_int64), ("params_formula", C.c_int64), ("n_params", C.c_int64)]


class OpConstT(C.Structure):
    _fields_ = [("W", C.c_double), ("W_prefill", C.c_double), ("avg_past", C.c_double), ("n_eff", C.c_int32),
                ("steps", C.c_int32), ("prefill", C.c_int32), ("sub", C.c_int32)]


class VertexT(C.Structure):
    _fields_ = [("role", C.c_int32), ("model", C.c_int32), ("topo_idx", C.c_int32), ("tau_slot", C.c_int32),
                ("unsplit", OpConstT), ("sub", (OpConstT * MAX_PH) * MAX_SPLIT)]


class EdgeT(C.Structure):
    _fields_ = [("src", C.c_int32), ("dst", C.c_int32), ("is_weight", C.c_int32), ("gen_inf", C.c_int32),
                ("full_bytes", C.c_int64), ("sub_bytes", (C.c_int64 * MAX_PH) * MAX_SPLIT)]


class PubT(C.Structure):
    _fields_ = [("src", C.c_int32), ("dst", C.c_int32), ("model", C.c_int32), ("tau_slot", C.c_int32)]


class PairT(C.Structure):
    _fields_ = [("u", C.c_int32), ("v", C.c_int32), ("model", C.c_int32), ("tau_slot", C.c_int32),
                ("reach", C.c_int32), ("pad", C.c_int32)]


class RelT(C.Structure):
    _fields_ = [("u", C.c_int32), ("v", C.c_int32), ("flags", C.c_int32), ("pad", C.c_int32)]


class StructT(C.Structure):
    _fields_ = [("n_vertex", C.c_int32), ("n_edge", C.c_int32), ("n_pub", C.c_int32), ("n_pair", C.c_int32),
                ("n_rel", C.c_int32), ("n_tau", C.c_int32),
                ("vertex", VertexT * MAX_V), ("edge", EdgeT * MAX_E), ("pub", PubT * MAX_PUB),
                ("pair", PairT * MAX_PAIR), ("rel", RelT * MAX_REL),
                ("reach", (C.c_uint8 * MAX_V) * MAX_V), ("trainable", C.c_uint8 * (MAX_MODEL + 3)),
                ("mem_trainable", C.c_uint8 * (MAX_MODEL + 3))]


class PhaseT(C.Structure):
    _fields_ = [("n_active", C.c_int32), ("n_seqs", C.c_int32), ("steps", C.c_int32), ("t_start", C.c_int32),
                ("prefill", C.c_int32), ("pad", C.c_int32)]


class ProblemT(C.Structure):
    _fields_ = [("abi_version", C.c_int32), ("n_struct", C.c_int32), ("n_split", C.c_int32), ("K_eval", C.c_int32),
                ("R", C.c_int32), ("N", C.c_int32), ("G", C.c_int32),
                ("B", C.c_int32), ("K", C.c_int32), ("S", C.c_int32), ("T", C.c_int32),
                ("optimizer_stage", C.c_int32), ("ckpt", C.c_int32), ("max_groups", C.c_int32),
                ("n_phase", C.c_int32 * MAX_SPLIT), ("transfer_both", C.c_int32),
                ("phase", (PhaseT * MAX_PH) * MAX_SPLIT),
                ("hw", C.c_double * len(HW_FIELDS)),
                ("cap", C.c_double), ("group_overhead", C.c_double), ("score_num", C.c_double),
                ("model", ModelT * MAX_MODEL), ("st", StructT * MAX_STRUCT)]


class PlanSoaT(C.Structure):
    _fields_ = [("vert", C.c_void_p), ("head", C.c_void_p), ("stride", C.c_uint64)]


class SaParamsT(C.Structure):
    _fields_ = [("n_chains", C.c_int32), ("n_steps", C.c_int32), ("K_x", C.c_int32), ("T_max", C.c_int32),
                ("K_elite", C.c_int32), ("stag_window", C.c_int32), ("restart_attempts", C.c_int32),
                ("gate_candidates", C.c_int32), ("geometric_cooling", C.c_int32),
                ("structure", C.c_int32), ("split", C.c_int32), ("n_variants", C.c_int32),
                ("tau", (C.c_uint8 * 2) * 8),
                ("T_init", C.c_double), ("T_warm", C.c_double), ("T_min", C.c_double), ("T_cool", C.c_double),
                ("alpha_pair", C.c_double), ("score_eps", C.c_double),
                ("seed", C.c_uint64),
                ("dir_n", C.c_int32 * MAX_V), ("dir", C.c_void_p * MAX_V), ("max_throughput_loss", C.c_double),
                ("fixed_mb", C.c_int32), ("uniform_vertex", C.c_int32), ("hard_oom", C.c_int32), ("timed", C.c_int32),
                ("deadline_s", C.c_double), ("deadline_struct_s", C.c_double), ("clock", C.c_void_p),
                ("clock_ctx", C.c_void_p)]


CLOCK_FN = C.CFUNCTYPE(C.c_double, C.c_void_p)   # rpeg_sa_params_t.clock


class SaResultT(C.Structure):
    _fields_ = [("best_plan", C.c_void_p), ("best_score", C.c_void_p), ("best_step", C.c_void_p),
                ("best_time", C.c_void_p), ("best_feasible", C.c_void_p), ("cur_plan", C.c_void_p),
                ("cur_score", C.c_void_p), ("restarts", C.c_void_p), ("n_eval", C.c_void_p), ("dead", C.c_void_p),
                ("log", C.c_void_p), ("wall_s", C.c_double), ("eval_s", C.c_double),
                ("n_launch", C.c_int64), ("n_plans", C.c_int64)]


class SaSerialResultT(C.Structure):
    _fields_ = [("best_plan", C.c_int16 * (MAX_V * FIELDS)), ("best_variant", C.c_int32), ("best_feasible", C.c_int32),
                ("best_score", C.c_double), ("E", C.c_int64), ("n_draws", C.c_int64), ("n_uncounted", C.c_int64),
                ("eval_log", C.c_void_p), ("eval_log_variant", C.c_void_p), ("eval_log_cap", C.c_int64),
                ("n_eval_log", C.c_int64), ("wall_s", C.c_double), ("best_family", C.c_int32), ("timed_out", C.c_int32),
                ("eval_log_score", C.c_void_p), ("eval_log_feasible", C.c_void_p), ("eval_log_util", C.c_void_p)]


class SaFamilyT(C.Structure):
    _fields_ = [("params", C.c_void_p), ("score_scale", C.c_double), ("elite_family", C.c_int32),
                ("valid_structure", C.c_int32)]
