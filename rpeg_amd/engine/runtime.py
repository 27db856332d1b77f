"""ctypes binding of librpeg_eval.so and the `Engine` host object.

PyTorch is used only to own device buffers and to name the current HIP stream; every number is
produced by the HIP kernels behind the C ABI (include/rpeg_eval.h).  There is no CPU fallback: a
missing library or a missing GPU raises.
"""

from __future__ import annotations

import ctypes as C
import os
from typing import Dict, Optional

import numpy as np

from . import abi
from .compile import compile_problem
from .problem import EvalProblem, PlanBatch

_LIB_PATH = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "librpeg_eval.so")
_lib = None

EXPORTS = ("rpeg_engine_create", "rpeg_engine_destroy", "rpeg_last_error", "rpeg_eval_batch",
           "rpeg_op_time_batch", "rpeg_eval_trace", "rpeg_engine_stats", "rpeg_engine_set_timing",
           "rpeg_engine_last_kernel_ms", "rpeg_device_exp", "rpeg_engine_reset_classes", "rpeg_eval_batch_mass",
           "rpeg_sa_run", "rpeg_sa_propose", "rpeg_eval_host_util", "rpeg_engine_set_state_lanes", "rpeg_engine_set_sa_groups", "rpeg_engine_set_side_layout", "rpeg_engine_host_us", "rpeg_engine_set_split_model", "rpeg_engine_set_quad_share", "rpeg_engine_set_ready_cap", "rpeg_engine_profile", "rpeg_sa_optimize", "rpeg_eval_host",
           "rpeg_sa_optimize_families", "rpeg_eval_trace_metrics", "rpeg_eval_batch_static", "rpeg_plan_detail",
           "rpeg_lower_plan")


class EngineError(RuntimeError):
    pass


def load_library(path: Optional[str] = None):
    """Loads the in-tree shared library (built by rpeg_amd/build.py); raises if it is absent."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or _LIB_PATH
    if not os.path.exists(p):
        raise EngineError(f"{p} is missing: build it with `python -m rpeg_amd.build` (hipcc, gfx950)")
    # torch first: it brings its own HIP runtime, and the library must bind to that copy -- loaded the other way
    # round the process holds a runtime that sees no device (rpeg_engine_create then fails with status -4)
    import torch  # noqa: F401
    lib = C.CDLL(p)
    vp, u64, u32, i32 = C.c_void_p, C.c_uint64, C.c_uint32, C.c_int32
    lib.rpeg_engine_create.restype = C.c_int
    lib.rpeg_engine_create.argtypes = [vp, C.POINTER(vp)]
    lib.rpeg_engine_destroy.restype = None
    lib.rpeg_engine_destroy.argtypes = [vp]
    lib.rpeg_last_error.restype = C.c_char_p
    lib.rpeg_last_error.argtypes = [vp]
    lib.rpeg_eval_batch.restype = C.c_int
    lib.rpeg_eval_batch.argtypes = [vp, u64, vp, u32, vp, vp, vp, vp, vp]
    lib.rpeg_eval_batch_static.restype = C.c_int
    lib.rpeg_eval_batch_static.argtypes = [vp, u64, vp, u32, vp, vp, vp, vp, vp]
    lib.rpeg_eval_batch_mass.restype = C.c_int
    lib.rpeg_eval_batch_mass.argtypes = [vp, u64, vp, u32, vp, vp, vp, vp, vp, vp]
    lib.rpeg_eval_host.restype = C.c_int
    lib.rpeg_eval_host.argtypes = [vp, u64, vp, u32, vp, vp, vp, vp, vp, vp]
    lib.rpeg_sa_run.restype = C.c_int
    lib.rpeg_sa_run.argtypes = [vp, vp, vp, vp, vp]
    lib.rpeg_sa_optimize.restype = C.c_int
    lib.rpeg_sa_optimize.argtypes = [vp, vp, i32, i32, i32, u64, u64, u64, vp, vp, vp]
    lib.rpeg_sa_optimize_families.restype = C.c_int
    lib.rpeg_sa_optimize_families.argtypes = [vp, i32, vp, vp, i32, i32, i32, u64, u64, u64, vp, vp, vp]
    lib.rpeg_op_time_batch.restype = C.c_int
    lib.rpeg_op_time_batch.argtypes = [vp, u64, i32, i32, vp, u64, vp, vp, vp]
    lib.rpeg_eval_trace.restype = C.c_int
    lib.rpeg_eval_trace.argtypes = [vp] * 13 + [i32, vp]
    lib.rpeg_eval_trace_metrics.restype = C.c_int
    lib.rpeg_eval_trace_metrics.argtypes = [vp] * 5
    lib.rpeg_lower_plan.restype = C.c_int
    lib.rpeg_lower_plan.argtypes = [vp] * 12 + [i32]
    lib.rpeg_plan_detail.restype = C.c_int
    lib.rpeg_plan_detail.argtypes = [vp, vp, vp, vp, vp, vp, i32, vp]
    lib.rpeg_engine_stats.restype = C.c_int
    lib.rpeg_engine_stats.argtypes = [vp, vp, i32]
    lib.rpeg_engine_set_timing.restype = C.c_int
    lib.rpeg_engine_set_timing.argtypes = [vp, i32]
    lib.rpeg_engine_last_kernel_ms.restype = C.c_double
    lib.rpeg_engine_last_kernel_ms.argtypes = [vp]
    lib.rpeg_engine_set_state_lanes.restype = C.c_int
    lib.rpeg_engine_set_state_lanes.argtypes = [vp, i32]
    lib.rpeg_engine_host_us.restype = C.c_int
    lib.rpeg_engine_host_us.argtypes = [vp, vp, i32]
    lib.rpeg_engine_set_split_model.restype = C.c_int
    lib.rpeg_engine_set_split_model.argtypes = [vp, vp, i32]
    lib.rpeg_engine_set_sa_groups.restype = C.c_int
    lib.rpeg_engine_set_sa_groups.argtypes = [vp, i32]
    lib.rpeg_engine_set_side_layout.restype = C.c_int
    lib.rpeg_engine_set_side_layout.argtypes = [vp, i32]
    lib.rpeg_engine_set_quad_share.restype = C.c_int
    lib.rpeg_engine_set_quad_share.argtypes = [vp, i32]
    lib.rpeg_engine_set_ready_cap.restype = C.c_int
    lib.rpeg_engine_set_ready_cap.argtypes = [vp, i32]
    lib.rpeg_engine_reset_classes.restype = C.c_int
    lib.rpeg_engine_reset_classes.argtypes = [vp]
    lib.rpeg_engine_profile.restype = C.c_int
    lib.rpeg_engine_profile.argtypes = [vp, i32, vp, u64]
    lib.rpeg_eval_host_util.restype = C.c_int
    lib.rpeg_eval_host_util.argtypes = [vp, u64, vp, u32, vp, vp, vp, vp, vp, vp]
    lib.rpeg_sa_propose.restype = C.c_int
    lib.rpeg_sa_propose.argtypes = [vp, vp, i32, u64, u64, u64, vp, vp, C.c_double, i32, i32, i32, vp, vp, vp]
    lib.rpeg_device_exp.restype = C.c_int
    lib.rpeg_device_exp.argtypes = [vp, u64, vp, vp, vp]
    if path is None:
        _lib = lib
    return lib


def set_directory(params: "abi.SaParamsT", directory):
    """Points params.dir at per-vertex int16 arrays [n, 6]; returns the arrays (keep them alive)."""
    keep = []
    for v in range(abi.MAX_V):
        if v < len(directory):
            a = np.ascontiguousarray(directory[v], dtype=np.int16).reshape(-1, 6)
            keep.append(a)
            params.dir_n[v] = a.shape[0]
            params.dir[v] = a.ctypes.data
        else:
            params.dir_n[v] = 0
            params.dir[v] = None
    return keep


def family_array(families):
    """rpeg_sa_family_t[] from [(params, directory, score_scale, elite_family, valid_structure)]; returns
    (array, objects to keep alive)."""
    arr = (abi.SaFamilyT * len(families))()
    keep = []
    for f, (params, directory, scale, elite_family, valid_structure) in enumerate(families):
        keep.append((params, set_directory(params, directory)))
        arr[f].params = C.addressof(params)
        arr[f].score_scale = float(scale)
        arr[f].elite_family = int(elite_family)
        arr[f].valid_structure = int(params.structure if valid_structure is None else valid_structure)
    return arr, keep


def serial_result(log_cap: int):
    res = abi.SaSerialResultT()
    log = np.zeros((max(log_cap, 1), abi.MAX_V * abi.FIELDS), np.int16)
    logv = np.zeros(max(log_cap, 1), np.uint8)
    res.eval_log, res.eval_log_variant, res.eval_log_cap = log.ctypes.data, logv.ctypes.data, log_cap
    stored = (np.zeros(max(log_cap, 1)), np.zeros(max(log_cap, 1), np.uint8), np.zeros(max(log_cap, 1)))
    res.eval_log_score, res.eval_log_feasible, res.eval_log_util = (a.ctypes.data for a in stored)
    res._stored = stored     # kept alive with the record
    return res, log, logv


def serial_dict(res, log, logv):
    n = min(res.n_eval_log, res.eval_log_cap)
    return dict(best_plan=np.array(res.best_plan, dtype=np.int16), best_variant=res.best_variant,
                best_feasible=bool(res.best_feasible), best_score=res.best_score, E=res.E, n_draws=res.n_draws,
                best_family=res.best_family, n_uncounted=res.n_uncounted, n_eval_log=res.n_eval_log, eval_log=log[:n].copy(),
                eval_log_variant=logv[:n].copy(), eval_log_score=res._stored[0][:n].copy(),
                eval_log_feasible=res._stored[1][:n].astype(bool), eval_log_util=res._stored[2][:n].copy(),
                wall_s=res.wall_s, timed_out=bool(res.timed_out))


def _torch():
    import torch
    if not torch.cuda.is_available():
        raise EngineError("no HIP device is visible; the evaluator has no CPU path")
    return torch


class DeviceBatch:
    """Plan tensors resident in device memory (what rpeg_plan_soa_t points at)."""

    def __init__(self, batch: PlanBatch, device="cuda:0"):
        torch = _torch()
        self.n = batch.n
        self.vert = torch.from_numpy(np.ascontiguousarray(batch.vert)).to(device)
        self.head = torch.from_numpy(np.ascontiguousarray(batch.head)).to(device)
        self.soa = abi.PlanSoaT(self.vert.data_ptr(), self.head.data_ptr(), self.vert.shape[1])


class Engine:
    """One compiled problem on one GPU.  Not thread-safe; use one engine per host thread."""

    def __init__(self, problem: EvalProblem, device: str = "cuda:0"):
        torch = _torch()
        self.lib = load_library()
        self.problem = problem
        self.device = torch.device(device)
        self.P = compile_problem(problem)
        self._h = C.c_void_p()
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_engine_create(C.addressof(self.P), C.byref(self._h))
        if rc != 0:
            raise EngineError(f"rpeg_engine_create failed with status {rc}")

    def close(self):
        if getattr(self, "_h", None) and self._h.value:
            self.lib.rpeg_engine_destroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def _check(self, rc: int, what: str):
        if rc < 0:
            raise EngineError(f"{what} failed ({rc}): {self.lib.rpeg_last_error(self._h).decode()}")

    def set_timing(self, on: bool):
        self.lib.rpeg_engine_set_timing(self._h, int(on))

    def set_state_lanes(self, lanes: int):
        """-1 automatic; 0 scheduler state in HBM (64 plans per wavefront); 8/16/32/64 state in LDS; 1 a plan per
        wavefront; 4 four lanes per plan."""
        self._check(self.lib.rpeg_engine_set_state_lanes(self._h, int(lanes)), "rpeg_engine_set_state_lanes")

    def host_us(self) -> Dict[str, float]:
        """Host time of the last laid-out `eval_device` call, microseconds (rpeg_engine_host_us)."""
        v = np.zeros(4)
        self._check(self.lib.rpeg_engine_host_us(self._h, v.ctypes.data, 4), "rpeg_engine_host_us")
        return dict(launch_gate=float(v[0]), wait_counts=float(v[1]), layout_and_split=float(v[2]), launch_schedulers=float(v[3]))

    def set_split_model(self, values):
        """The nine fitted figures of the split between the scheduling kernels (rpeg_engine_set_split_model)."""
        v = np.ascontiguousarray(values, dtype=np.float64)
        self._check(self.lib.rpeg_engine_set_split_model(self._h, v.ctypes.data, len(v)), "rpeg_engine_set_split_model")

    def set_sa_groups(self, groups: int):
        """Groups of chains (1..8) whose evaluations overlap the host's work on the others in `sa_run`."""
        self._check(self.lib.rpeg_engine_set_sa_groups(self._h, int(groups)), "rpeg_engine_set_sa_groups")

    def set_side_layout(self, on: bool):
        """Cost-model launch, layout and main kernel of a full batch on a side stream (default) or on the caller's."""
        self._check(self.lib.rpeg_engine_set_side_layout(self._h, 1 if on else 0), "rpeg_engine_set_side_layout")

    def set_quad_share(self, percent: int):
        """Percentage of a full batch that the four-lanes-per-plan kernel takes beside the main kernel (0: none)."""
        self._check(self.lib.rpeg_engine_set_quad_share(self._h, int(percent)), "rpeg_engine_set_quad_share")

    def set_ready_cap(self, entries: int):
        """Ready-list entries per plan in the main kernel (8, 16, 24 or 32); plans that need more are redone by the
        launch that ends the call, without a bound."""
        self._check(self.lib.rpeg_engine_set_ready_cap(self._h, int(entries)), "rpeg_engine_set_ready_cap")

    def reset_classes(self):
        self.lib.rpeg_engine_reset_classes(self._h)

    def last_kernel_ms(self) -> float:
        return float(self.lib.rpeg_engine_last_kernel_ms(self._h))

    def stats(self) -> Dict[str, int]:
        buf = (C.c_uint64 * 8)()
        self.lib.rpeg_engine_stats(self._h, buf, 8)
        return dict(classes=buf[0], classes_lowered=buf[1], wave_tasks=buf[2], lds_bytes=buf[3], workspace_bytes=buf[4],
                    state_lanes=buf[5], single_plan_tasks=buf[6], quad_tasks=buf[7])

    def alloc_outputs(self, n: int):
        torch = _torch()
        return dict(makespan=torch.empty(n, dtype=torch.float64, device=self.device),
                    peak=torch.empty(n, dtype=torch.float64, device=self.device),
                    score=torch.empty(n, dtype=torch.float64, device=self.device),
                    mask=torch.empty(n, dtype=torch.uint8, device=self.device))

    def eval_device(self, dbatch: DeviceBatch, out=None, gate_stale: bool = True, n: Optional[int] = None):
        """Evaluates plans already resident on the device into device outputs (no host copies of
        plan data or results)."""
        torch = _torch()
        n = dbatch.n if n is None else n
        out = out or self.alloc_outputs(n)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_eval_batch(self._h, n, C.addressof(dbatch.soa), abi.GATE_STALE if gate_stale else 0,
                                          out["makespan"].data_ptr(), out["peak"].data_ptr(), out["score"].data_ptr(),
                                          out["mask"].data_ptr(), stream)
        self._check(rc, "rpeg_eval_batch")
        return out

    def eval_device_static(self, dbatch: DeviceBatch, out=None, gate_stale: bool = True, n: Optional[int] = None,
                           no_wait: bool = False):
        """eval_device through the entry point that allocates nothing (rpeg_eval_batch_static): at most
        abi.STATIC_MAX_PLANS plans whose lowering classes an earlier eval_device call has met.  `out` must be
        given by a caller that may not allocate.  `no_wait`: only enqueue (RPEG_NO_WAIT), as a caller under HIP
        stream capture needs it."""
        torch = _torch()
        n = dbatch.n if n is None else n
        out = out or self.alloc_outputs(n)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_eval_batch_static(self._h, n, C.addressof(dbatch.soa),
                                                 (abi.GATE_STALE if gate_stale else 0) | (abi.NO_WAIT if no_wait else 0),
                                                 out["makespan"].data_ptr(), out["peak"].data_ptr(),
                                                 out["score"].data_ptr(), out["mask"].data_ptr(), stream)
        self._check(rc, "rpeg_eval_batch_static")
        return out

    def eval(self, batch: PlanBatch, gate_stale: bool = True, mass: bool = False) -> Dict[str, np.ndarray]:
        """Plans and results in host memory (rpeg_eval_host): a batch of up to a few thousand plans is one
        copy, one launch and one wait; larger ones are staged through device memory by the library."""
        torch = _torch()
        n = batch.n
        vert = np.ascontiguousarray(batch.vert, dtype=np.int16)
        head = np.ascontiguousarray(batch.head, dtype=np.uint8)
        soa = abi.PlanSoaT(vert.ctypes.data, head.ctypes.data, vert.shape[1])
        out = dict(makespan=np.empty(n, np.float64), peak=np.empty(n, np.float64), score=np.empty(n, np.float64),
                   mask=np.empty(n, np.uint8))
        if mass:
            out["mass"] = np.empty((n, abi.MAX_V), np.float64)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_eval_host(self._h, n, C.addressof(soa), abi.GATE_STALE if gate_stale else 0,
                                         out["makespan"].ctypes.data, out["peak"].ctypes.data, out["score"].ctypes.data,
                                         out["mask"].ctypes.data, out["mass"].ctypes.data if mass else None, stream)
        self._check(rc, "rpeg_eval_host")
        return out

    def eval_util(self, batch: PlanBatch, gate_stale: bool = False) -> Dict[str, np.ndarray]:
        """`eval` plus Trace.utilization() of every plan from the same launches (rpeg_eval_host_util): the dict of
        `eval` with "util", float64 [n]."""
        torch = _torch()
        n = batch.n
        out = dict(makespan=np.empty(n), peak=np.empty(n), score=np.empty(n), mask=np.empty(n, np.uint8), util=np.empty(n))
        if n == 0:
            return out
        vert, head = np.ascontiguousarray(batch.vert), np.ascontiguousarray(batch.head)
        soa = abi.PlanSoaT(vert.ctypes.data, head.ctypes.data, vert.shape[1])
        stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_eval_host_util(self._h, n, C.addressof(soa), abi.GATE_STALE if gate_stale else 0,
                                              out["makespan"].ctypes.data, out["peak"].ctypes.data, out["score"].ctypes.data,
                                              out["mask"].ctypes.data, out["util"].ctypes.data, stream)
        self._check(rc, "rpeg_eval_host_util")
        return out

    def eval_mass(self, batch: PlanBatch, gate_stale: bool = False) -> Dict[str, np.ndarray]:
        """`eval` plus the critical-chain mass per template vertex, float64 [n, MAX_V]."""
        return self.eval(batch, gate_stale=gate_stale, mass=True)

    def eval_mass_device(self, batch: PlanBatch, gate_stale: bool = False) -> Dict[str, np.ndarray]:
        """The same through device tensors (rpeg_eval_batch_mass)."""
        torch = _torch()
        db = DeviceBatch(batch, self.device)
        out = self.alloc_outputs(db.n)
        out["mass"] = torch.empty((db.n, abi.MAX_V), dtype=torch.float64, device=self.device)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_eval_batch_mass(self._h, db.n, C.addressof(db.soa), abi.GATE_STALE if gate_stale else 0,
                                               out["makespan"].data_ptr(), out["peak"].data_ptr(),
                                               out["score"].data_ptr(), out["mask"].data_ptr(),
                                               out["mass"].data_ptr(), stream)
        self._check(rc, "rpeg_eval_batch_mass")
        torch.cuda.synchronize(self.device)
        return {k: v.cpu().numpy() for k, v in out.items()}

    def eval_resident(self, batch: PlanBatch, gate_stale: bool = True) -> Dict[str, np.ndarray]:
        """Upload with torch, evaluate device tensors (rpeg_eval_batch), download."""
        out = self.eval_device(DeviceBatch(batch, self.device), gate_stale=gate_stale)
        _torch().cuda.synchronize(self.device)
        return {k: v.cpu().numpy() for k, v in out.items()}

    def sa_run(self, params: "abi.SaParamsT", directory, base_plan: Optional[np.ndarray] = None) -> Dict[str, object]:
        """Runs the batched simulated annealing (rpeg_sa_run).  `directory` is a list of int16 arrays
        [n_v, 6] (dp pp tp r_ext n_ext mb, ascending by time), one per template vertex."""
        torch = _torch()
        keep = []
        for v in range(abi.MAX_V):
            if v < len(directory):
                a = np.ascontiguousarray(directory[v], dtype=np.int16).reshape(-1, 6)
                keep.append(a)
                params.dir_n[v] = a.shape[0]
                params.dir[v] = a.ctypes.data
            else:
                params.dir_n[v] = 0
                params.dir[v] = None
        nc, ns = params.n_chains, params.n_steps
        W = abi.MAX_V * abi.FIELDS
        out = dict(best_plan=np.zeros((nc, W), np.int16), best_score=np.zeros(nc), best_step=np.zeros(nc, np.int32),
                   best_time=np.zeros(nc), best_feasible=np.zeros(nc, np.uint8), cur_plan=np.zeros((nc, W), np.int16),
                   cur_score=np.zeros(nc), restarts=np.zeros(nc, np.int32), n_eval=np.zeros(nc, np.int64),
                   dead=np.zeros(nc, np.uint8), log=np.zeros((nc, max(ns, 1)), np.uint8))
        res = abi.SaResultT()
        for k, a in out.items():
            setattr(res, k, a.ctypes.data)
        base = None
        if base_plan is not None:
            base = np.ascontiguousarray(base_plan, dtype=np.int16).reshape(W)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_sa_run(self._h, C.addressof(params), base.ctypes.data if base is not None else None,
                                      C.addressof(res), stream)
        self._check(rc, "rpeg_sa_run")
        out["log"] = out["log"][:, :ns]
        out.update(wall_s=res.wall_s, eval_s=res.eval_s, n_launch=res.n_launch, n_plans=res.n_plans)
        return out

    def sa_optimize(self, params: "abi.SaParamsT", directory, base_plan: np.ndarray, E_max: int, E_struct: int,
                    R_max: int = 10000, stream_key=(0, 0, 0), log_cap: int = 0) -> Dict[str, object]:
        """optimize() as the reference runs it (rpeg_sa_optimize): one chain at a time, cache and budgets."""
        torch = _torch()
        keep = set_directory(params, directory)
        res, log, logv = serial_result(log_cap)
        base = np.ascontiguousarray(base_plan, dtype=np.int16).reshape(abi.MAX_V * abi.FIELDS)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_sa_optimize(self._h, C.addressof(params), E_max, E_struct, R_max,
                                           *[int(x) for x in stream_key], base.ctypes.data, C.addressof(res), stream)
        self._check(rc, "rpeg_sa_optimize")
        del keep
        return serial_dict(res, log, logv)

    def sa_optimize_families(self, families, base_tau, base_plan: np.ndarray, E_max: int, E_struct: int,
                             R_max: int = 10000, stream_key=(0, 0, 0), log_cap: int = 0) -> Dict[str, object]:
        """optimize() over several structural families (rpeg_sa_optimize_families).  `families` is a list of
        (params, directory, score_scale, elite_family, valid_structure or None); `base_plan` belongs to
        family 0's template and has staleness `base_tau`."""
        torch = _torch()
        arr, keep = family_array(families)
        res, log, logv = serial_result(log_cap)
        base = np.ascontiguousarray(base_plan, dtype=np.int16).reshape(abi.MAX_V * abi.FIELDS)
        tau = (C.c_uint8 * 2)(*([int(t) for t in base_tau] + [0, 0])[:2])
        stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_sa_optimize_families(self._h, len(families), arr, tau, E_max, E_struct, R_max,
                                                    *[int(x) for x in stream_key], base.ctypes.data,
                                                    C.addressof(res), stream)
        self._check(rc, "rpeg_sa_optimize_families")
        del keep
        return serial_dict(res, log, logv)

    def sa_propose(self, params: "abi.SaParamsT", directory, what: int, stream_key=(0, 0, 0), plan=None, mass=None,
                   T: float = 0.0, v: int = 0, r_lo: int = 0, r_hi: int = 0, skip: int = 0):
        """One draw of a proposal kernel (rpeg_sa_propose) on the stream (params.seed, *stream_key), continued
        after `skip` words: what = 0 move_gen, 1 donor/receiver pair, 2 region sample of vertex v on racks
        [r_lo, r_hi).  Returns (rows [n, MAX_V*10] -- [n, 10] for what = 2 --, words drawn so far, fallback)."""
        keep = set_directory(params, directory)
        W = abi.MAX_V * abi.FIELDS
        out = np.zeros((max(params.K_x, 1), W), np.int16)
        draws, fb = C.c_int64(skip), C.c_int32(0)
        p = None if plan is None else np.ascontiguousarray(plan, dtype=np.int16).reshape(W)
        m = None if mass is None else np.ascontiguousarray(mass, dtype=np.float64)
        n = self.lib.rpeg_sa_propose(self._h, C.addressof(params), what, *[int(x) for x in stream_key],
                                     p.ctypes.data if p is not None else None, m.ctypes.data if m is not None else None,
                                     float(T), v, r_lo, r_hi, out.ctypes.data, C.addressof(draws), C.addressof(fb))
        self._check(n, "rpeg_sa_propose")
        del keep
        if what == 2:
            return out.reshape(-1)[:abi.FIELDS * n].reshape(n, abi.FIELDS), draws.value, fb.value
        return out[:n], draws.value, fb.value

    def op_time(self, structure: int, vertex: int, strat: np.ndarray):
        """time() and peak_bytes() of mock nodes: strat is int16 [7, n] = dp pp tp mb r_ext n_ext g_ext."""
        torch = _torch()
        strat = np.ascontiguousarray(strat, dtype=np.int16)
        n = strat.shape[1]
        d = torch.from_numpy(strat).to(self.device)
        t = torch.empty(n, dtype=torch.float64, device=self.device)
        p = torch.empty(n, dtype=torch.float64, device=self.device)
        stream = torch.cuda.current_stream(self.device).cuda_stream
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_op_time_batch(self._h, n, structure, vertex, d.data_ptr(), n, t.data_ptr(), p.data_ptr(), stream)
        self._check(rc, "rpeg_op_time_batch")
        torch.cuda.synchronize(self.device)
        return t.cpu().numpy(), p.cpu().numpy()

    def trace(self, batch: PlanBatch, i: int, cap: int = 4096):
        """Start/finish of every lowered node of plan i, in the reference's node order."""
        torch = _torch()
        vert = np.ascontiguousarray(batch.vert[:, i], dtype=np.int16)
        head = np.ascontiguousarray(batch.head[:, i], dtype=np.uint8)
        start, finish = np.zeros(cap), np.zeros(cap)
        kind, vertex, step, sub, src, order = (np.zeros(cap, np.int32) for _ in range(6))
        edges = np.zeros(2 * cap, np.int32)
        reserved = np.zeros(cap, np.uint8)
        ne = C.c_int32(0)
        with torch.cuda.device(self.device):
            n = self.lib.rpeg_eval_trace(self._h, vert.ctypes.data, head.ctypes.data, start.ctypes.data,
                                         finish.ctypes.data, order.ctypes.data, kind.ctypes.data, vertex.ctypes.data, step.ctypes.data,
                                         sub.ctypes.data, src.ctypes.data, edges.ctypes.data, C.addressof(ne), cap,
                                         reserved.ctypes.data)
        self._check(n, "rpeg_eval_trace")
        return dict(start=start[:n], finish=finish[:n], order=order[:n], kind=kind[:n], vertex=vertex[:n], step=step[:n],
                    sub=sub[:n], src=src[:n], edges=edges[:2 * ne.value].reshape(-1, 2), reserved=reserved[:n])

    def plan_detail(self, batch: PlanBatch, i: int, cap: int = 4096):
        """NodeCostModel.time, payload bytes and label reference of every lowered node of plan i (the reference's
        node order), and the device peak of every set of template vertices whose allocations all intersect
        (rpeg_plan_detail)."""
        torch = _torch()
        vert = np.ascontiguousarray(batch.vert[:, i], dtype=np.int16)
        head = np.ascontiguousarray(batch.head[:, i], dtype=np.uint8)
        time, payload, ref, peaks = np.zeros(cap), np.zeros(cap, np.int64), np.zeros(cap, np.int32), np.zeros(64)
        with torch.cuda.device(self.device):
            n = self.lib.rpeg_plan_detail(self._h, vert.ctypes.data, head.ctypes.data, time.ctypes.data,
                                          payload.ctypes.data, ref.ctypes.data, cap, peaks.ctypes.data)
        self._check(n, "rpeg_plan_detail")
        return dict(time=time[:n], payload=payload[:n], ref=ref[:n], set_peak=peaks)

    def trace_metrics(self, batch: PlanBatch, i: int):
        """(Trace.utilization(), Trace.n_active()) of plan i, folded by the library (rpeg_eval_trace_metrics)."""
        torch = _torch()
        vert = np.ascontiguousarray(batch.vert[:, i], dtype=np.int16)
        head = np.ascontiguousarray(batch.head[:, i], dtype=np.uint8)
        util, act = C.c_double(0.0), C.c_int32(0)
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_eval_trace_metrics(self._h, vert.ctypes.data, head.ctypes.data, C.addressof(util),
                                                  C.addressof(act))
        self._check(rc, "rpeg_eval_trace_metrics")
        return util.value, act.value

    def device_exp(self, x: np.ndarray) -> np.ndarray:
        torch = _torch()
        d = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float64)).to(self.device)
        y = torch.empty_like(d)
        with torch.cuda.device(self.device):
            rc = self.lib.rpeg_device_exp(self._h, d.numel(), d.data_ptr(), y.data_ptr(),
                                          torch.cuda.current_stream(self.device).cuda_stream)
        self._check(rc, "rpeg_device_exp")
        torch.cuda.synchronize(self.device)
        return y.cpu().numpy()
