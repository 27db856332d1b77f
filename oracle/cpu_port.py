"""ctypes wrapper of oracle/_build/libcpu_port.so (host build of the evaluator's arithmetic).
TEST INFRASTRUCTURE ONLY: used by tests and by bench.py's cpu_baseline leg."""

import ctypes as C
import os

import numpy as np

from rpeg_amd.engine import abi
from rpeg_amd.engine.compile import compile_problem

from . import build as _build

_lib = None


def lib():
    global _lib
    if _lib is None:
        path = _build.OUT if os.path.exists(_build.OUT) else _build.build()
        _lib = C.CDLL(path)
        _lib.port_create.restype = C.c_void_p
        _lib.port_create.argtypes = [C.c_void_p]
        _lib.port_destroy.argtypes = [C.c_void_p]
        _lib.port_error.restype = C.c_char_p
        _lib.port_error.argtypes = [C.c_void_p]
        _lib.port_n_classes.restype = C.c_long
        _lib.port_n_classes.argtypes = [C.c_void_p]
        _lib.port_eval.restype = C.c_int
        _lib.port_eval.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint32] + \
            [C.c_void_p] * 6 + [C.c_int, C.c_void_p]
        _lib.port_set_sa_groups.restype = None
        _lib.port_set_sa_groups.argtypes = [C.c_int]
        _lib.port_sa_run.restype = C.c_int
        _lib.port_sa_run.argtypes = [C.c_void_p] * 4 + [C.c_int]
        _lib.port_sa_optimize.restype = C.c_int
        _lib.port_sa_optimize.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_uint64, C.c_uint64,
                                          C.c_uint64, C.c_void_p, C.c_void_p, C.c_int]
        _lib.port_sa_optimize_families.restype = C.c_int
        _lib.port_sa_optimize_families.argtypes = [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32,
                                                   C.c_int32, C.c_uint64, C.c_uint64, C.c_uint64, C.c_void_p, C.c_void_p,
                                                   C.c_int]
        _lib.port_sa_propose.restype = C.c_int
        _lib.port_sa_propose.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_uint64, C.c_uint64, C.c_uint64,
                                         C.c_uint64, C.c_void_p, C.c_void_p, C.c_double, C.c_int, C.c_int, C.c_int,
                                         C.c_void_p, C.c_void_p, C.c_void_p]
        _lib.port_lower.restype = C.c_int
        _lib.port_lower.argtypes = [C.c_void_p] * 9 + [C.c_int32, C.c_void_p]
        _lib.port_op_time.restype = C.c_int
        _lib.port_op_time.argtypes = [C.c_void_p, C.c_uint64, C.c_int, C.c_int, C.c_void_p, C.c_uint64,
                                      C.c_void_p, C.c_void_p]
        _lib.port_exp.argtypes = [C.c_uint64, C.c_void_p, C.c_void_p]
    return _lib


class CpuPort:
    def __init__(self, problem):
        self.problem = problem
        self.P = compile_problem(problem)
        self.h = lib().port_create(C.addressof(self.P))

    def __del__(self):
        if getattr(self, "h", None):
            lib().port_destroy(self.h)
            self.h = None

    def n_classes(self):
        return lib().port_n_classes(self.h)

    def eval(self, batch, flags=0, threads=1, want_mass=False):
        n = batch.n
        vert = np.ascontiguousarray(batch.vert)
        head = np.ascontiguousarray(batch.head)
        out = dict(makespan=np.empty(n), peak=np.empty(n), score=np.empty(n), mask=np.empty(n, np.uint8),
                   sig=np.empty(n, np.uint64))
        mr = C.c_int32(0)
        if want_mass:
            out["mass"] = np.empty((n, abi.MAX_V))
        rc = lib().port_eval(self.h, n, vert.ctypes.data, head.ctypes.data, n, flags,
                             out["makespan"].ctypes.data, out["peak"].ctypes.data, out["score"].ctypes.data,
                             out["mask"].ctypes.data, out["sig"].ctypes.data, C.addressof(mr), threads,
                             out["mass"].ctypes.data if want_mass else None)
        if rc != 0:
            raise RuntimeError(lib().port_error(self.h).decode())
        out["max_ready"] = mr.value
        return out

    def lower(self, batch, i, cap=4096):
        vert = np.ascontiguousarray(batch.vert[:, i])
        head = np.ascontiguousarray(batch.head[:, i])
        kind, vertex, step, sub = (np.zeros(cap, np.int32) for _ in range(4))
        dur = np.zeros(cap)
        edges = np.zeros(2 * cap, np.int32)
        ne = C.c_int32(0)
        n = lib().port_lower(self.h, vert.ctypes.data, head.ctypes.data, kind.ctypes.data, vertex.ctypes.data,
                             step.ctypes.data, sub.ctypes.data, dur.ctypes.data, edges.ctypes.data, cap, C.addressof(ne))
        if n < 0:
            raise RuntimeError(f"port_lower failed ({n}): {lib().port_error(self.h).decode()}")
        return dict(kind=kind[:n], vertex=vertex[:n], step=step[:n], sub=sub[:n], dur=dur[:n],
                    edges=edges[:2 * ne.value].reshape(-1, 2))

    @staticmethod
    def _set_directory(params, directory):
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

    def sa_run(self, params, directory, base_plan=None, threads=1, groups=1):
        """The host annealing logic of rpeg_amd/csrc/rpeg_sa.h over this CPU evaluator.  `groups`: the chains are
        dealt to that many groups that take their steps in turn (what the GPU library does to overlap evaluation and
        host work); the result does not depend on it."""
        lib().port_set_sa_groups(int(groups))
        keep = self._set_directory(params, directory)
        nc, ns = params.n_chains, params.n_steps
        W = abi.MAX_V * abi.FIELDS
        out = dict(best_plan=np.zeros((nc, W), np.int16), best_score=np.zeros(nc), best_step=np.zeros(nc, np.int32),
                   best_time=np.zeros(nc), best_feasible=np.zeros(nc, np.uint8), cur_plan=np.zeros((nc, W), np.int16),
                   cur_score=np.zeros(nc), restarts=np.zeros(nc, np.int32), n_eval=np.zeros(nc, np.int64),
                   dead=np.zeros(nc, np.uint8), log=np.zeros((nc, max(ns, 1)), np.uint8))
        res = abi.SaResultT()
        for k, a in out.items():
            setattr(res, k, a.ctypes.data)
        base = None if base_plan is None else np.ascontiguousarray(base_plan, dtype=np.int16).reshape(W)
        rc = lib().port_sa_run(self.h, C.addressof(params), base.ctypes.data if base is not None else None,
                               C.addressof(res), threads)
        if rc != 0:
            raise RuntimeError(f"port_sa_run failed ({rc}): {lib().port_error(self.h).decode()}")
        del keep
        out["log"] = out["log"][:, :ns]
        out["wall_s"] = res.wall_s
        return out

    def sa_optimize(self, params, directory, base_plan, E_max, E_struct, R_max=10000, stream_key=(0, 0, 0), log_cap=0,
                    threads=1):
        """The reference-style optimize of rpeg_amd/csrc/rpeg_sa.h (SaSerial) over this CPU evaluator."""
        from rpeg_amd.engine.runtime import serial_dict, serial_result
        keep = self._set_directory(params, directory)
        res, log, logv = serial_result(log_cap)
        base = np.ascontiguousarray(base_plan, dtype=np.int16).reshape(abi.MAX_V * abi.FIELDS)
        rc = lib().port_sa_optimize(self.h, C.addressof(params), E_max, E_struct, R_max, *[int(x) for x in stream_key],
                                    base.ctypes.data, C.addressof(res), threads)
        if rc != 0:
            raise RuntimeError(f"port_sa_optimize failed ({rc}): {lib().port_error(self.h).decode()}")
        del keep
        return serial_dict(res, log, logv)

    def sa_optimize_families(self, families, base_tau, base_plan, E_max, E_struct, R_max=10000, stream_key=(0, 0, 0),
                             log_cap=0, threads=1):
        """SaSerial over several structural families (the CPU twin of rpeg_sa_optimize_families)."""
        from rpeg_amd.engine.runtime import family_array, serial_dict, serial_result
        arr, keep = family_array(families)
        res, log, logv = serial_result(log_cap)
        base = np.ascontiguousarray(base_plan, dtype=np.int16).reshape(abi.MAX_V * abi.FIELDS)
        tau = (C.c_uint8 * 2)(*([int(t) for t in base_tau] + [0, 0])[:2])
        rc = lib().port_sa_optimize_families(self.h, len(families), arr, tau, E_max, E_struct, R_max,
                                             *[int(x) for x in stream_key], base.ctypes.data, C.addressof(res), threads)
        if rc != 0:
            raise RuntimeError(f"port_sa_optimize_families failed ({rc})")
        del keep
        return serial_dict(res, log, logv)

    def sa_propose(self, params, directory, what, stream, plan=None, mass=None, T=0.0, v=0, r_lo=0, r_hi=0, skip=0):
        """One proposal with generator stream (seed, a, b, c): what = 0 move_gen, 1 donor/receiver pair,
        2 region sample.  Returns (rows [n, MAX_V*10] or [n, 10], words drawn so far, fallback count)."""
        keep = self._set_directory(params, directory)
        W = abi.MAX_V * abi.FIELDS
        out = np.zeros((max(params.K_x, 1), W), np.int16)
        draws, fb = C.c_int64(skip), C.c_int32(0)
        p = None if plan is None else np.ascontiguousarray(plan, dtype=np.int16).reshape(W)
        m = None if mass is None else np.ascontiguousarray(mass, dtype=np.float64)
        n = lib().port_sa_propose(self.h, C.addressof(params), what, *[int(x) for x in stream],
                                  p.ctypes.data if p is not None else None, m.ctypes.data if m is not None else None,
                                  float(T), v, r_lo, r_hi, out.ctypes.data, C.addressof(draws), C.addressof(fb))
        del keep
        if what == 2:
            return out.reshape(-1)[:10 * n].reshape(n, 10), draws.value, fb.value
        return out[:n], draws.value, fb.value

    def op_time(self, structure, vertex, strat):
        strat = np.ascontiguousarray(strat, dtype=np.int16)
        n = strat.shape[1]
        t, p = np.empty(n), np.empty(n)
        lib().port_op_time(self.h, n, structure, vertex, strat.ctypes.data, n, t.ctypes.data, p.ctypes.data)
        return t, p


def exp_libm(x):
    x = np.ascontiguousarray(x, dtype=np.float64)
    y = np.empty_like(x)
    lib().port_exp(x.size, x.ctypes.data, y.ctypes.data)
    return y


def count_flops(problem, batch, flags=0):
    """fp64 operations of the plans of `batch`, as the kernels' arithmetic executes them (flop_count.cpp):
    dict with the per-plan means of add (additions and subtractions), mul, div, fma, cmp (comparisons, max and
    min included) and `total` = add + mul + div + cmp + 2 fma, plus `plans` (valid plans counted)."""
    path = _build.FLOPS if os.path.exists(_build.FLOPS) else (_build.build(force=True) and _build.FLOPS)
    fl = C.CDLL(path)
    fl.flop_count.restype = C.c_int
    fl.flop_count.argtypes = [C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint32, C.c_void_p]
    P = compile_problem(problem)
    vert = np.ascontiguousarray(batch.vert)
    head = np.ascontiguousarray(batch.head)
    out = (C.c_uint64 * 6)()
    rc = fl.flop_count(C.addressof(P), batch.n, vert.ctypes.data, head.ctypes.data, vert.shape[1], flags, out)
    if rc != 0:
        raise RuntimeError("flop_count failed")
    n = max(1, out[5])
    res = dict(add=out[0] / n, mul=out[1] / n, div=out[2] / n, fma=out[3] / n, cmp=out[4] / n, plans=int(out[5]))
    res["total"] = res["add"] + res["mul"] + res["div"] + res["cmp"] + 2 * res["fma"]
    return res
