"""CPU restatement of the simulated-annealing neighbourhood and chain loop.  TEST INFRASTRUCTURE.

Only tests/, the smoke check and the CPU-baseline leg of the benchmark may import this module;
the product never does.

It restates, in plain Python on duck-typed plans:

* the strategy enumeration and candidate directory (RPEG/search/moves.py:97-198, 393-551),
* the critical-chain vertex bias (moves.py:590-642),
* the single-vertex kernel `move_gen` (moves.py:645-825),
* the samplers and the donor/receiver kernel `multi_move_pair` (moves.py:202-390, 845-950),
* restarts and the elite list (RPEG/search/optimizer.py:175-362),
* one Metropolis-Hastings step and the chain loop (optimizer.py:690-946), for a population of
  independent chains that run a fixed number of steps.

Every random choice goes through an explicit generator object with the four methods the
reference calls on Python's `random` module (`random`, `choice`, `choices`, `randint`).  The
reference draws from MT19937; here the generator is counter based (`CounterRng`), so a chain's
trajectory is a pure function of (seed, chain, step).  The proposal functions are pinned against
the reference by handing the reference's own functions the same generator object
(tests/golden/make_golden_sa.py): same draws in the same order give the same proposals.  The
chain loop is pinned the same way: `serial_chain` reproduces, evaluation by evaluation, what the
reference's own optimize() does on that generator (tests/golden/make_golden_optimize.py), and
`polish` what its polish() returns (tests/golden/make_golden_polish.py).

Differences from the reference, all deliberate:

* `_critical_mass` sums `finish - start` over a Python set of nodes hashed by their string id,
  i.e. in an order that changes from process to process; here the sum runs along the chain from
  the sink backwards.
* With an empty candidate table `move_gen` of the reference raises (randint on an empty range);
  here the strategy loop is skipped.
* The chain loop runs `n_steps` iterations per chain instead of an evaluation budget, evaluates
  every candidate (no evaluation cache: results do not depend on it), and draws random restarts
  in batches of `restart_attempts` complete plans of which the first valid one is taken.  Where
  the reference gives a structural setting up (no valid restart), a chain goes on from its
  current plan; a chain with no base plan and no valid random start begins at its first random
  plan and relies on the soft memory penalty, as the reference does from an infeasible baseline.
"""

from __future__ import annotations

import math
from bisect import bisect_right
from itertools import accumulate

from . import rpeg_oracle as O

MASK64 = (1 << 64) - 1
GOLD = 0x9E3779B97F4A7C15
MIN_B_LOCAL = 8            # moves.py:146
SA_TAG = 0x5A


def mix64(x):
    x &= MASK64
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & MASK64
    return x ^ (x >> 31)


class CounterRng:
    """Counter-based stand-in for the `random` module: word k of stream (seed, a, b, c)."""

    def __init__(self, seed, a=0, b=0, c=0):
        h = mix64(seed + GOLD * (SA_TAG + 1))
        h = mix64(h + GOLD * (a + 1))
        h = mix64(h + GOLD * (b + 1))
        self.h = mix64(h + GOLD * (c + 1))
        self.k = 0

    def word(self):
        self.k += 1
        return mix64(self.h + GOLD * self.k)

    def random(self):
        return (self.word() >> 11) * (1.0 / 9007199254740992.0)

    def below(self, n):
        return ((self.word() >> 32) * n) >> 32

    def choice(self, seq):
        return seq[self.below(len(seq))]

    def randint(self, a, b):
        return a + self.below(b - a + 1)

    def choices(self, population, weights=None, k=1):
        # CPython's random.choices: bisect of random()*total in the running sums
        cum = list(accumulate(weights))
        total = cum[-1] + 0.0
        hi = len(population) - 1
        return [population[bisect_right(cum, self.random() * total, 0, hi)] for _ in range(k)]


# ----------------------------------------------------------------------------- strategy space
def valid_tp_degrees(G):
    """moves.py:97-107."""
    return [tp for tp in range(1, G + 1) if G % tp == 0]


def valid_pp_degrees(R, N, G, L):
    """moves.py:109-122: divisors of L that are 1 or even."""
    return [d for d in range(1, R * N * G + 1) if L % d == 0 and (d == 1 or d % 2 == 0)]


def valid_dp_degrees(R, N, B, G=1):
    """moves.py:125-137."""
    return [d for d in range(1, R * N * G + 1) if B % d == 0]


ABLATION_FIXED_MB = False   # moves.py:155-156: tests set it around a directory build


def valid_mb_counts(pp, dp, B):
    """moves.py:162-199."""
    local = B // dp
    if local < MIN_B_LOCAL and dp > 1:
        return []
    if pp == 1:
        return [1]
    if ABLATION_FIXED_MB:
        return [1] if local % pp != 0 else [pp]
    max_mb = local // MIN_B_LOCAL
    return [mb for mb in range(pp, min(max_mb, local) + 1) if local % mb == 0]


def enumerate_strategies(v, suite, space, workload):
    """moves.py:393-426: every (dp, pp, tp, r_ext, n_ext, mb) of the proposal support."""
    R, N, G, B = space.R, space.N, space.G, workload.B
    L = suite.specs[v.kind.model].L
    out = []
    for tp in valid_tp_degrees(G):
        for pp in valid_pp_degrees(R, N, G, L):
            s = min(pp, G // tp)
            if pp % s != 0:
                continue
            for dp in valid_dp_degrees(R, N, B, G):
                mbs = valid_mb_counts(pp, dp, B)
                if not mbs:
                    continue
                geom = O.packing_geometry(dp, pp, tp, G)
                if geom is None:
                    continue
                for r_ext, n_ext in O.rectangular_node_layouts(geom[1], R, N):
                    for mb in mbs:
                        out.append((dp, pp, tp, r_ext, n_ext, mb))
    return out


class _Alloc:
    __slots__ = ("origin", "extent")

    def __init__(self, origin, extent):
        self.origin, self.extent = origin, extent


def mock_node(v, dp, pp, tp, r_ext, n_ext, mb, g_ext):
    """moves.py:429-461: an unsplit step-0 operator node at the origin."""
    return O.XNode("_approx", O.OP, (_Alloc((0, 0, 0), (r_ext, n_ext, g_ext)),), tpl=v, k=0,
                   model=v.kind.model, pi=(dp, pp, tp), mb=mb)


def build_candidate_directory(rpeg, suite, space, workload, cost, mem, max_per_vertex=1000):
    """moves.py:464-551.  table[v] = [(dp, pp, tp, r_ext, n_ext, mb, time)] ascending by time
    (stable), memory-infeasible strategies dropped, cut to max_per_vertex; index[v][key] = position."""
    table, index = {}, {}
    cap = mem.capacity()
    for v in rpeg.vertices:
        cands = []
        for strat in enumerate_strategies(v, suite, space, workload):
            dp, pp, tp, r_ext, n_ext, mb = strat
            g_ext = O.packing_geometry(dp, pp, tp, space.G)[0]
            nd = mock_node(v, dp, pp, tp, r_ext, n_ext, mb, g_ext)
            if mem.peak_bytes(nd) > cap:
                continue
            cands.append(strat + (cost.time(nd),))
        cands.sort(key=lambda c: c[6])
        cands = cands[:max_per_vertex]
        table[v] = cands
        index[v] = {c[:6]: j for j, c in enumerate(cands)}
    return table, index


def find_current_position(v, plan, index_v, n_candidates):
    """moves.py:554-586; returns (position, used_fallback)."""
    dp, pp, tp = plan.pi[v]
    r_ext, n_ext, _ = plan.sigma[v].extent
    key = (dp, pp, tp, r_ext, n_ext, plan.mb[v])
    if key in index_v:
        return index_v[key], False
    return n_candidates // 2, True


# ----------------------------------------------------------------------------- critical chain
def critical_chain(nodes, edges, finish):
    """moves.py:590-619: from the first node of largest finish time, follow the first
    predecessor (in edge order) of largest finish time.  Returns the chain as a list."""
    pred = {n.id: [] for n in nodes}
    for a, b in edges:
        pred[b.id].append(a)
    cur = max(nodes, key=lambda n: finish[n.id])
    chain = [cur]
    while pred[cur.id]:
        cur = max(pred[cur.id], key=lambda n: finish[n.id])
        chain.append(cur)
    return chain


def critical_mass(chain, rpeg, start, finish):
    """moves.py:622-642: per template vertex, the summed durations of its operator nodes on the
    chain (summed from the sink backwards)."""
    mass = {v: 0.0 for v in rpeg.vertices}
    for n in chain:
        if n.kind != O.OP:
            continue
        mass[n.tpl] += finish[n.id] - start[n.id]
    return mass


# ----------------------------------------------------------------------------- single-vertex kernel
def _new_plan(plan, changes):
    sigma, pi, mb = dict(plan.sigma), dict(plan.pi), dict(plan.mb)
    for v, (alloc, par, m) in changes.items():
        sigma[v], pi[v], mb[v] = alloc, par, m
    return type(plan)(sigma=sigma, pi=pi, mb=mb)


def sample_origin(rng, space, extent):
    """moves.py:685-694: three draws, also when only one origin exists."""
    r_ext, n_ext, g_ext = extent
    r_o = rng.choice([i * r_ext for i in range(space.R // r_ext)])
    n_o = rng.choice([i * n_ext for i in range(space.N // n_ext)])
    g_o = rng.choice([i * g_ext for i in range(space.G // g_ext)])
    return (r_o, n_o, g_o)


def move_gen(rng, rpeg, plan, space, mass, table, index, K_x, T_max, T, T_init, stats=None):
    """moves.py:645-825 without intra-stage fusion.  `mass` is the critical mass of the current
    plan's trace (a dict vertex -> seconds) or a callable that computes it when the biased
    branch is taken.  Returns the list of proposed plans."""
    vertices = rpeg.vertices
    if rng.random() >= 0.4:
        m = mass() if callable(mass) else mass
        weights = [m[v] + 1e-6 for v in vertices]
        v = rng.choices(vertices, weights=weights, k=1)[0]
    else:
        v = rng.choice(vertices)

    v_cands = table[v]
    frac = min(1.0, T / T_init)
    w = max(5, int(len(v_cands) * frac))
    j_star, fell_back = find_current_position(v, plan, index[v], len(v_cands))
    if stats is not None and fell_back:
        stats["n_fallback"] = stats.get("n_fallback", 0) + 1
    low, high = max(0, j_star - w), min(len(v_cands) - 1, j_star + w)

    Alloc = type(plan.sigma[v])
    out, seen = [], set()
    curr_alloc, curr_pi, curr_mb = plan.sigma[v], plan.pi[v], plan.mb[v]

    for _ in range(min(5, T_max)):
        o = sample_origin(rng, space, curr_alloc.extent)
        if o != tuple(curr_alloc.origin):
            seen.add((tuple(curr_pi), o, curr_mb))
            out.append(_new_plan(plan, {v: (Alloc(o, curr_alloc.extent), curr_pi, curr_mb)}))
            break

    for _ in range(T_max):
        if len(out) >= K_x or high < low:
            break
        j = rng.randint(low, high)
        if j == j_star:
            continue
        dp, pp, tp, r_ext, n_ext, mb, _t = v_cands[j]
        g_ext = O.packing_geometry(dp, pp, tp, space.G)[0]
        o = sample_origin(rng, space, (r_ext, n_ext, g_ext))
        key = ((dp, pp, tp), o, mb)
        if key in seen:
            continue
        seen.add(key)
        out.append(_new_plan(plan, {v: (Alloc(o, (r_ext, n_ext, g_ext)), (dp, pp, tp), mb)}))
    return out


# ----------------------------------------------------------------------------- samplers
def sample_expl_in_region(rng, v, suite, space, workload, r_lo=0, r_hi=None):
    """moves.py:180-278: (origin, extent, (dp, pp, tp), mb) or None."""
    R, N, G, B = space.R, space.N, space.G, workload.B
    L = suite.specs[v.kind.model].L
    if r_hi is None:
        r_hi = R
    R_eff = r_hi - r_lo
    tp = rng.choice(valid_tp_degrees(G))
    pps = valid_pp_degrees(R, N, G, L)
    if not pps:
        return None
    pp = rng.choice(pps)
    s = min(pp, G // tp)
    if pp % s != 0:
        return None
    dps = []
    for d in valid_dp_degrees(R, N, B, G):
        geom = O.packing_geometry(d, pp, tp, G)
        if geom is not None and geom[1] <= R_eff * N:
            dps.append(d)
    if not dps:
        return None
    dp = rng.choice(dps)
    g_ext, need = O.packing_geometry(dp, pp, tp, G)
    layouts = [(r, n, g_ext) for r, n in O.rectangular_node_layouts(need, R_eff, N)]
    if not layouts:
        return None
    r_ext, n_ext, g_ext = rng.choice(layouts)
    r_origins = [r_lo + i * r_ext for i in range(R_eff // r_ext)]
    if not r_origins:
        return None
    r_o = rng.choice(r_origins)
    n_o = rng.choice([i * n_ext for i in range(N // n_ext)])
    g_o = rng.choice([i * g_ext for i in range(G // g_ext)])
    mbs = valid_mb_counts(pp, dp, B)
    if not mbs:
        return None
    mb = rng.choice(mbs)
    return (r_o, n_o, g_o), (r_ext, n_ext, g_ext), (dp, pp, tp), mb


def multi_move_pair(rng, rpeg, plan, space, suite, workload, max_retries=100):
    """moves.py:845-950 without intra-stage fusion: the proposed plan or None."""
    vertices = list(rpeg.vertices)
    R = space.R
    counts = [float(plan.sigma[v].extent[0] * plan.sigma[v].extent[1] * plan.sigma[v].extent[2])
              for v in vertices]
    if sum(counts) == 0:
        return None
    v_d = rng.choices(vertices, weights=counts, k=1)[0]
    overlap = [v for v in vertices
               if v is not v_d and O.allocations_overlap(plan.sigma[v], plan.sigma[v_d])]
    if not overlap:
        return None
    v_r = rng.choice(overlap)

    d_alloc = plan.sigma[v_d]
    d_lo, d_ext = d_alloc.origin[0], d_alloc.extent[0]
    if d_ext > 1:
        new_ext = rng.randint(1, d_ext - 1)
        new_lo = rng.choice(list(range(d_lo, d_lo + d_ext - new_ext + 1)))
    else:
        new_lo, new_ext = d_lo, 1

    donor = None
    for _ in range(max_retries):
        donor = sample_expl_in_region(rng, v_d, suite, space, workload, new_lo, new_lo + new_ext)
        if donor is not None:
            break
    if donor is None:
        return None

    freed = set(range(d_lo, d_lo + d_ext)) - set(range(new_lo, new_lo + new_ext))
    if freed:
        r_alloc = plan.sigma[v_r]
        combined = set(range(r_alloc.origin[0], r_alloc.origin[0] + r_alloc.extent[0])) | freed
        recv_lo, recv_hi = min(combined), max(combined) + 1
    else:
        recv_lo, recv_hi = 0, R

    recv = None
    for _ in range(max_retries):
        recv = sample_expl_in_region(rng, v_r, suite, space, workload, recv_lo, recv_hi)
        if recv is not None:
            break
    if recv is None:
        return None
    Alloc = type(d_alloc)
    return _new_plan(plan, {v_d: (Alloc(donor[0], donor[1]), donor[2], donor[3]),
                            v_r: (Alloc(recv[0], recv[1]), recv[2], recv[3])})


def sample_all_vertices(rng, rpeg, plan_type, alloc_type, suite, space, workload):
    """optimizer.py:201-256 without fusion: a complete random plan, or None where the reference
    raises (a vertex whose sampler failed 100 times)."""
    sigma, pi, mb = {}, {}, {}
    for v in rpeg.vertices:
        s = None
        for _ in range(100):
            s = sample_expl_in_region(rng, v, suite, space, workload)
            if s is not None:
                break
        if s is None:
            return None
        sigma[v], pi[v], mb[v] = alloc_type(s[0], s[1]), s[2], s[3]
    return plan_type(sigma=sigma, pi=pi, mb=mb)


# ----------------------------------------------------------------------------- elites
def plan_fingerprint(plan):
    """optimizer.py:158-172."""
    verts = sorted(plan.pi.keys(), key=lambda v: v.id)
    return tuple((v.id, tuple(plan.pi[v]), tuple(plan.sigma[v].origin), plan.mb[v]) for v in verts)


def elite_insert(raw, entry, plan, elite, seen, K):
    """optimizer.py:175-198 for one family: `elite` is a list of (raw, entry) sorted descending."""
    fp = plan_fingerprint(plan)
    if fp in seen:
        return
    if len(elite) >= K and raw <= elite[-1][0]:
        return
    elite[:] = sorted(elite + [(raw, entry)], key=lambda x: -x[0])[:K]
    seen.add(fp)


# ----------------------------------------------------------------------------- chains
class SaParams:
    """The optimizer settings that reach the chain loop (optimizer.py:33-63)."""

    def __init__(self, K_x=6, T_max=50, T_init=0.30, T_warm=0.05, T_min=0.01, K_elite=3,
                 alpha_pair=0.28, stag_window=20, score_eps=1e-4, geometric_cooling=False,
                 E_struct=400, restart_attempts=50, gate_candidates=False, seed=42):
        self.K_x, self.T_max, self.T_init, self.T_warm, self.T_min = K_x, T_max, T_init, T_warm, T_min
        self.K_elite, self.alpha_pair, self.stag_window, self.score_eps = K_elite, alpha_pair, stag_window, score_eps
        self.geometric_cooling, self.restart_attempts = geometric_cooling, restart_attempts
        self.gate_candidates, self.seed = gate_candidates, seed
        I_max = int(E_struct / ((K_x + 1) / 2) * 0.5)                       # optimizer.py:123-125
        self.T_cool = (T_min / T_init) ** (1.0 / (0.7 * I_max))             # :128


class Evaluated:
    __slots__ = ("plan", "score", "gated", "mem_ok", "stale_ok", "mass")

    def __init__(self, plan, score, gated, mem_ok, stale_ok, mass):
        self.plan, self.score, self.gated = plan, score, gated
        self.mem_ok, self.stale_ok, self.mass = mem_ok, stale_ok, mass


def oracle_evaluator(rpeg, space, suite, workload, hw, K_eval, policy=None,
                     transfer_policy=("destination_only", "destination_only")):
    """plan -> Evaluated, through the Python restatement of the evaluation path."""
    def run(plan):
        r = O.evaluate_plan(rpeg, plan, space, suite, workload, hw, K_eval, policy, check_stale=False,
                            want_trace=True, transfer_policy=transfer_policy)
        chain = critical_chain(r["nodes"], r["edges"], r["finish"])
        mass = critical_mass(chain, rpeg, r["start"], r["finish"])
        gated = r["score"] if r["stale_ok"] else 0.0
        return Evaluated(plan, r["score"], gated, r["feasible"], r["stale_ok"], mass)
    return run


class Chain:
    def __init__(self, cid):
        self.id = cid
        self.cur = None            # Evaluated of the current plan
        self.score = 0.0           # score_curr
        self.T = 0.0
        self.rej = 0               # consecutive rejections
        self.r = 0                 # restarts so far
        self.dead = False
        self.elite, self.seen = [], set()
        self.best, self.best_score, self.best_step = None, -math.inf, -1
        self.best_feasible, self.best_feasible_score, self.best_feasible_step = None, -math.inf, -1
        self.n_eval = 0
        self.log = []              # (step, kind, n_candidates, accepted)


def _is_valid(rpeg, ev, space, suite, workload):
    """evaluate.py:143-232: integer rules, stale layout, memory (peaks do not depend on K_eval)."""
    return (O.plan_structurally_valid(rpeg, ev.plan, space, suite, workload) and ev.stale_ok and ev.mem_ok)


def _note(ch, ev, score, step, p, gated_feasible):
    """Bookkeeping shared by restarts and candidates (optimizer.py:676-686, 846-861)."""
    if gated_feasible:
        elite_insert(ev.score, ev, ev.plan, ch.elite, ch.seen, p.K_elite)
    if ch.best is None or score > ch.best_score * (1.0 + p.score_eps):
        ch.best, ch.best_score, ch.best_step = ev, score, step
    if gated_feasible and score > ch.best_feasible_score:
        ch.best_feasible, ch.best_feasible_score, ch.best_feasible_step = ev, score, step


def _random_restart(ch, step, rpeg, plan_type, alloc_type, space, suite, workload, evaluate, p):
    """optimizer.py:259-289: (first valid one of `restart_attempts` complete random plans, first attempt)."""
    first = None
    for a in range(p.restart_attempts):
        rng = CounterRng(p.seed, ch.id, step + 1, 1 + a)
        plan = sample_all_vertices(rng, rpeg, plan_type, alloc_type, suite, space, workload)
        if plan is None:
            break
        ev = evaluate(plan)
        ch.n_eval += 1
        if first is None:
            first = ev
        if _is_valid(rpeg, ev, space, suite, workload):
            return ev, first
    return None, first


def _enter(ch, ev, step, T, p):
    """Start of a restart: evaluate_cached semantics for the current plan (optimizer.py:666-694)."""
    ch.cur = ev
    ch.score = ev.gated
    feasible = ev.mem_ok and ev.stale_ok
    _note(ch, ev, ch.score, step, p, feasible)
    ch.T, ch.rej = T, 0


def propose(rng, rpeg, cur, space, suite, workload, table, index, p, T):
    """Kernel selection and proposals of one iteration (optimizer.py:726-765).  Returns (kind, plans);
    plans is None when the donor/receiver kernel failed to sample."""
    frac = min(1.0, T / p.T_init)
    if rng.random() < p.alpha_pair * frac:
        nb = multi_move_pair(rng, rpeg, cur.plan, space, suite, workload)
        return "pair", (None if nb is None else [nb])
    return "single", move_gen(rng, rpeg, cur.plan, space, cur.mass, table, index, p.K_x, p.T_max, T, p.T_init)


def mh_accept(rng, best_s, score_curr, T):
    """One Metropolis-Hastings test (optimizer.py:881-895): None below the noise threshold (no draw)."""
    delta = (best_s - score_curr) / (abs(score_curr) + 1e-12)
    if abs(delta) < 1e-6:
        return None
    prob = 1.0 if delta >= 0.0 else math.exp(delta / T)
    return rng.random() < prob


def run_chains(rpeg_of_chain, plan_type, alloc_type, space, suite, workload, evaluate_of_chain, tables,
               n_chains, n_steps, params, base_plan=None, first_chain=0):
    """`n_chains` independent chains of `n_steps` Metropolis-Hastings steps each.

    rpeg_of_chain(c) and evaluate_of_chain(c) give chain c's template (its staleness variant) and
    evaluator; tables = (table, index) of the candidate directory; chains are numbered from
    `first_chain` (the number keys the chain's random stream).  Returns the list of Chain."""
    p = params
    table, index = tables
    chains = [Chain(first_chain + c) for c in range(n_chains)]
    for ch in chains:
        rpeg, evaluate = rpeg_of_chain(ch.id), evaluate_of_chain(ch.id)
        # the base plan if valid, else a valid random plan, else the base plan as it is (the soft memory
        # penalty guides the search, optimizer.py:612-616), else the first random plan as it is
        start = None
        if base_plan is not None:
            ev = evaluate(base_plan)
            ch.n_eval += 1
            if _is_valid(rpeg, ev, space, suite, workload):
                start = ev
            else:
                start = _random_restart(ch, -1, rpeg, plan_type, alloc_type, space, suite, workload, evaluate, p)[0] or ev
        else:
            found, first = _random_restart(ch, -1, rpeg, plan_type, alloc_type, space, suite, workload, evaluate, p)
            start = found or first
        if start is None:
            ch.dead = True
            continue
        _enter(ch, start, -1, p.T_init, p)

    for step in range(n_steps):
        for ch in chains:
            if ch.dead:
                continue
            rpeg, evaluate = rpeg_of_chain(ch.id), evaluate_of_chain(ch.id)
            rng = CounterRng(p.seed, ch.id, step + 1, 0)
            restart = False
            kind, cands = propose(rng, rpeg, ch.cur, space, suite, workload, table, index, p, ch.T)
            if cands is None:
                ch.T = max(p.T_min, ch.T * p.T_cool)                # optimizer.py:737-740
                ch.log.append((step, "pair", 0, None))
                continue
            accepted = None
            if not cands:
                restart = True                                       # "chain stuck" (optimizer.py:767-769)
            else:
                best_ev, best_s = None, -math.inf
                for plan in cands:
                    ev = evaluate(plan)
                    ch.n_eval += 1
                    s = ev.gated if p.gate_candidates else ev.score
                    feas = ev.mem_ok and (ev.stale_ok or not p.gate_candidates)
                    _note(ch, ev, s, step, p, feas)
                    if s > best_s:
                        best_ev, best_s = ev, s
                accepted = mh_accept(rng, best_s, ch.score, ch.T)
                if accepted:
                    ch.cur, ch.score, ch.rej = best_ev, best_s, 0
                elif accepted is not None:
                    ch.rej += 1
                if p.geometric_cooling:
                    ch.T = max(p.T_min, ch.T * p.T_cool)
                if p.stag_window > 0 and ch.rej >= p.stag_window:
                    restart = True
            ch.log.append((step, kind, len(cands), accepted))
            if restart:
                ch.r += 1
                warm = ch.elite[0][1] if ch.elite else None
                if warm is not None and _is_valid(rpeg, warm, space, suite, workload):
                    nxt = warm
                else:
                    nxt = _random_restart(ch, step, rpeg, plan_type, alloc_type, space, suite, workload, evaluate, p)[0]
                if nxt is None:
                    ch.T, ch.rej = p.T_warm, 0      # no valid restart: go on from the current plan
                    continue
                _enter(ch, nxt, step, p.T_warm, p)
    return chains


def serial_chain(rng, rpeg, base_plan, space, suite, workload, evaluate, tables, params, E_max, E_struct,
                 R_max=10000):
    """optimize() (optimizer.py:365-946) for ONE structural setting, as the reference runs it: one chain
    at a time on one continuous random stream, an evaluation cache (hits cost no budget and are merged
    before fresh results), the budgets E_max / E_struct counted in cache misses, restarts from the best
    elite plan.  It shares `propose`, `mh_accept`, `elite_insert` and the bookkeeping with `run_chains`;
    it exists so that those can be pinned against the reference's own optimize() driven by the same
    generator (tests/golden/make_golden_optimize.py).  The base plan must be valid and the elite plans
    stay valid (no random restart is restated).

    Returns (best feasible plan or best plan, evaluation log): the log lists every plan handed to the
    evaluator (cache misses only), in order."""
    p = params
    table, index = tables
    cache, order = {}, []

    def key(q):
        return tuple((tuple(q.pi[v]), q.mb[v], tuple(q.sigma[v].origin), tuple(q.sigma[v].extent)) for v in rpeg.vertices)

    def cached(q, gated):
        """(Evaluated, miss).  The cache stores what the first evaluation stored: evaluate_cached stores the
        gated score, the merge of fresh candidates the score of _eval_worker (optimizer.py:838, evaluate.py:372-374)."""
        k = key(q)
        if k in cache:
            return cache[k], False
        ev = evaluate(q)
        order.append(q)
        stored = (ev.gated if gated else ev.score, ev.mem_ok and (ev.stale_ok or not gated), ev)
        cache[k] = stored
        return stored, True

    ch = Chain(0)
    (s0, f0, ev0), _ = cached(base_plan, True)
    ch.best, ch.best_score = ev0, s0
    if f0:
        ch.best_feasible, ch.best_feasible_score = ev0, s0
        elite_insert(s0, ev0, ev0.plan, ch.elite, ch.seen, p.K_elite)
    E, E_s = 1, 0
    cur = ev0
    r, no_progress, exhausted = 0, 0, False
    while r < R_max and not exhausted:
        restart_E_s = E_s
        if r > 0:
            cur = ch.elite[0][1] if ch.elite else cur          # warm restart (optimizer.py:640-660)
            no_progress = 0
        (score_curr, feasible, cur), miss = cached(cur.plan, True)
        if miss:
            E += 1; E_s += 1
        if feasible:
            elite_insert(score_curr, cur, cur.plan, ch.elite, ch.seen, p.K_elite)
        if score_curr > ch.best_score * (1.0 + p.score_eps):
            ch.best, ch.best_score = cur, score_curr
        if feasible and score_curr > ch.best_feasible_score:
            ch.best_feasible, ch.best_feasible_score = cur, score_curr
        T = p.T_warm if r > 0 else p.T_init
        rej = 0
        while True:
            if E >= E_max:
                return (ch.best_feasible or ch.best).plan, order
            if E_s >= E_struct:
                exhausted = True
                break
            kind, cands = propose(rng, rpeg, cur, space, suite, workload, table, index, p, T)
            if cands is None:
                T = max(p.T_min, T * p.T_cool)
                continue
            if not cands:
                break
            hits, fresh = [], []
            for plan in cands:                                  # optimizer.py:781-789
                k = key(plan)
                (hits if k in cache else fresh).append(plan)
            best_ev, best_s = None, -math.inf
            for plan in hits + fresh:                           # optimizer.py:807-861
                (s, f, ev), miss = cached(plan, False)
                if miss:
                    E += 1; E_s += 1
                if f:
                    elite_insert(s, ev, ev.plan, ch.elite, ch.seen, p.K_elite)
                if s > ch.best_score * (1.0 + p.score_eps):
                    ch.best, ch.best_score = ev, s
                if f and s > ch.best_feasible_score:
                    ch.best_feasible, ch.best_feasible_score = ev, s
                if s > best_s:
                    best_ev, best_s = ev, s
            if E >= E_max:
                return (ch.best_feasible or ch.best).plan, order
            if E_s >= E_struct:
                exhausted = True
            if not exhausted:
                accepted = mh_accept(rng, best_s, score_curr, T)
                if accepted:
                    cur, score_curr, rej = best_ev, best_s, 0
                elif accepted is not None:
                    rej += 1
            if p.geometric_cooling:
                T = max(p.T_min, T * p.T_cool)
            if exhausted:
                break
            if p.stag_window > 0 and rej >= p.stag_window:
                break
        r += 1
        if E_s == restart_E_s:
            no_progress += 1
            if no_progress >= 2:
                exhausted = True
        else:
            no_progress = 0
    return (ch.best_feasible or ch.best).plan, order


# ----------------------------------------------------------------------------- polish
def polish(rpeg, plan, space, suite, workload, evaluate, table, index, T_min, T_init, max_rounds=50):
    """optimizer.py:949-1188 without fusion, AC-share penalty and utilisation weighting: greedy
    coordinate descent.  Vertices in id order; for each, every strategy of the directory window
    [j*-w, j*+w] (w = max(5, int(n*T_min/T_init))) placed at origin (0,0,0) is evaluated (as
    `_eval_worker` scores it, memory-infeasible candidates dropped) and the best strict
    improvement is taken; passes repeat until one brings no improvement.

    `evaluate(plan)` returns an Evaluated.  Returns (plan, score, rounds, distinct plans evaluated)."""
    Alloc = type(next(iter(plan.sigma.values())))
    seen = {}                                             # the evaluation cache: every plan is scored once

    def key(q):
        return tuple((tuple(q.pi[v]), q.mb[v], tuple(q.sigma[v].origin), tuple(q.sigma[v].extent)) for v in rpeg.vertices)

    def cached(q):
        k = key(q)
        if k not in seen:
            seen[k] = evaluate(q)
        return seen[k]
    cur = cached(plan)
    score = cur.gated                                     # evaluate_cached (optimizer.py:1044)
    rounds = 0
    w_frac = T_min / T_init
    order = sorted(rpeg.vertices, key=lambda v: v.id)
    for round_idx in range(max_rounds):
        rounds = round_idx + 1
        improved = False
        for v in order:
            best_s, best_plan = score, None
            tab = table[v]
            n = len(tab)
            w = max(5, int(n * w_frac))
            dp, pp, tp = plan.pi[v]
            r_ext, n_ext, _ = plan.sigma[v].extent
            j_star = index[v].get((dp, pp, tp, r_ext, n_ext, plan.mb[v]), n // 2)
            cands = []
            for j in range(max(0, j_star - w), min(n - 1, j_star + w) + 1):
                if j == j_star:
                    continue
                d2, p2, t2, re2, ne2, mb2 = tab[j][:6]
                g_ext = O.packing_geometry(d2, p2, t2, space.G)[0]
                cands.append(_new_plan(plan, {v: (Alloc((0, 0, 0), (re2, ne2, g_ext)), (d2, p2, t2), mb2)}))
            # cache hits are merged before fresh results (optimizer.py:1151-1166): equal scores resolve that way
            hits = [c for c in cands if key(c) in seen]
            fresh = [c for c in cands if key(c) not in seen]
            for cand in hits + fresh:
                ev = cached(cand)
                if not ev.mem_ok:
                    continue
                if ev.score > best_s:
                    best_s, best_plan = ev.score, cand
            if best_plan is not None:
                plan, score, improved = best_plan, best_s, True
        if not improved:
            break
    return plan, score, rounds, len(seen)
