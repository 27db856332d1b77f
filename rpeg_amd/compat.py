"""Import-path drop-in: the reference's module names for this package's modules.

The reference is a source tree put on `sys.path`, so its call sites read `from search.evaluate import evaluate`,
`from ir.plan import ExecutionPlan`, `from core.types import Allocation` (RPEG/search/optimizer.py:16-29,
pipeline.py:40-60).  `install()` makes those statements resolve to `rpeg_amd.*`:

    import rpeg_amd.compat
    rpeg_amd.compat.install()
    from search.optimizer import optimize, polish, OptimizerConfig     # the GPU engine behind the same names

Registered: core.types; ir.plan, ir.rpeg, ir.ppo, ir.grpo, ir.dpo, ir.ac_share, ir.serialize; model.cost,
model.hardware, model.memory, model.models, model.workload; passes.unroll, passes.lower; schedule.scheduler,
schedule.trace; search.cache, search.evaluate, search.inter_model, search.moves, search.optimizer.  (The search
part of pipeline.py is rpeg_amd.search.pipeline.search_plan; it has no module of the reference's tree to stand
for.)  With them the call sequence of the reference's pipeline runs on the engine:

    lowered = lower(rpeg, unroll(rpeg, K_eval), plan, suite, K_eval, workload=workload)
    trace = schedule(executable=lowered, cost_model=NodeCostModel(hw, suite, workload), device_space=space)
    violation = mem_worst_violation(lowered, NodeMemoryModel(hw, suite, workload, trainable=...))
    t = cost_model.time(node)

Not registered: passes.transfer_resources (the reservations are `Trace.reserved_allocations`) and the reference's
runtime, scripts and logging packages.
"""

from __future__ import annotations

import importlib
import sys
import types

PACKAGES = ("core", "ir", "model", "passes", "schedule", "search")
MODULES = ("core.types",
           "ir.plan", "ir.rpeg", "ir.ppo", "ir.grpo", "ir.dpo", "ir.ac_share", "ir.serialize",
           "model.cost", "model.hardware", "model.memory", "model.models", "model.workload",
           "passes.unroll", "passes.lower", "schedule.scheduler", "schedule.trace",
           "search.cache", "search.evaluate", "search.inter_model", "search.moves", "search.optimizer")
_installed: dict = {}


def install(force: bool = False) -> None:
    """Registers the names above in sys.modules.  A name that is already taken by another module -- the reference
    tree itself is on the path and was imported, or an unrelated package called `model` or `search` -- raises
    ImportError unless `force`, in which case it is replaced (and put back by `uninstall`)."""
    taken = [n for n in PACKAGES + MODULES if n in sys.modules and n not in _installed]
    if taken and not force:
        raise ImportError("already imported from elsewhere: " + ", ".join(taken) +
                          " (call install(force=True) to replace them for this process)")
    for name in PACKAGES:
        real = importlib.import_module("rpeg_amd." + name)
        pkg = types.ModuleType(name, f"rpeg_amd.{name} under the reference's name")
        pkg.__path__ = []                      # a package with no directory: only the registered modules exist
        pkg.__package__ = name
        pkg.__rpeg_amd__ = real
        _register(name, pkg)
    for name in MODULES:
        mod = importlib.import_module("rpeg_amd." + name)
        _register(name, mod)
        setattr(sys.modules[name.split(".")[0]], name.split(".")[1], mod)


def _register(name: str, module) -> None:
    if name not in _installed:
        _installed[name] = sys.modules.get(name)
    sys.modules[name] = module


def uninstall() -> None:
    """Takes the names out again (what they named before comes back)."""
    for name, before in _installed.items():
        if before is None:
            sys.modules.pop(name, None)
        else:
            sys.modules[name] = before
    _installed.clear()


def installed() -> bool:
    return bool(_installed)
