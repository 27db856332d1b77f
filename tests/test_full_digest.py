"""The WHOLE seeded candidate sets of configurations 1-4 (4,096 / 65,536 / 262,144 / 1,048,576 plans), and the first
16,384 seeded plans of configuration 5 (the annealing configuration, which has no fixed set), against digests
the reference itself wrote (tests/golden/ref_full_cfg{c}.json, make_golden_full.py): per chunk of 4,096 plans the CRC
of every makespan, peak, score (with and without the stale-layout gate) and feasibility flag, the best plan and the 32
best plans in ranking order.  Bit-exact; a mismatch names its chunk."""

import importlib.util
import json
import os

import numpy as np
import pytest

from rpeg_amd import configs
from rpeg_amd.engine import abi
from tests.helpers import GOLDEN, seeded_batch


def _generator():
    spec = importlib.util.spec_from_file_location("make_golden_full", os.path.join(GOLDEN, "make_golden_full.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _gold(c):
    path = os.path.join(GOLDEN, f"ref_full_cfg{c}.json" if c != 5 else "ref_full_cfg5_first16384.json")
    if not os.path.exists(path):
        pytest.skip(f"{os.path.basename(path)} has not been generated")
    with open(path) as f:
        return json.load(f)


def check(gold, plain, gated):
    """`plain` / `gated`: outputs without / with the stale-layout gate (dicts of makespan, peak, score, mask)."""
    gen = _generator()
    n = gold["n"]
    assert np.all((plain["mask"] & abi.MASK_VALID) != 0) and not np.any(plain["mask"] & abi.MASK_ERROR)
    flags = ((plain["mask"] & abi.MASK_MEM_OK) != 0).astype(np.uint8) | \
        (((plain["mask"] & abi.MASK_STALE_OK) != 0).astype(np.uint8) << 1)
    got = gen.digest(plain["makespan"], plain["peak"], plain["score"], gated["score"], flags,
                     np.full((n, 3), -1, np.int16))
    for k, (a, b) in enumerate(zip(got["chunks"], gold["chunks"])):
        assert a[:5] == b[:5], f"chunk {k} (plans {k * gold['chunk']}..): makespan, peak, score, gated score, flags"
    for key in ("n", "argmax", "argmax_gated", "top", "top_gated", "best", "best_gated", "n_feasible", "n_stale_ok"):
        assert got[key] == gold[key], key
    assert np.array_equal(gated["makespan"].view(np.uint64), plain["makespan"].view(np.uint64))


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_host_build_equals_reference_digest(c):
    """The host build of the kernels' arithmetic headers (the checker of the full-size GPU tests) on the whole set."""
    from oracle.cpu_port import CpuPort
    gold = _gold(c)
    cfg, batch = seeded_batch(c, gold["n"])
    port = CpuPort(cfg.problem)
    check(gold, port.eval(batch, flags=0, threads=8), port.eval(batch, flags=abi.GATE_STALE, threads=8))


@pytest.mark.gpu
@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_full_sets_equal_reference_digest(c):
    from rpeg_amd.engine.runtime import Engine
    gold = _gold(c)
    cfg, batch = seeded_batch(c, gold["n"])
    eng = Engine(cfg.problem)
    try:
        for _ in range(2):     # the second call runs the layout the engine learned from the first
            check(gold, eng.eval(batch, gate_stale=False), eng.eval(batch, gate_stale=True))
    finally:
        eng.close()


@pytest.mark.gpu
@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_violating_devices_of_the_first_chunk_equal_reference(c):
    """The device mem_worst_violation names for each plan of the first chunk (4,096 plans), through the drop-in
    `lower` and `mem_worst_violation`: the CRC of all of them equals the one the reference's own run recorded."""
    import rpeg_amd.compat as compat
    gen, gold = _generator(), _gold(c)
    m = min(gold["n"], gold["chunk"])
    cfg, batch = seeded_batch(c, m)
    p = cfg.problem
    compat.install()
    try:
        from model.memory import NodeMemoryModel, mem_worst_violation
        from passes.lower import lower
        device = np.full((m, 3), -1, np.int16)
        for i in range(m):
            rpeg, plan, wl = batch.configuration(p, i)
            lowered = lower(rpeg, None, plan, p.suite, 1, workload=wl)
            mm = NodeMemoryModel.from_policy(p.hw, p.suite, wl, p.memory_policy, trainable=frozenset(rpeg.trainable))
            v = mem_worst_violation(lowered, mm)
            if v is not None:
                device[i] = v[0]
    finally:
        compat.uninstall()
    import zlib
    assert zlib.crc32(np.ascontiguousarray(device, "<i2").tobytes()) == gold["chunks"][0][5]
