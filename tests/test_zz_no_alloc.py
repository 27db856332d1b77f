"""The entry point that allocates nothing (rpeg_eval_batch_static) against rpeg_eval_batch, through the C ABI.

Bar: every output bit for bit, masks equal.  Two calls in a row on one engine, the second with a smaller
batch (the file-scope scratch array keeps the first call's contents), then the error statuses."""

import ctypes as C

import numpy as np
import pytest

from rpeg_amd import configs
from rpeg_amd.engine import abi
from tests.helpers import seeded_batch

pytestmark = pytest.mark.gpu


def bits(t):
    return t.cpu().numpy().view(np.uint64 if t.element_size() == 8 else np.uint8)


def compare(eng, db, n, gate_stale=True):
    import torch
    want = eng.eval_device(db, n=n, gate_stale=gate_stale)
    torch.cuda.synchronize()
    got = eng.alloc_outputs(n)
    for t in got.values():      # whatever the call does not write would show
        t.fill_(7)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    eng.eval_device_static(db, out=got, n=n, gate_stale=gate_stale)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before      # the call took no device memory
    assert eng.stats()["quad_tasks"] == 0 and eng.stats()["wave_tasks"] == n
    for k in ("makespan", "peak", "score", "mask"):
        assert np.array_equal(bits(got[k]), bits(want[k])), (k, n)
    return want


@pytest.mark.parametrize("c,n1,n2", [(2, 8192, 1000), (1, 4096, 37), (4, 32768, 5)])
def test_static_entry_equals_eval_batch_twice(c, n1, n2):
    from rpeg_amd.engine.runtime import DeviceBatch, Engine
    cfg, batch = seeded_batch(c, n1)
    # some plans that break an integer rule: they are skipped by the evaluation kernel
    batch.vert[3, 5] = 3      # micro-batch count of vertex 0 of plan 5 (pp == 1 needs 1, else a divisor)
    batch.vert[0, 11] = 7     # dp of vertex 0 of plan 11 does not divide the batch
    eng = Engine(cfg.problem)
    db = DeviceBatch(batch)
    first = compare(eng, db, n1)
    assert int(first["mask"][5]) == 0 or int(first["mask"][11]) == 0
    # a smaller batch right after: a suffix of the same tensors, other stale-layout handling
    sub = DeviceBatch(batch.take(np.arange(n1 - n2, n1)))
    compare(eng, sub, n2, gate_stale=False)
    compare(eng, db, n1)
    eng.close()


def test_static_entry_rejects_what_it_cannot_do():
    from rpeg_amd.engine.runtime import DeviceBatch, Engine, EngineError
    cfg, batch = seeded_batch(2, abi.STATIC_MAX_PLANS + 1)
    eng = Engine(cfg.problem)
    db = DeviceBatch(batch)
    with pytest.raises(EngineError, match="not on the device"):      # no rpeg_eval_batch call yet
        eng.eval_device_static(db, n=64)
    eng.eval_device(db, n=64)
    with pytest.raises(EngineError, match="at most 32768 plans"):
        eng.eval_device_static(db)
    # classes the engine has not met: status -11, the known plans still get their results
    import torch
    out = eng.alloc_outputs(4096)
    with pytest.raises(EngineError, match="has not met"):
        eng.eval_device_static(db, out=out, n=4096)
    torch.cuda.synchronize()
    want = eng.eval_device(db, n=4096)
    torch.cuda.synchronize()
    m = out["mask"].cpu().numpy()
    unknown = (m & abi.MASK_ERROR) != 0
    assert unknown.any() and not unknown[:64].any()
    assert np.array_equal(bits(out["score"])[~unknown], bits(want["score"])[~unknown])
    assert np.isnan(out["score"].cpu().numpy()[unknown]).all()
    eng.eval_device_static(db, out=out, n=4096)      # now every class is known
    torch.cuda.synchronize()
    assert np.array_equal(bits(out["score"]), bits(want["score"]))
    eng.close()


def test_two_engines_share_the_array_in_turn():
    """Two engines on one GPU call the static entry alternately (sequentially): each finds the other's task list and
    counters in the shared array and must not be misled by them."""
    from rpeg_amd.engine.runtime import DeviceBatch, Engine
    cfg_a, batch_a = seeded_batch(2, 6000)
    cfg_b, batch_b = seeded_batch(4, 900)
    eng_a, eng_b = Engine(cfg_a.problem), Engine(cfg_b.problem)
    da, db = DeviceBatch(batch_a), DeviceBatch(batch_b)
    for _ in range(2):
        compare(eng_a, da, 6000)
        compare(eng_b, db, 900)
    eng_a.close()
    eng_b.close()


def test_static_entry_inside_a_captured_graph():
    """With RPEG_NO_WAIT the call is three kernel launches and nothing else, so it may stand inside a stream capture
    (which rejects allocations, copies to pageable memory and waits).  The captured graph is replayed several times on
    the same buffers, with eager work and synchronisations between the replays and changed inputs, and every replay
    is held to the eager rpeg_eval_batch result."""
    import torch
    from rpeg_amd.engine.runtime import DeviceBatch, Engine
    n = 5000
    cfg, batch = seeded_batch(2, 2 * n)
    eng = Engine(cfg.problem)
    whole = DeviceBatch(batch)
    eng.eval_device(whole)                        # every class of the set is on the device
    torch.cuda.synchronize()
    first, second = batch.slice(0, n), batch.slice(n, 2 * n)
    db = DeviceBatch(first)
    out = eng.alloc_outputs(n)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        eng.eval_device_static(db, out=out, n=n, no_wait=True)
    for k, src in enumerate((first, second, first, second)):
        db.vert.copy_(torch.from_numpy(np.ascontiguousarray(src.vert)))      # eager work between the replays
        db.head.copy_(torch.from_numpy(np.ascontiguousarray(src.head)))
        for t in out.values():
            t.fill_(3)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = eng.eval_device(DeviceBatch(src))
        torch.cuda.synchronize()
        for key in ("makespan", "peak", "score", "mask"):
            assert np.array_equal(bits(out[key]), bits(want[key])), (k, key)
    eng.close()
