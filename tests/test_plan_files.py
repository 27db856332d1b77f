"""Plan files and configuration files: the reference's schemas.  Plan artifacts are compared with
what the reference's own ir/serialize.py wrote for the same plans (tests/golden/make_golden_plans.py)."""

import json
import os

import pytest

from rpeg_amd import config_io, configs
from rpeg_amd.ir import serialize as ser
from rpeg_amd.search.evaluate import Configuration
from tests.helpers import GOLDEN, seeded_batch

CONFIG_DIR = os.path.join(os.path.dirname(os.path.abspath(config_io.__file__)), "config_files")


def _gold():
    with open(os.path.join(GOLDEN, "ref_plans.json")) as f:
        return json.load(f)


def _configuration(c, i):
    cfg, batch = seeded_batch(c, 3)
    rpeg, plan, wl = batch.configuration(cfg.problem, i)
    return cfg, Configuration(rpeg, plan, cfg.problem.device_space), wl


@pytest.mark.parametrize("c,algo", [(1, "PPO"), (2, "GRPO"), (4, "DPO")])
def test_optimized_plan_artifact_equals_reference(c, algo, tmp_path):
    for rec in _gold()[str(c)]:
        cfg, config, wl = _configuration(c, rec["i"])
        got = ser.optimized_plan_to_dict(config, algo, wl, source_config_hash="sha256:test")
        assert got == rec["optimized"]
        assert list(got) == list(rec["optimized"])                      # key order of the artifact
        assert got["plan_hash"] == rec["optimized"]["plan_hash"]
        for ext in ("json", "yaml"):
            path = str(tmp_path / f"plan{rec['i']}.{ext}")
            ser.save_optimized_plan(config, path, algo, wl, source_config_hash="sha256:test")
            assert ser.load_optimized_plan(path) == rec["optimized"]
            plan = ser.load_plan(path, config.rpeg)
            assert plan.sigma == config.plan.sigma and plan.pi == config.plan.pi and plan.mb == config.plan.mb
            ser.save_plan(config, path)
            assert ser.load_plan(path, config.rpeg).pi == config.plan.pi
            with pytest.raises(ValueError):
                ser.load_optimized_plan(path)                           # the plain schema has no version


def test_plan_hash_covers_every_field():
    cfg, config, wl = _configuration(1, 0)
    a = ser.optimized_plan_to_dict(config, "ppo", wl)
    v = config.rpeg.vertices[0]
    config.plan.mb[v] = config.plan.mb[v] + 1
    b = ser.optimized_plan_to_dict(config, "ppo", wl)
    assert a["plan_hash"] != b["plan_hash"]
    sched = {"policy": "x", "horizon": 1, "predicted_makespan_s": 1.0, "nodes": []}
    c = ser.optimized_plan_to_dict(config, "ppo", wl, execution_schedule=sched)
    assert c["plan_hash"] != b["plan_hash"] and list(c)[-1] == "execution_schedule"
    with pytest.raises(ValueError):
        ser.execution_schedule_to_dict(None, horizon=0)


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
def test_config_files_describe_the_benchmark_problems(c):
    cfg = config_io.load_config(os.path.join(CONFIG_DIR, f"cfg{c}.yaml"))
    config_io.validate_config(cfg)
    p = config_io.problem_from_config(cfg)
    want = configs.config(c).problem
    assert p.device_space == want.device_space and p.workload == want.workload and p.hw == want.hw
    assert p.K_eval == want.K_eval and p.suite.specs == want.suite.specs
    assert p.structures[0].name == want.structures[0].name


def test_config_loader_and_validation(tmp_path):
    text = open(os.path.join(CONFIG_DIR, "cfg5.yaml")).read().replace("flops_per_gpu: 440000000000000.0",
                                                                       "flops_per_gpu: 440e12")
    path = str(tmp_path / "c.yaml")
    open(path, "w").write(text)
    cfg = config_io.load_config(path)
    assert cfg["hardware"]["flops_per_gpu"] == 4.4e14 and isinstance(cfg["hardware"]["flops_per_gpu"], float)
    opt = config_io.build_optimizer_config(cfg, allow_ac_share=False, algorithm="ppo")
    assert (opt.K_x, opt.T_init, opt.T_min, opt.T_warm, opt.stag_window) == (6, 0.05, 0.05, 0.10, 10)
    from rpeg_amd.core.types import Model
    assert opt.T_cand[Model.ACTOR] == {0, 1} and opt.T_cand[Model.CRITIC] == {0} and opt.T_cand[Model.AC_SHARE] == set()
    assert opt.T_cool == 1.0
    bad = dict(cfg, optimizer=dict(cfg["optimizer"], k_eval=0))
    with pytest.raises(ValueError):
        config_io.validate_config(bad)
    bad = dict(cfg, models={"actor": cfg["models"]["actor"]})
    with pytest.raises(ValueError):
        config_io.validate_config(bad)
    bad = dict(cfg, policy={"algorithm": "sac"})
    with pytest.raises(ValueError):
        config_io.validate_config(bad)
    grpo = config_io.build_optimizer_config(config_io.load_config(os.path.join(CONFIG_DIR, "cfg2.yaml")), False, "grpo")
    assert grpo.T_cand == {Model.ACTOR: {0, 1}}


def test_hardware_overlay_merges_like_the_reference(tmp_path):
    """The `--hw` overlay of RPEG/pipeline.py:1288-1302: key: value lines, comments and trailing comments dropped,
    non-numeric values ignored, later keys win over the configuration's."""
    from rpeg_amd import config_io
    path = tmp_path / "hw.yaml"
    path.write_text("# calibrated\n\nflops_per_gpu: 9.5e14   # measured\nmemory_bandwidth: 3.1e12\nname: mi355x\n"
                    "  gemm_m_half : 512\nnot a pair\n")
    cfg = {"hardware": {"flops_per_gpu": 1.0, "racks": 2}}
    out = config_io.merge_hardware_overlay(cfg, str(path))
    assert out is cfg
    assert cfg["hardware"] == {"flops_per_gpu": 9.5e14, "racks": 2, "memory_bandwidth": 3.1e12, "gemm_m_half": 512.0}
    assert config_io.merge_hardware_overlay({}, str(path))["hardware"]["memory_bandwidth"] == 3.1e12
