"""Builds oracle/_build/libcpu_port.so: the host build of the evaluator's arithmetic (test
infrastructure, see cpu_port.cpp).  No reference sources are compiled: the reference is pure
Python, so there is nothing to build under oracle/_ref."""

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "_build", "libcpu_port.so")
FLOPS = os.path.join(HERE, "_build", "libflop_count.so")


def build(force: bool = False) -> str:
    src = os.path.join(HERE, "cpu_port.cpp")
    deps = [src, os.path.join(HERE, "flop_count.cpp")] + [os.path.join(HERE, "..", "rpeg_amd", "csrc", f) for f in
                    ("rpeg_core.h", "rpeg_class.h", "rpeg_lower.h", "rpeg_plan.h", "rpeg_sa.h", "rpeg_exp_table.inc")]
    deps.append(os.path.join(HERE, "..", "include", "rpeg_eval.h"))
    if not force and os.path.exists(OUT) and os.path.exists(FLOPS) and all(os.path.getmtime(OUT) >= os.path.getmtime(d) for d in deps):
        return OUT
    os.makedirs(os.path.dirname(OUT), exist_ok=True)
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fopenmp", "-ffp-contract=off", "-mfma",
           "-Wall", "-Wno-unknown-pragmas", "-o", OUT, src]
    subprocess.run(cmd, check=True)
    # the operation counter: the same headers with `double` replaced by a counting type (flop_count.cpp)
    subprocess.run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off", "-mfma", "-Wall",
                    "-Wno-unknown-pragmas", "-Wno-class-memaccess", "-o", FLOPS, os.path.join(HERE, "flop_count.cpp")], check=True)
    return OUT


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))
