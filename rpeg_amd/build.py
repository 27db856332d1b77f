"""Builds rpeg_amd/librpeg_eval.so (HIP kernels + C ABI) for gfx950 with hipcc.

The library is built in-tree; it has no CPU fallback and refuses to create an engine without a GPU.
"""

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "librpeg_eval.so")
SOURCES = [os.path.join(HERE, "csrc", "rpeg_engine.hip")]
HEADERS = [os.path.join(HERE, "csrc", f) for f in
           ("rpeg_core.h", "rpeg_class.h", "rpeg_lower.h", "rpeg_plan.h", "rpeg_sa.h", "rpeg_kernel_eval.h",
            "rpeg_kernel_plan.h", "rpeg_kernel_quad.h", "rpeg_exp_table.inc")] + \
          [os.path.join(HERE, "..", "include", "rpeg_eval.h")]

# -ffp-contract=off: scores must equal the reference's Python floats, which never fuse a*b+c.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-pthread", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function", "-Wno-unused-value", "-Wno-unused-result"]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    raise RuntimeError("hipcc not found")


PROFILE_LIB = os.path.join(HERE, "librpeg_eval_prof.so")   # the same library with the scheduling loop's section clocks


def build(force: bool = True, verbose: bool = False) -> str:
    if not force and os.path.exists(LIB) and all(os.path.getmtime(LIB) >= os.path.getmtime(f) for f in SOURCES + HEADERS):
        return LIB
    cmd = [hipcc()] + FLAGS + ["-o", LIB] + SOURCES
    if verbose:
        print(" ".join(cmd))
    subprocess.run(cmd, check=True)
    return LIB


def build_profile(verbose: bool = False) -> str:
    """The measurement build (-DKE_FINE_PROF): k_eval sums the shader clocks of the four sections of its
    scheduling loop per wavefront (rpeg_amd.engine.profile --sections reads them).  Not loaded by anything else."""
    cmd = [hipcc()] + FLAGS + ["-DKE_FINE_PROF", "-o", PROFILE_LIB] + SOURCES
    if verbose:
        print(" ".join(cmd))
    subprocess.run(cmd, check=True)
    return PROFILE_LIB


if __name__ == "__main__":
    import sys
    print(build_profile(verbose=True) if "--profile" in sys.argv else build(force=True, verbose=True))
