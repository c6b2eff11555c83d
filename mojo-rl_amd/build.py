"""Builds libmrl_hip.so for gfx950 with hipcc (cross-compiles without a GPU)."""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libmrl_hip.so")
SOURCES = ["mrl_core.hip", "mrl_env.hip", "mrl_mlp.hip", "mrl_mlp3.hip", "mrl_ppo.hip", "mrl_policy.hip", "mrl_rollout.hip", "mrl_collect.hip", "mrl_update.hip"]
# -ffp-contract=off: fp32/fp64 results follow the written order of operations (the GEMM inner
# loops spell out fmaf / MFMA themselves).  The -target-feature pair switches packed-fp32
# code generation off.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-value"]


def build(verbose=False):
    srcs = [os.path.join(CSRC, s) for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    cmd = ["hipcc"] + FLAGS + ["-o", LIB] + srcs
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
