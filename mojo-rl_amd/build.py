"""Builds libmrl_hip.so for gfx950 with hipcc (cross-compiles without a GPU): one object per
translation unit, compiled side by side, then linked."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(HERE, "libmrl_hip.so")
SOURCES = ["mrl_core.hip", "mrl_env.hip", "mrl_mlp.hip", "mrl_mlp3.hip", "mrl_ppo.hip", "mrl_policy.hip", "mrl_rollout.hip", "mrl_collect.hip", "mrl_collect_walkers.hip", "mrl_update.hip", "mrl_shuffle.hip"]
# -ffp-contract=off: fp32/fp64 results follow the written order of operations (the GEMM inner
# loops spell out fmaf / MFMA themselves).  The -target-feature pair switches packed-fp32
# code generation off.
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wno-unused-value"]
# The collection kernels run a long env step inside a loop over the rollout steps.  The machine-level
# loop-invariant code motion lifts the double-precision constants of that step (the polynomial
# coefficients of exp / log / sincos, two registers each) out of the loop into registers of their own,
# the register allocator then spills them, and every use becomes a dependent load from private memory in
# the middle of the solver wavefront's chain.  Without that pass these kernels need no private memory.
EXTRA_FLAGS = {"mrl_collect.hip": ["-mllvm", "-disable-machine-licm"],
               "mrl_collect_walkers.hip": ["-mllvm", "-disable-machine-licm"]}


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops' is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)


def build(verbose=False, incremental=False, jobs=8):
    """Compiles every translation unit (incremental=True: only those older than a source or header
    they could include) and links the library."""
    os.makedirs(OBJ, exist_ok=True)
    headers = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    headers.append(os.path.join(HERE, "..", "include", "mrl.h"))
    newest_header = max(os.path.getmtime(h) for h in headers)
    todo, objs = [], []
    for s in SOURCES:
        src, obj = os.path.join(CSRC, s), os.path.join(OBJ, s[:-4] + ".o")
        objs.append(obj)
        fresh = os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(src), newest_header)
        if not (incremental and fresh):
            todo.append(["hipcc"] + FLAGS + EXTRA_FLAGS.get(s, []) + ["-c", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(lambda c: _run(c, verbose), todo))
    _run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs, verbose)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True, incremental="--incremental" in sys.argv))
    sys.exit(0)
