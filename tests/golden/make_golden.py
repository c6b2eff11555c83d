"""Writes the fixtures in this directory.

  philox4x32_10_kat.json   Random123's published known-answer vectors for philox4x32, 10 rounds
                           (kat_vectors in the Random123 distribution) -- typed in, not computed.
  adam_first_step.json     the first-step numbers the reference's own optimiser test expects
                           (tests/test_optimizers_cpu.mojo:178-189: g = 0.5 -> m = 0.05, v = 0.00025).
  trajectories.npz         64-step seeded trajectories of the five environments, 8 envs each,
                           produced by the CPU oracle in this repository (NOT by the reference,
                           which cannot run here): per step the actions fed in and the observations,
                           rewards and done flags that came out, with selective reset after each
                           step.  They freeze the oracle's behaviour, so a later change to the
                           oracle or to a kernel shows up as a diff against a committed file.

Run from the repository root:  python tests/golden/make_golden.py
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

N, T = 8, 64


def rollout(lib, name, rng):
    """Returns dict of arrays for one environment family."""
    from oracle import orc as orcmod  # noqa: F401
    out = {}
    if name == "cartpole":
        s = np.zeros((N, 4), np.float32); steps = np.zeros(N, np.int32)
        lib.orc_cartpole_reset_batch(s, steps, N, 12345)
        od, aw = 4, 1
    elif name == "pendulum":
        s = np.zeros((N, 8), np.float32)
        lib.orc_pendulum_reset_batch(s, N, 7)
        od, aw = 3, 1
    elif name == "lunar":
        s = np.zeros((N, 192), np.float32)
        lib.orc_ll_reset_batch(s, N, 7)
        od, aw = 8, 1
    elif name == "bipedal":
        s = np.zeros((N, 950), np.float32)
        lib.orc_bw_reset_batch(s, None, N, 7)
        od, aw = 24, 4
    else:
        s = np.zeros((N, 253), np.float32)
        lib.orc_hc_reset_batch(s, None, N, 7)
        od, aw = 17, 6
    out["state0"] = s.copy()
    A = np.zeros((T, N, aw), np.float32)
    O = np.zeros((T, N, od), np.float32)
    R = np.zeros((T, N), np.float32)
    D = np.zeros((T, N), np.float32)
    r, d, o = np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros((N, od), np.float32)
    for t in range(T):
        if name == "cartpole":
            a = rng.integers(0, 2, N).astype(np.float32)
            lib.orc_cartpole_step_batch(s, steps, a, r, d, o, N)
        elif name == "pendulum":
            a = rng.uniform(-1, 1, N).astype(np.float32)
            lib.orc_pendulum_step_batch(s, a, r, d, o, N)
        elif name == "lunar":
            a = rng.integers(0, 4, N).astype(np.float32)
            lib.orc_ll_step_batch(s, a, r, d, o, N, 1)
        elif name == "bipedal":
            a = rng.uniform(-1, 1, (N, 4)).astype(np.float32)
            lib.orc_bw_step_batch(s, a, r, d, o, N, 1)
        else:
            a = rng.uniform(-1, 1, (N, 6)).astype(np.float32)
            lib.orc_hc_step_batch(s, a, r, d, o, N, 1)
        A[t] = a.reshape(N, aw); O[t] = o; R[t] = r; D[t] = d
        seed = 1000 + t
        if name == "cartpole":
            lib.orc_cartpole_selective_reset_batch(s, steps, d, N, seed)
        elif name == "pendulum":
            lib.orc_pendulum_selective_reset_batch(s, d, N, seed)
        elif name == "lunar":
            lib.orc_ll_selective_reset_batch(s, d, N, seed)
        elif name == "bipedal":
            lib.orc_bw_reset_batch(s, d.ctypes.data, N, seed)
        else:
            lib.orc_hc_reset_batch(s, d.ctypes.data, N, seed)
    out.update(actions=A, obs=O, rewards=R, dones=D, state_end=s.copy())
    return out


def main():
    from oracle import orc as orcmod
    lib = orcmod.load()
    kat = [
        {"counter": ["00000000"] * 4, "key": ["00000000"] * 2,
         "output": ["6627e8d5", "e169c58d", "bc57ac4c", "9b00dbd8"]},
        {"counter": ["ffffffff"] * 4, "key": ["ffffffff"] * 2,
         "output": ["408f276d", "41c83b0e", "a20bc7c6", "6d5451fd"]},
        {"counter": ["243f6a88", "85a308d3", "13198a2e", "03707344"], "key": ["a4093822", "299f31d0"],
         "output": ["d16cfe09", "94fdcceb", "5001e420", "24126ea1"]},
    ]
    with open(os.path.join(HERE, "philox4x32_10_kat.json"), "w") as f:
        json.dump({"source": "Random123 kat_vectors, philox4x32 with 10 rounds", "vectors": kat}, f, indent=1)
    with open(os.path.join(HERE, "adam_first_step.json"), "w") as f:
        json.dump({"source": "tests/test_optimizers_cpu.mojo:178-189 of the reference",
                   "lr": 0.001, "beta1": 0.9, "beta2": 0.999, "eps": 1e-8, "grad": 0.5,
                   "m_after": 0.05, "v_after": 0.00025, "tolerance": 1e-5}, f, indent=1)
    arrays = {}
    for i, name in enumerate(("cartpole", "pendulum", "lunar", "bipedal", "cheetah")):
        rng = np.random.default_rng(100 + i)
        for k, v in rollout(lib, name, rng).items():
            arrays["%s_%s" % (name, k)] = v
    np.savez_compressed(os.path.join(HERE, "trajectories.npz"), **arrays)
    print("wrote", sorted(os.listdir(HERE)))


if __name__ == "__main__":
    main()
