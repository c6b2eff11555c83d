"""Committed fixtures (tests/golden, written by tests/golden/make_golden.py) against the oracle
(CPU) and against the HIP path through the C ABI (GPU).

The trajectories were produced by this repository's oracle, not by the reference (which cannot
run here): they are regression anchors.  Observations, rewards, done flags and the final state rows
are compared bit for bit, for every environment, on the CPU (oracle) and on the GPU (HIP path),
with no resynchronisation between the 64 steps."""
import json
import os

import numpy as np
import pytest

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


@pytest.fixture(scope="module")
def traj():
    return np.load(os.path.join(GOLD, "trajectories.npz"))


def test_philox_kat_fixture(orc):
    with open(os.path.join(GOLD, "philox4x32_10_kat.json")) as f:
        kat = json.load(f)["vectors"]
    assert len(kat) == 3
    for v in kat:
        ctr = np.array([int(x, 16) for x in v["counter"]], np.uint32)
        key = np.array([int(x, 16) for x in v["key"]], np.uint32)
        out = np.zeros(4, np.uint32)
        orc.orc_philox4x32_10(ctr, key, out)
        assert ["%08x" % int(x) for x in out] == v["output"]


def test_adam_first_step_fixture(orc):
    with open(os.path.join(GOLD, "adam_first_step.json")) as f:
        g = json.load(f)
    p, grad, st = np.zeros(1, np.float32), np.array([g["grad"]], np.float32), np.zeros(2, np.float32)
    orc.orc_adam_step(p, grad, st, 1, 1, g["lr"], g["beta1"], g["beta2"], g["eps"])
    assert abs(st[0] - g["m_after"]) < g["tolerance"] and abs(st[1] - g["v_after"]) < g["tolerance"]
    # first Adam step moves a parameter by lr * sign(g) (bias corrections cancel)
    assert abs(p[0] + g["lr"]) < 1e-6


def _replay_oracle(orc, name, traj):
    A, O, R, D = (traj["%s_%s" % (name, k)] for k in ("actions", "obs", "rewards", "dones"))
    T, N = R.shape
    s = traj["%s_state0" % name].copy()
    steps = np.zeros(N, np.int32)
    r, d, o = np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros(O.shape[1:], np.float32)
    for t in range(T):
        a = np.ascontiguousarray(A[t].reshape(-1) if A.shape[2] == 1 else A[t])
        if name == "cartpole":
            orc.orc_cartpole_step_batch(s, steps, a, r, d, o, N)
        elif name == "pendulum":
            orc.orc_pendulum_step_batch(s, a, r, d, o, N)
        elif name == "lunar":
            orc.orc_ll_step_batch(s, a, r, d, o, N, 1)
        elif name == "bipedal":
            orc.orc_bw_step_batch(s, a, r, d, o, N, 1)
        else:
            orc.orc_hc_step_batch(s, a, r, d, o, N, 1)
        np.testing.assert_array_equal(o, O[t]); np.testing.assert_array_equal(r, R[t])
        np.testing.assert_array_equal(d, D[t])
        seed = 1000 + t
        if name == "cartpole":
            orc.orc_cartpole_selective_reset_batch(s, steps, d, N, seed)
        elif name == "pendulum":
            orc.orc_pendulum_selective_reset_batch(s, d, N, seed)
        elif name == "lunar":
            orc.orc_ll_selective_reset_batch(s, d, N, seed)
        elif name == "bipedal":
            orc.orc_bw_reset_batch(s, d.ctypes.data, N, seed)
        else:
            orc.orc_hc_reset_batch(s, d.ctypes.data, N, seed)
    np.testing.assert_array_equal(s, traj["%s_state_end" % name])


@pytest.mark.parametrize("name", ["cartpole", "pendulum", "lunar", "bipedal", "cheetah"])
def test_oracle_reproduces_golden_trajectories(orc, traj, name):
    _replay_oracle(orc, name, traj)


@pytest.mark.gpu
@pytest.mark.parametrize("name,cls", [("cartpole", "CartPoleEnv"), ("pendulum", "PendulumV2"), ("lunar", "LunarLanderV2"),
                                      ("bipedal", "BipedalWalkerV2"), ("cheetah", "HalfCheetahPlanarV2")])
def test_hip_path_reproduces_golden_trajectories(mrl, traj, name, cls):
    import torch
    ctx = mrl.DeviceContext("cuda:0")
    E = getattr(mrl, cls)
    A, O, R, D = (traj["%s_%s" % (name, k)] for k in ("actions", "obs", "rewards", "dones"))
    T, N = R.shape
    s = torch.from_numpy(traj["%s_state0" % name].copy()).cuda().reshape(-1)
    r, d, o = torch.zeros(N, device="cuda"), torch.zeros(N, device="cuda"), torch.zeros(O[0].size, device="cuda")
    if name == "cartpole":      # the step counters behind the 500-step truncation, in the caller's hands
        steps = torch.zeros(N, dtype=torch.int32, device="cuda")
        E.bind_step_counters(ctx, s, steps)
    for t in range(T):
        print(name, "step", t, flush=True)
        a = torch.from_numpy(np.ascontiguousarray(A[t].reshape(-1))).cuda()
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        ctx.synchronize()
        # no resynchronisation between steps: the whole trajectory has to stay on the oracle's bits
        np.testing.assert_array_equal(o.cpu().numpy().reshape(O[t].shape), O[t])
        np.testing.assert_array_equal(r.cpu().numpy(), R[t])
        np.testing.assert_array_equal(d.cpu().numpy(), D[t])
        E.selective_reset_kernel_gpu(ctx, s, d, 1000 + t)
    ctx.synchronize()
    np.testing.assert_array_equal(s.cpu().numpy().reshape(N, -1), traj["%s_state_end" % name])
    if name == "cartpole":
        # a counter holds the steps since its row's last reset
        since = np.array([T - 1 - (np.nonzero(D[:, i])[0].max() if D[:, i].any() else -1) for i in range(N)])
        np.testing.assert_array_equal(steps.cpu().numpy(), since)
