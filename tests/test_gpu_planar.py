"""GPU parity: HopperPlanar / Walker2dPlanar (reset, step, selective reset, auto-reset) through the C ABI
against the oracle.

These envs compute in Float64.  Joint angles and velocities, the torso's velocity, the counters, the
done flags and the reset rows involve no transcendental function and are compared bit for bit.  The
bodies' positions go through sin / cos of Float64, where the device's routine and the host libm's may
round differently in the last place; the torso's height takes up such a difference through the ground
push.  Tolerances: positions and heights 1e-14 absolute (values are of order 1, up to 384 sub-steps; measured: below 1e-15), fp32
observation entry 0 (height) and the rewards one fp32 unit in the last place.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def ctx(mrl):
    return mrl.DeviceContext("cuda:0")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def envs(mrl):
    return {0: mrl.HopperPlanar, 1: mrl.Walker2dPlanar}


def split(E, rows):
    """(obs fp32, doubles) views of host rows [batch, STATE]."""
    rows = np.ascontiguousarray(rows, np.float32)
    return rows[:, :E.OBS_DIM], rows[:, E.OBS_DIM + 1:].copy().view(np.float64)


def compare_rows(E, got, want, what):
    nj = E.ACTION_DIM
    og, dg = split(E, got)
    ow, dw = split(E, want)
    exact = np.ones(dw.shape[1], bool)
    exact[1] = False                       # torso height
    exact[6:6 + 3 * nj] = False            # body positions (their angles are sums of joint angles: exact)
    exact[8:6 + 3 * nj:3] = True
    exact[6 + 5 * nj + 2] = False          # total reward
    bad = dg[:, exact].view(np.uint64) != dw[:, exact].view(np.uint64)
    assert not bad.any(), "%s: %d exact doubles differ, first at %s" % (what, int(bad.sum()), np.argwhere(bad)[0])
    np.testing.assert_allclose(dg[:, ~exact], dw[:, ~exact], rtol=0, atol=1e-14, err_msg=what)
    assert np.array_equal(og[:, 1:].view(np.uint32), ow[:, 1:].view(np.uint32)), what + ": observation"
    np.testing.assert_allclose(og[:, 0], ow[:, 0], rtol=1.2e-7, atol=0, err_msg=what + ": height entry")
    return float(np.abs(dg - dw).max())


def actions(rng, batch, nj, t):
    a = rng.uniform(-1.3, 1.3, (batch, nj)).astype(np.float32)
    a[::3] = -1.0            # every third row folds its legs and falls: episodes end
    return a


@pytest.mark.parametrize("which,batch,seed", [(0, 1, 1), (0, 37, 2), (0, 4096, 3), (1, 1, 4), (1, 37, 5), (1, 4096, 6)])
def test_planar_reset_and_rollout_parity(mrl, orc, ctx, which, batch, seed):
    E = envs(mrl)[which]
    S, OBS, nj = E.STATE_SIZE, E.OBS_DIM, E.ACTION_DIM
    say("planar env", E.__name__, "batch", batch)
    s_h = np.zeros((batch, S), np.float32)
    orc.orc_planar_reset_batch(which, s_h.reshape(-1), None, batch, seed)
    s = torch.full((batch * S,), 7.0, device="cuda")          # garbage: the reset must write every float
    E.reset_kernel_gpu(ctx, s, seed)
    ctx.synchronize()
    got = s.cpu().numpy().reshape(batch, S)
    assert np.array_equal(got.view(np.uint32), s_h.view(np.uint32)), "reset rows differ"
    a = torch.zeros(batch * nj, device="cuda")
    r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch * OBS))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, OBS), np.float32)
    rng = np.random.default_rng(seed)
    n_done, worst = 0, 0.0
    for t in range(64 if which == 0 else 96):   # the walker's weaker motors take longer to fold its legs
        act = actions(rng, batch, nj, t)
        a.copy_(dev(act.reshape(-1)))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_planar_step_batch(which, s_h.reshape(-1), act.reshape(-1), r_h, d_h, o_h.reshape(-1), batch, 8)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, S)
        worst = max(worst, compare_rows(E, sg, s_h, "step %d" % t))
        assert torch.equal(o.view(batch, OBS), s.view(batch, S)[:, :OBS])
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_allclose(r.cpu().numpy(), r_h, rtol=1.2e-7, atol=1e-7)
        n_done += int(d_h.sum())
        dn = d_h.copy()
        E.selective_reset_kernel_gpu(ctx, s, d, 500 + t)
        orc.orc_planar_reset_batch(which, s_h.reshape(-1), dn.ctypes.data, batch, 500 + t)
        ctx.synchronize()
        compare_rows(E, s.cpu().numpy().reshape(batch, S), s_h, "after reset, step %d" % t)
        assert d.sum().item() == 0        # the selective reset clears the flags it has served
    say("  finished rows", n_done, "largest difference of a Float64 entry", worst)
    if batch > 100:
        assert n_done >= batch // 4


@pytest.mark.parametrize("which", [0, 1])
def test_planar_single_step_from_identical_rows(mrl, orc, ctx, which):
    """One step from rows the oracle made (poses over the whole joint range, feet in and out of the
    ground, torsos near the health thresholds): what differs after one step is only what sin / cos
    rounding explains: a few units in the last place of a position."""
    E = envs(mrl)[which]
    S, OBS, nj = E.STATE_SIZE, E.OBS_DIM, E.ACTION_DIM
    batch = 2048
    rng = np.random.default_rng(17 + which)
    s_h = np.zeros((batch, S), np.float32)
    orc.orc_planar_reset_batch(which, s_h.reshape(-1), None, batch, 3)
    dbl = s_h[:, OBS + 1:].view(np.float64)          # a view: writes land in s_h
    lim = [(-2.61799, 0.0), (-2.61799, 0.0), (-0.785398, 0.785398)] if which == 0 else [(-1.0, 0.7), (-1.2, 0.0), (-0.5, 0.5)]
    for j in range(nj):
        dbl[:, 6 + 3 * nj + j] = rng.uniform(lim[j % 3][0] - 0.01, lim[j % 3][1] + 0.01, batch)
        dbl[:, 6 + 4 * nj + j] = rng.uniform(-3, 3, batch)
    dbl[:, 0] = rng.uniform(-5, 5, batch)
    dbl[:, 1] = rng.uniform(0.6, 2.1, batch)
    dbl[:, 2] = rng.uniform(-1.1, 1.1, batch) * (rng.random(batch) < 0.3)
    dbl[:, 3] = rng.uniform(-1, 1, batch)
    dbl[:, 4] = rng.uniform(-2, 1, batch)
    s = dev(s_h.reshape(-1))
    act = rng.uniform(-1.5, 1.5, (batch, nj)).astype(np.float32)
    r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch * OBS))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, OBS), np.float32)
    E.step_kernel_gpu(ctx, s, dev(act.reshape(-1)), r, d, o, 0)
    orc.orc_planar_step_batch(which, s_h.reshape(-1), act.reshape(-1), r_h, d_h, o_h.reshape(-1), batch, 8)
    ctx.synchronize()
    sg = s.cpu().numpy().reshape(batch, S)
    _, dg = split(E, sg)
    _, dw = split(E, s_h)
    ulp = np.abs(dg - dw) / np.spacing(np.maximum(np.abs(dw), 0.25))
    say("  ", E.__name__, "one step: entries that differ", int((dg != dw).sum()), "of", dg.size, "largest",
        float(ulp.max()), "units in the last place; done rows", int(d_h.sum()))
    assert ulp.max() <= 16
    compare_rows(E, sg, s_h, "single step")
    np.testing.assert_array_equal(d.cpu().numpy(), d_h)
    assert 0.05 * batch < d_h.sum() < 0.95 * batch
    np.testing.assert_allclose(r.cpu().numpy(), r_h, rtol=1.2e-7, atol=1e-7)


@pytest.mark.parametrize("which", [0, 1])
def test_planar_done_rows_stay_untouched_and_autoreset(mrl, ctx, which):
    E = envs(mrl)[which]
    S, OBS, nj = E.STATE_SIZE, E.OBS_DIM, E.ACTION_DIM
    batch = 300
    done_at = OBS + 1 + 2 * (6 + 5 * nj + 1)
    s = torch.zeros(batch * S, device="cuda")
    E.reset_kernel_gpu(ctx, s, 9)
    s.view(batch, S)[::2, done_at + 1] = 1.875        # upper half of the double 1.0
    before = s.clone()
    a = torch.ones(batch * nj, device="cuda")
    r, d, o = (torch.full((n,), 5.0, device="cuda") for n in (batch, batch, batch * OBS))
    E.step_kernel_gpu(ctx, s, a, r, d, o, 0)
    ctx.synchronize()
    bits = lambda x: x.view(torch.int32).view(batch, S)
    assert torch.equal(bits(s)[::2], bits(before)[::2])
    assert (r[::2] == 0).all() and (d[::2] == 1).all() and (d[1::2] == 0).all()
    assert not torch.equal(bits(s)[1::2], bits(before)[1::2])
    assert torch.equal(o.view(batch, OBS), s.view(batch, S)[:, :OBS])
    # auto-reset = step, then selective reset, observation of the row as it stands afterwards
    s1 = torch.zeros(batch * S, device="cuda")
    E.reset_kernel_gpu(ctx, s1, 5)
    s2 = s1.clone()
    bufs = lambda: tuple(torch.zeros(n, device="cuda") for n in (batch, batch, batch * OBS))
    r1, d1, o1 = bufs(); r2, d2, o2 = bufs()
    g = torch.Generator(device="cuda").manual_seed(1)
    ended = 0
    for t in range(100):
        a = torch.rand(batch * nj, device="cuda", generator=g) * 2 - 1
        a.view(batch, nj)[::2] = -1.0
        E.step_kernel_gpu(ctx, s1, a, r1, d1, o1, t)
        ended += int(d1.sum().item())
        E.selective_reset_kernel_gpu(ctx, s1, d1.clone(), 50 + t)
        E.step_autoreset_kernel_gpu(ctx, s2, a, r2, d2, o2, t, 50 + t)
        ctx.synchronize()
        # rows as bit patterns: the halves of a double read as floats include NaN patterns
        assert torch.equal(s1.view(torch.int32), s2.view(torch.int32)) and torch.equal(r1, r2) and torch.equal(d1, d2)
        assert torch.equal(o2.view(batch, OBS), s2.view(batch, S)[:, :OBS])
    assert ended >= batch // 4
    with pytest.raises(mrl.MrlError, match="8-byte"):
        E.reset_kernel_gpu(ctx, torch.zeros(batch * S + 1, device="cuda")[1:], 1)


def test_continuous_agent_runs_on_the_planar_envs(mrl, ctx):
    for E in (mrl.HopperPlanar, mrl.Walker2dPlanar):
        agent = mrl.DeepPPOContinuousAgent(obs_dim=E.OBS_DIM, action_dim=E.ACTION_DIM, hidden_dim=64, rollout_len=32,
                                           n_envs=256, gpu_minibatch_size=1024, num_epochs=2, target_kl=0.0,
                                           init_seed=5)
        m = agent.train_gpu(ctx, E, num_episodes=10**9, max_rollouts=2, seed=3)
        assert m.rollouts == 2 and m.total_steps == 2 * 32 * 256
        assert torch.isfinite(agent.actor.params).all() and torch.isfinite(agent.rb.r_rewards).all()
        assert torch.isfinite(agent.rb.states.view(256, E.STATE_SIZE)[:, :E.OBS_DIM]).all()
