"""GPU parity: env kernels (through the C ABI) against the CPU oracle on identical seeded inputs.

Bar: per-step fp32 state and observations within 1e-5 relative (1e-6 absolute); reward and done
flags exact over the first 64 steps.
"""
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
RTOL, ATOL = 1e-5, 1e-6


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def ctx(mrl):
    return mrl.DeviceContext("cuda:0")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def close(a, b):
    np.testing.assert_allclose(a, b, rtol=RTOL, atol=ATOL)


def same_bits(a, b, what):
    """Bit-for-bit equality of two fp32 arrays (the kernels and the oracle run the same fp32 / fp64
    operations in the same order, contraction off on both sides)."""
    a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
    bad = a.view(np.uint32) != b.view(np.uint32)
    assert not bad.any(), "%s: %d of %d floats differ, first at %s: %r vs %r" % (
        what, int(bad.sum()), bad.size, np.argwhere(bad)[0], a[bad][0], b[bad][0])


@pytest.mark.parametrize("batch", [1, 63, 4096])
def test_cartpole_rollout_parity(mrl, orc, ctx, batch):
    say("cartpole batch", batch)
    E = mrl.CartPoleEnv
    s_h = np.zeros((batch, 4), np.float32); st_h = np.zeros(batch, np.int32)
    orc.orc_cartpole_reset_batch(s_h, st_h, batch, 12345)
    s = torch.zeros(batch * 4, device="cuda")
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch, batch * 4))
    E.reset_kernel_gpu(ctx, s, 0)
    ctx.synchronize()
    np.testing.assert_array_equal(s.cpu().numpy().reshape(batch, 4), s_h)
    rng = np.random.default_rng(0)
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 4), np.float32)
    for t in range(64):
        act = rng.integers(0, 2, batch).astype(np.float32)
        a.copy_(dev(act))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_cartpole_step_batch(s_h, st_h, act, r_h, d_h, o_h, batch)
        ctx.synchronize()
        close(s.cpu().numpy().reshape(batch, 4), s_h)
        close(o.cpu().numpy().reshape(batch, 4), o_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        seed = 1000 + t
        E.selective_reset_kernel_gpu(ctx, s, d, seed)
        orc.orc_cartpole_selective_reset_batch(s_h, st_h, d_h, batch, seed)
        ctx.synchronize()
        np.testing.assert_array_equal(s.cpu().numpy().reshape(batch, 4), s_h)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)


def test_cartpole_caller_owned_step_counters(mrl, ctx):
    """Step counters bound by the caller travel with the rows: a copy of the rows, bound to a copy of
    the counters, carries on exactly like the original -- including the 500-step truncation."""
    batch = 64
    E = mrl.CartPoleEnv
    s1 = torch.zeros(batch * 4, device="cuda")
    steps1 = torch.full((batch,), 495, dtype=torch.int32, device="cuda")
    E.bind_step_counters(ctx, s1, steps1)
    bufs = lambda: tuple(torch.zeros(n, device="cuda") for n in (batch, batch, batch * 4))
    r1, d1, o1 = bufs(); r2, d2, o2 = bufs()
    act = lambda t: ((torch.arange(batch, device="cuda") + t) % 2).float()       # push left and right in turn
    for t in range(3):
        E.step_kernel_gpu(ctx, s1, act(t), r1, d1, o1, t)
    ctx.synchronize()
    assert steps1.tolist() == [498] * batch and d1.sum().item() == 0
    s2, steps2 = s1.clone(), steps1.clone()          # the rows move: the counters move with them
    E.bind_step_counters(ctx, s2, steps2)
    for t in range(3, 6):
        E.step_kernel_gpu(ctx, s1, act(t), r1, d1, o1, t)
        E.step_kernel_gpu(ctx, s2, act(t), r2, d2, o2, t)
        ctx.synchronize()
        assert torch.equal(s1, s2) and torch.equal(d1, d2) and torch.equal(steps1, steps2)
        assert d1.sum().item() == (batch if t == 4 else 0)   # step 500 truncates every env
        E.selective_reset_kernel_gpu(ctx, s1, d1, 9)
        E.selective_reset_kernel_gpu(ctx, s2, d2, 9)
    with pytest.raises(mrl.MrlError):
        E.bind_step_counters(ctx, s1, torch.zeros(3, dtype=torch.int32, device="cuda"))     # one counter per env
    E.bind_step_counters(ctx, s1, None)
    E.bind_step_counters(ctx, s2, None)


def test_cartpole_truncation_counter(mrl, orc, ctx):
    # always push towards the centre: the pole survives past 500 steps only by truncation
    batch = 8
    E = mrl.CartPoleEnv
    s = torch.zeros(batch * 4, device="cuda")
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch, batch * 4))
    E.reset_kernel_gpu(ctx, s, 0)
    s_h = np.zeros((batch, 4), np.float32); st_h = np.zeros(batch, np.int32)
    orc.orc_cartpole_reset_batch(s_h, st_h, batch, 12345)
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 4), np.float32)
    saw_trunc = False
    for t in range(520):
        act = (s_h[:, 2] + 0.5 * s_h[:, 3] > 0).astype(np.float32)   # bang-bang on the angle
        a.copy_(dev(act))
        E.step_kernel_gpu(ctx, s, a, r, d, o)
        orc.orc_cartpole_step_batch(s_h, st_h, act, r_h, d_h, o_h, batch)
        ctx.synchronize()
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)
        saw_trunc |= bool(((d_h > 0.5) & (r_h > 0.5)).any())
        E.selective_reset_kernel_gpu(ctx, s, d, t)
        orc.orc_cartpole_selective_reset_batch(s_h, st_h, d_h, batch, t)
    assert saw_trunc


@pytest.mark.parametrize("batch", [1, 257, 16384])
def test_pendulum_rollout_parity(mrl, orc, ctx, batch):
    say("pendulum batch", batch)
    E = mrl.PendulumV2
    s_h = np.zeros((batch, 8), np.float32)
    orc.orc_pendulum_reset_batch(s_h, batch, 42)
    s = torch.zeros(batch * 8, device="cuda")
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch, batch * 3))
    E.reset_kernel_gpu(ctx, s, 42)
    ctx.synchronize()
    close(s.cpu().numpy().reshape(batch, 8), s_h)
    rng = np.random.default_rng(1)
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 3), np.float32)
    s_h[:, 4] = 150; s[4::8] = 150                        # so the 200-step truncation falls inside the test
    for t in range(64):
        act = rng.uniform(-1.3, 1.3, batch).astype(np.float32)
        a.copy_(dev(act))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_pendulum_step_batch(s_h, act, r_h, d_h, o_h, batch)
        ctx.synchronize()
        close(s.cpu().numpy().reshape(batch, 8), s_h)
        close(o.cpu().numpy().reshape(batch, 3), o_h)
        close(r.cpu().numpy(), r_h)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        s_h[:] = s.cpu().numpy().reshape(batch, 8)        # re-synchronise: per-step parity, not drift
        E.selective_reset_kernel_gpu(ctx, s, d, 7 + t)
        orc.orc_pendulum_selective_reset_batch(s_h, d_h, batch, 7 + t)
        ctx.synchronize()
        close(s.cpu().numpy().reshape(batch, 8), s_h)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        s_h[:] = s.cpu().numpy().reshape(batch, 8)


def ll_policy(rng, obs, t):
    """A seeded stand-in policy that fires engines often enough to exercise every action."""
    a = rng.integers(0, 4, obs.shape[0])
    a[obs[:, 3] < -0.3] = 2                                 # falling fast: main engine
    return a.astype(np.float32)


@pytest.mark.parametrize("batch,seed", [(1, 3), (65, 4), (8192, 5)])
def test_lunar_lander_rollout_parity(mrl, orc, ctx, batch, seed):
    say("lunar batch", batch)
    E = mrl.LunarLanderV2
    s_h = np.zeros((batch, 192), np.float32)
    orc.orc_ll_reset_batch(s_h, batch, seed)
    s = torch.full((batch * 192,), 7.0, device="cuda")     # garbage: reset must write every float
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch, batch * 8))
    E.reset_kernel_gpu(ctx, s, seed)
    ctx.synchronize()
    close(s.cpu().numpy().reshape(batch, 192), s_h)
    s_h[:] = s.cpu().numpy().reshape(batch, 192)
    rng = np.random.default_rng(seed)
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 8), np.float32)
    n_done = 0
    for t in range(64):
        act = ll_policy(rng, s_h[:, :8], t)
        a.copy_(dev(act))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_ll_step_batch(s_h, act, r_h, d_h, o_h, batch, 8)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 192)
        same_bits(sg, s_h, "state, step %d" % t)
        same_bits(o.cpu().numpy().reshape(batch, 8), o_h, "obs, step %d" % t)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)   # reward exact
        n_done += int(d_h.sum())
        s_h[:] = sg
    say("  finished rows seen:", n_done)


def test_lunar_lander_contacts_and_reset_cycle(mrl, orc, ctx):
    # start low over the pad so that contacts, crashes and landings all occur within 64 steps
    batch = 2048
    E = mrl.LunarLanderV2
    s_h = np.zeros((batch, 192), np.float32)
    orc.orc_ll_reset_batch(s_h, batch, 11)
    rng = np.random.default_rng(11)
    b = s_h[:, 8:47].reshape(batch, 3, 13)
    drop = rng.uniform(7.5, 9.4, batch).astype(np.float32)
    b[:, :, 1] -= drop[:, None]
    b[:, :, 0] += rng.uniform(-6, 6, batch).astype(np.float32)[:, None]
    b[:, 0, 2] = rng.uniform(-0.4, 0.4, batch).astype(np.float32)
    s = dev(s_h.reshape(-1))
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch, batch * 8))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 8), np.float32)
    crashes = lands = 0
    for t in range(64):
        act = rng.integers(0, 4, batch).astype(np.float32)
        a.copy_(dev(act))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_ll_step_batch(s_h, act, r_h, d_h, o_h, batch, 8)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 192)
        same_bits(sg, s_h, "state, step %d" % t)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)
        crashes += int((r_h == -100).sum()); lands += int((o_h[:, 6] + o_h[:, 7] > 0).sum())
        s_h[:] = sg
        E.selective_reset_kernel_gpu(ctx, s, d, 900 + t)
        orc.orc_ll_selective_reset_batch(s_h, d_h, batch, 900 + t)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 192)
        same_bits(sg, s_h, "state, step %d" % t)
        s_h[:] = sg
    say("  crashes", crashes, "leg-contact observations", lands)
    assert crashes > 50 and lands > 500


def llc_policy(rng, obs):
    """Continuous stand-in policy: throttle and side control beyond [-1, 1] now and then, the dead
    band of the side engines, and full throttle when falling fast."""
    n = obs.shape[0]
    a = rng.uniform(-1.4, 1.4, (n, 2)).astype(np.float32)
    a[rng.random(n) < 0.2, 1] = 0.5           # edge of the dead band
    a[obs[:, 3] < -0.3, 0] = 1.0
    return a


@pytest.mark.parametrize("batch,seed,low", [(1, 3, False), (65, 4, False), (8192, 5, False), (2048, 6, True)])
def test_lunar_lander_continuous_rollout_parity(mrl, orc, ctx, batch, seed, low):
    say("lunar continuous batch", batch, "low start", low)
    E = mrl.LunarLanderV2Continuous
    s_h = np.zeros((batch, 192), np.float32)
    orc.orc_ll_reset_batch(s_h, batch, seed)
    rng = np.random.default_rng(seed)
    if low:   # start low over the pad: contacts, crashes and landings within the 64 steps
        b = s_h[:, 8:47].reshape(batch, 3, 13)
        b[:, :, 1] -= rng.uniform(7.5, 9.4, batch).astype(np.float32)[:, None]
        b[:, :, 0] += rng.uniform(-6, 6, batch).astype(np.float32)[:, None]
    s = torch.full((batch * 192,), 7.0, device="cuda")
    E.reset_kernel_gpu(ctx, s, seed)
    ctx.synchronize()
    if low:
        s.copy_(dev(s_h.reshape(-1)))
    else:
        close(s.cpu().numpy().reshape(batch, 192), s_h)
        s_h[:] = s.cpu().numpy().reshape(batch, 192)
    a = torch.zeros(batch * 2, device="cuda")
    r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch * 8))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 8), np.float32)
    n_done = 0
    for t in range(64):
        act = llc_policy(rng, s_h[:, :8])
        a.copy_(dev(act.reshape(-1)))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_ll_step_continuous_batch(s_h, act, r_h, d_h, o_h, batch)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 192)
        same_bits(sg, s_h, "state, step %d" % t)
        same_bits(o.cpu().numpy().reshape(batch, 8), o_h, "obs, step %d" % t)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)   # reward exact
        n_done += int(d_h.sum())
        s_h[:] = sg
    say("  finished rows seen:", n_done)
    assert not low or n_done > 100


@pytest.mark.parametrize("cont", [False, True])
def test_lunar_lander_large_batch_form_parity(mrl, orc, ctx, cont):
    """Above 8192 rows the stand-alone step runs one lane per env on rows left in global memory (contact
    detection inline on the env's own lane) instead of a 32-row workgroup with the detection spread over
    seven wavefronts: same results, bit for bit, through steps, contacts, crashes and in-place resets.  The
    batch has a ragged last wavefront."""
    batch = 32768 + 5
    E = mrl.LunarLanderV2Continuous if cont else mrl.LunarLanderV2
    say("lunar large batch", batch, "continuous", cont)
    s_h = np.zeros((batch, 192), np.float32)
    orc.orc_ll_reset_batch(s_h, batch, 31)
    rng = np.random.default_rng(31)
    b = s_h[:, 8:47].reshape(batch, 3, 13)
    b[:, :, 1] -= rng.uniform(7.5, 9.4, batch).astype(np.float32)[:, None]
    b[:, :, 0] += rng.uniform(-6, 6, batch).astype(np.float32)[:, None]
    s = dev(s_h.reshape(-1))
    aw = 2 if cont else 1
    a = torch.zeros(batch * aw, device="cuda")
    r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch * 8))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 8), np.float32)
    n_done = 0
    for t in range(12):
        if cont:
            act = llc_policy(rng, s_h[:, :8])
        else:
            act = rng.integers(0, 4, batch).astype(np.float32)
        a.copy_(dev(act.reshape(-1)))
        if t % 2 == 0:      # both entry points take the large-batch form
            E.step_autoreset_kernel_gpu(ctx, s, a, r, d, o, t, 600 + t)
        else:
            E.step_kernel_gpu(ctx, s, a, r, d, o, t)
            E.selective_reset_kernel_gpu(ctx, s, d.clone(), 600 + t)
        if cont:
            orc.orc_ll_step_continuous_batch(s_h, act, r_h, d_h, o_h, batch)
        else:
            orc.orc_ll_step_batch(s_h, act, r_h, d_h, o_h, batch, 8)
        orc.orc_ll_selective_reset_batch(s_h, d_h, batch, 600 + t)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 192)
        same_bits(sg, s_h, "state, step %d" % t)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)
        if t % 2 == 0:      # the observation of the row as it stands after the reset
            same_bits(o.cpu().numpy().reshape(batch, 8), sg[:, :8], "obs, step %d" % t)
        n_done += int(d_h.sum())
        s_h[:] = sg
    say("  finished rows seen:", n_done)
    assert n_done > 1000


@pytest.mark.parametrize("cont", [False, True])
def test_lunar_lander_wind_parity(mrl, orc, cont):
    """ENABLE_WIND (lunar_lander_v2.mojo:123-127, :983-1023) as a setting of the context: 64 steps of both
    action forms against the oracle with the same setting, bit for bit; the rows start at different step
    counts (the gusts are a function of the step count), a quarter of them low enough to touch down,
    where the wind stops."""
    batch, seed = 2048, 12
    say("lunar wind, continuous", cont)
    own = mrl.DeviceContext("cuda:0")           # the setting belongs to the context: not the shared one
    E = mrl.LunarLanderV2Continuous if cont else mrl.LunarLanderV2
    s_h = np.zeros((batch, 192), np.float32)
    orc.orc_ll_reset_batch(s_h, batch, seed)
    rng = np.random.default_rng(seed)
    s_h[:, 188] = rng.integers(0, 900, batch)
    b = s_h[:, 8:47].reshape(batch, 3, 13)
    b[::4, :, 1] -= rng.uniform(7.5, 9.4, batch // 4).astype(np.float32)[:, None]
    s = dev(s_h.reshape(-1))
    aw = 2 if cont else 1
    a = torch.zeros(batch * aw, device="cuda")
    r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch * 8))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 8), np.float32)
    E.set_wind(own, True, 15.0, 1.5)
    orc.orc_ll_set_wind(1, 15.0, 1.5)
    legs = 0
    try:
        for t in range(64):
            if t == 40:       # other powers from here on
                E.set_wind(own, True, 7.0, 3.0)
                orc.orc_ll_set_wind(1, 7.0, 3.0)
            act = llc_policy(rng, s_h[:, :8]) if cont else ll_policy(rng, s_h[:, :8], t)
            a.copy_(dev(act.reshape(-1)))
            E.step_kernel_gpu(own, s, a, r, d, o, t)
            if cont:
                orc.orc_ll_step_continuous_batch(s_h, act, r_h, d_h, o_h, batch)
            else:
                orc.orc_ll_step_batch(s_h, act, r_h, d_h, o_h, batch, 8)
            own.synchronize()
            sg = s.cpu().numpy().reshape(batch, 192)
            same_bits(sg, s_h, "state, step %d" % t)
            np.testing.assert_array_equal(d.cpu().numpy(), d_h)
            np.testing.assert_array_equal(r.cpu().numpy(), r_h)
            legs += int((o_h[:, 6] + o_h[:, 7] > 0).sum())
            s_h[:] = sg
    finally:
        orc.orc_ll_set_wind(0, 15.0, 1.5)
    say("  leg-contact observations:", legs)
    assert legs > 100
    # switched off again, a step is the calm step
    E.set_wind(own, False)
    act = llc_policy(rng, s_h[:, :8]) if cont else ll_policy(rng, s_h[:, :8], 0)
    a.copy_(dev(act.reshape(-1)))
    E.step_kernel_gpu(own, s, a, r, d, o, 0)
    if cont:
        orc.orc_ll_step_continuous_batch(s_h, act, r_h, d_h, o_h, batch)
    else:
        orc.orc_ll_step_batch(s_h, act, r_h, d_h, o_h, batch, 8)
    own.synchronize()
    same_bits(s.cpu().numpy().reshape(batch, 192), s_h, "state, calm step")


def test_lunar_lander_continuous_corners_equal_discrete_actions(mrl, ctx):
    batch = 512
    D, Cn = mrl.LunarLanderV2, mrl.LunarLanderV2Continuous
    s1 = torch.zeros(batch * 192, device="cuda")
    D.reset_kernel_gpu(ctx, s1, 8)
    s2 = s1.clone()
    g = torch.Generator(device="cuda").manual_seed(3)
    table = torch.tensor([[-1.0, 0.0], [-1.0, -1.0], [1.0, 0.25], [-1.0, 1.0]], device="cuda")
    bufs = lambda: tuple(torch.zeros(n, device="cuda") for n in (batch, batch, batch * 8))
    r1, d1, o1 = bufs(); r2, d2, o2 = bufs()
    for t in range(30):
        a = torch.randint(0, 4, (batch,), device="cuda", generator=g)
        D.step_autoreset_kernel_gpu(ctx, s1, a.float(), r1, d1, o1, t, 70 + t)
        Cn.step_autoreset_kernel_gpu(ctx, s2, table[a].reshape(-1).contiguous(), r2, d2, o2, t, 70 + t)
        ctx.synchronize()
        assert torch.equal(s1, s2) and torch.equal(r1, r2) and torch.equal(d1, d2) and torch.equal(o1, o2)


def test_lunar_lander_autoreset_equals_step_then_selective_reset(mrl, ctx):
    batch = 1000
    E = mrl.LunarLanderV2
    s1 = torch.zeros(batch * 192, device="cuda")
    E.reset_kernel_gpu(ctx, s1, 21)
    s1.view(batch, 192)[:, 188] = torch.randint(990, 1000, (batch,), device="cuda").float()  # near the step limit
    s2 = s1.clone()
    bufs = lambda: tuple(torch.zeros(n, device="cuda") for n in (batch, batch, batch * 8))
    r1, d1, o1 = bufs(); r2, d2, o2 = bufs()
    a = torch.randint(0, 4, (batch,), device="cuda").float()
    ended = 0
    for t in range(12):
        E.step_kernel_gpu(ctx, s1, a, r1, d1, o1, t)
        E.selective_reset_kernel_gpu(ctx, s1, d1, 50 + t)
        E.step_autoreset_kernel_gpu(ctx, s2, a, r2, d2, o2, t, 50 + t)
        ctx.synchronize()
        assert torch.equal(s1, s2) and torch.equal(r1, r2) and torch.equal(d1, d2)
        assert torch.equal(o2.view(batch, 8), s2.view(batch, 192)[:, :8])
        ended += int(d1.sum().item())
    assert ended >= batch        # every row started within 10 steps of the limit


def test_env_argument_errors(mrl, ctx):
    s = torch.zeros(10, device="cuda")
    with pytest.raises(mrl.MrlError):
        mrl.LunarLanderV2.reset_kernel_gpu(ctx, s, 0)            # not a multiple of STATE_SIZE
    s = torch.zeros(192, device="cuda")
    with pytest.raises(mrl.MrlError):
        mrl.LunarLanderV2.step_kernel_gpu(ctx, s, torch.zeros(2, device="cuda"), torch.zeros(1, device="cuda"),
                                          torch.zeros(1, device="cuda"), torch.zeros(8, device="cuda"))
    with pytest.raises(mrl.MrlError):
        mrl.LunarLanderV2.reset_kernel_gpu(ctx, torch.zeros(192), 0)  # host tensor
    empty = torch.zeros(0, device="cuda")
    mrl.LunarLanderV2.reset_kernel_gpu(ctx, empty, 0)            # empty batch is a no-op


@pytest.mark.parametrize("batch,seed", [(1, 1), (33, 2), (4096, 3)])
def test_bipedal_walker_rollout_parity(mrl, orc, ctx, batch, seed):
    say("bipedal batch", batch)
    E = mrl.BipedalWalkerV2
    s_h = np.zeros((batch, 950), np.float32)
    orc.orc_bw_reset_batch(s_h, None, batch, seed)
    s = torch.full((batch * 950,), 7.0, device="cuda")
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch * 4, batch, batch, batch * 24))
    E.reset_kernel_gpu(ctx, s, seed)
    ctx.synchronize()
    close(s.cpu().numpy().reshape(batch, 950), s_h)
    s_h[:] = s.cpu().numpy().reshape(batch, 950)
    rng = np.random.default_rng(seed)
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 24), np.float32)
    n_done = contacts = 0
    for t in range(64):
        act = rng.uniform(-1.3, 1.3, (batch, 4)).astype(np.float32)
        a.copy_(dev(act.reshape(-1)))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_bw_step_batch(s_h, act, r_h, d_h, o_h, batch, 8)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 950)
        same_bits(sg, s_h, "state, step %d" % t)
        same_bits(o.cpu().numpy().reshape(batch, 24), o_h, "obs, step %d" % t)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)   # reward exact
        term = d_h > 0.5
        n_done += int(term.sum()); contacts += int((o_h[:, 8] + o_h[:, 13] > 0).sum())
        s_h[:] = sg
        E.selective_reset_kernel_gpu(ctx, s, d, 300 + t)
        orc.orc_bw_reset_batch(s_h, d_h.ctypes.data, batch, 300 + t)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 950)
        same_bits(sg, s_h, "state after reset, step %d" % t)
        s_h[:] = sg
    say("  finished rows", n_done, "leg-contact observations", contacts)
    if batch > 1000:
        assert n_done > 100 and contacts > 1000


@pytest.mark.parametrize("batch,seed", [(1, 1), (65, 2), (4096, 3)])
def test_half_cheetah_rollout_parity(mrl, orc, ctx, batch, seed):
    say("cheetah batch", batch)
    E = mrl.HalfCheetahPlanarV2
    s_h = np.zeros((batch, 253), np.float32)
    orc.orc_hc_reset_batch(s_h, None, batch, seed)
    s = torch.full((batch * 253,), 7.0, device="cuda")
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch * 6, batch, batch, batch * 17))
    E.reset_kernel_gpu(ctx, s, seed)
    ctx.synchronize()
    close(s.cpu().numpy().reshape(batch, 253), s_h)
    s_h[:] = s.cpu().numpy().reshape(batch, 253)
    s_h[:, 245] = 960; s.view(batch, 253)[:, 245] = 960        # so the 1000-step limit falls inside the test
    rng = np.random.default_rng(seed)
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 17), np.float32)
    pen = n_done = 0
    for t in range(64):
        act = rng.uniform(-1.4, 1.4, (batch, 6)).astype(np.float32)
        a.copy_(dev(act.reshape(-1)))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_hc_step_batch(s_h, act, r_h, d_h, o_h, batch, 8)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 253)
        same_bits(sg, s_h, "state, step %d" % t)
        same_bits(o.cpu().numpy().reshape(batch, 17), o_h, "obs, step %d" % t)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)   # reward exact
        pen += int((s_h[:, 17 + 1] < 0.2).sum())             # torso lower than standing height: on the ground
        n_done += int(d_h.sum())
        s_h[:] = sg
        E.selective_reset_kernel_gpu(ctx, s, d, 300 + t)
        orc.orc_hc_reset_batch(s_h, d_h.ctypes.data, batch, 300 + t)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 253)
        same_bits(sg, s_h, "state after reset, step %d" % t)
        s_h[:] = sg
    say("  rows at the step limit", n_done, "torso-low observations", pen)
    assert n_done == batch and pen > batch      # every row hits the 1000-step limit once; bodies reach the ground


def test_half_cheetah_rows_with_other_wiring_take_the_one_lane_form(mrl, orc, ctx):
    """The body-per-lane step assumes HalfCheetah's own joint table; a row that differs (here: the
    front foot's joint removed in every other env, so that foot comes off) is stepped by the generic
    one-lane form.  Both kinds of rows sit side by side in one wavefront and must match the oracle."""
    batch = 100
    E = mrl.HalfCheetahPlanarV2
    s_h = np.zeros((batch, 253), np.float32)
    orc.orc_hc_reset_batch(s_h, None, batch, 9)
    s_h[::2, 17 + 91 + 21 + 102] = 5.0          # joint count
    s = dev(s_h.reshape(-1))
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch * 6, batch, batch, batch * 17))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 17), np.float32)
    rng = np.random.default_rng(9)
    for t in range(40):
        act = rng.uniform(-1.2, 1.2, (batch, 6)).astype(np.float32)
        a.copy_(dev(act.reshape(-1)))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_hc_step_batch(s_h, act, r_h, d_h, o_h, batch, 4)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 253)
        same_bits(sg, s_h, "state, step %d" % t)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)
        s_h[:] = sg
    # the loose foot has fallen away from its shin in the rows without the joint
    foot, shin = s_h[:, 17 + 13 * 6: 17 + 13 * 6 + 3], s_h[:, 17 + 13 * 5: 17 + 13 * 5 + 3]
    rot = lambda body, ly: np.stack([body[:, 0] - ly * np.sin(body[:, 2]), body[:, 1] + ly * np.cos(body[:, 2])], 1)
    gap = np.hypot(*(rot(shin, -0.106 / 2) - rot(foot, 0.07 / 2)).T)      # distance between the two anchors
    assert np.median(gap[::2]) > 0.09 and gap[1::2].max() < 0.08


def test_bipedal_walker_rows_with_other_wiring_take_the_one_lane_form(mrl, orc, ctx):
    """The walker's solver runs with one lane per body for rows that have the walker's own four joints; a
    row with another joint table (here: the last joint missing, so that lower leg 2 hangs loose) is stepped
    by the one-lane form.  Both kinds of rows sit side by side in one workgroup and must match the oracle."""
    batch = 100
    E = mrl.BipedalWalkerV2
    s_h = np.zeros((batch, 950), np.float32)
    orc.orc_bw_reset_batch(s_h, None, batch, 9)
    JOINT_COUNT = 24 + 65 + 15 + 68
    assert (s_h[:, JOINT_COUNT] == 4.0).all()
    s_h[::2, JOINT_COUNT] = 3.0
    s = dev(s_h.reshape(-1))
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch * 4, batch, batch, batch * 24))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 24), np.float32)
    rng = np.random.default_rng(9)
    for t in range(40):
        act = rng.uniform(-1.2, 1.2, (batch, 4)).astype(np.float32)
        a.copy_(dev(act.reshape(-1)))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_bw_step_batch(s_h, act, r_h, d_h, o_h, batch, 4)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 950)
        same_bits(sg, s_h, "state, step %d" % t)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        s_h[:] = sg
        if t == 20:
            # the loose lower leg has come away from its upper leg in the rows without the joint
            up, low = s_h[:, 24 + 13 * 3: 24 + 13 * 3 + 3], s_h[:, 24 + 13 * 4: 24 + 13 * 4 + 3]
            J = s_h[:, 24 + 65 + 15 + 3 * 17: 24 + 65 + 15 + 4 * 17]       # [type, a, b, ax, ay, bx, by, ...]
            world = lambda body, lx, ly: np.stack([body[:, 0] + lx * np.cos(body[:, 2]) - ly * np.sin(body[:, 2]),
                                                   body[:, 1] + lx * np.sin(body[:, 2]) + ly * np.cos(body[:, 2])], 1)
            gap = np.hypot(*(world(up, J[:, 3], J[:, 4]) - world(low, J[:, 5], J[:, 6])).T)   # between the two anchors
            say("  anchor gap of joint 3, medians: without the joint %.3f, with it %.3f" % (np.median(gap[::2]), np.median(gap[1::2])))
            assert np.median(gap[::2]) > 0.3 and np.median(gap[1::2]) < 0.05


def test_bipedal_walker_bodies_strewn_over_the_terrain(mrl, orc, ctx):
    """Contact detection picks, once per env, the terrain edges near any of its bodies and each (body, vertex)
    pair then looks only at those: rows whose bodies lie metres apart (with the joints, which then pull them
    together violently, and without), rows with a NaN or infinite body position and ordinary rows side by
    side must all match the oracle bit for bit, contacts of the far bodies included."""
    def same(a, b, what):
        # bit for bit, except that a NaN matches any NaN (host and GPU differ in the sign of a generated NaN)
        a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
        bad = (a.view(np.uint32) != b.view(np.uint32)) & ~(np.isnan(a) & np.isnan(b))
        assert not bad.any(), "%s: %d of %d floats differ, first at %s: %r vs %r" % (
            what, int(bad.sum()), bad.size, np.argwhere(bad)[0], a[bad][0], b[bad][0])

    batch = 96
    E = mrl.BipedalWalkerV2
    s_h = np.zeros((batch, 950), np.float32)
    orc.orc_bw_reset_batch(s_h, None, batch, 21)
    BODIES, JOINT_COUNT = 24, 24 + 65 + 15 + 68
    rng = np.random.default_rng(21)
    for i in range(batch):
        kind = i % 4
        if kind == 3:
            continue
        for b in range(5):
            s_h[i, BODIES + 13 * b] += np.float32((b - 1) * rng.uniform(3.0, 9.0))     # x: up to 27 m to the right, one 9 m to the left
            s_h[i, BODIES + 13 * b + 1] -= np.float32(rng.uniform(0.0, 0.6))              # y: towards / into the ground
            s_h[i, BODIES + 13 * b + 2] = np.float32(rng.uniform(-3.0, 3.0))              # angle
        if kind == 1:
            s_h[i, JOINT_COUNT] = 0.0
        if kind == 2 and i % 8 == 2:
            s_h[i, BODIES + 13 * (i % 5)] = np.float32(np.nan if i % 16 == 2 else np.inf)
    s = dev(s_h.reshape(-1))
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch * 4, batch, batch, batch * 24))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 24), np.float32)
    touched = 0
    for t in range(12):
        act = rng.uniform(-1.2, 1.2, (batch, 4)).astype(np.float32)
        a.copy_(dev(act.reshape(-1)))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_bw_step_batch(s_h, act, r_h, d_h, o_h, batch, 4)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 950)
        same(sg, s_h, "state, step %d" % t)
        same(r.cpu().numpy(), r_h, "reward, step %d" % t)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        same(o.cpu().numpy().reshape(batch, 24), o_h, "observation, step %d" % t)
        s_h[:] = sg
        if t == 0:
            # the far legs did touch the ground: their contact flags in the observation
            touched = int((o_h[:, 8] > 0.5).sum() + (o_h[:, 13] > 0.5).sum())
    say("  leg contact flags set after the first step: %d" % touched)
    assert touched > 10


@pytest.mark.parametrize("name", ["CartPoleEnv", "PendulumV2", "BipedalWalkerV2", "HalfCheetahPlanarV2",
                                  "LunarLanderV2Continuous"])
def test_autoreset_equals_step_then_selective_reset(mrl, ctx, name):
    E = getattr(mrl, name)
    batch = 777
    aw = E.ACTION_DIM if E.ACTION_DIM else 1
    s1 = torch.zeros(batch * E.STATE_SIZE, device="cuda")
    E.reset_kernel_gpu(ctx, s1, 5)
    s2 = s1.clone()
    # each env type gets its own pair of state buffers (CartPole's step counters are keyed by buffer)
    E.reset_kernel_gpu(ctx, s2, 5)
    bufs = lambda: tuple(torch.zeros(n, device="cuda") for n in (batch, batch, batch * E.OBS_DIM))
    r1, d1, o1 = bufs(); r2, d2, o2 = bufs()
    g = torch.Generator(device="cuda").manual_seed(1)
    ended = 0
    for t in range(40):
        if E.NUM_ACTIONS:
            a = torch.randint(0, E.NUM_ACTIONS, (batch,), device="cuda", generator=g).float()
        else:
            a = (torch.rand(batch * aw, device="cuda", generator=g) * 2 - 1) * 1.2
        if name == "PendulumV2" and t == 0:
            s1.view(batch, 8)[:, 4] = 170; s2.view(batch, 8)[:, 4] = 170
        if name == "LunarLanderV2Continuous" and t == 0:
            s1.view(batch, 192)[:, 188] = 970; s2.view(batch, 192)[:, 188] = 970
        E.step_kernel_gpu(ctx, s1, a, r1, d1, o1, t)
        dstep = d1.clone()
        E.selective_reset_kernel_gpu(ctx, s1, d1, 50 + t)
        E.step_autoreset_kernel_gpu(ctx, s2, a, r2, d2, o2, t, 50 + t)
        ctx.synchronize()
        assert torch.equal(s1, s2) and torch.equal(r1, r2) and torch.equal(dstep, d2)
        assert torch.equal(o2.view(batch, E.OBS_DIM), s2.view(batch, E.STATE_SIZE)[:, :E.OBS_DIM])
        ended += int(d2.sum().item())
    assert ended > 0 or name == "HalfCheetahPlanarV2"


def _crowd_edges(rows, edges_off, first, count, x_center, y):
    """Rewrites `count` consecutive terrain edges of every row into a staircase of tiny flat edges
    around x_center at height y: a vertex above them passes the x-range pre-check of all of them."""
    for k in range(count):
        e = rows[:, edges_off + 6 * (first + k): edges_off + 6 * (first + k + 1)]
        x0 = x_center - 0.02 + 0.01 * k
        e[:, 0], e[:, 1], e[:, 2], e[:, 3], e[:, 4], e[:, 5] = x0, y, x0 + 0.01, y, 0.0, 1.0


def test_walker_vertex_over_many_edges_takes_the_serial_detector(mrl, orc, ctx):
    """A vertex that touches four or more edges overflows its per-task contact list; the env then
    falls back to the one-lane detector inside the step.  Terrain with a cluster of tiny edges under
    the feet forces that path (and the MAX_CONTACTS cut-off of the merged list)."""
    batch = 96
    E = mrl.BipedalWalkerV2
    s_h = np.zeros((batch, 950), np.float32)
    orc.orc_bw_reset_batch(s_h, None, batch, 4)
    hull_x = float(s_h[0, 24])
    foot_y = float(s_h[:, 24 + 13 * 4 + 1].min()) - 34.0 / 30.0 / 2
    assert abs(hull_x - 20 * 14.0 / 30.0) < 1e-3
    # edges start after obs 24, bodies 5*13, forces 5*3, joints 4*17, joint count 1
    edges_off = 24 + 65 + 15 + 68 + 1
    assert abs(s_h[0, edges_off + 6 * 19 + 2] - hull_x) < 1e-3      # edge 19 ends under the hull
    _crowd_edges(s_h[::2], edges_off, 17, 6, hull_x, foot_y + 0.05)   # every other env
    s = dev(s_h.reshape(-1))
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch * 4, batch, batch, batch * 24))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 24), np.float32)
    rng = np.random.default_rng(4)
    touched = 0
    for t in range(12):
        act = rng.uniform(-1.0, 1.0, (batch, 4)).astype(np.float32)
        a.copy_(dev(act.reshape(-1)))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_bw_step_batch(s_h, act, r_h, d_h, o_h, batch, 8)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 950)
        same_bits(sg, s_h, "state, step %d" % t)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)
        touched += int((o_h[::2, 8] + o_h[::2, 13] > 0).sum())
        s_h[:] = sg
    say("  leg-contact observations on the crowded terrain:", touched)
    assert touched > 100


def test_lander_vertex_over_many_edges_takes_the_serial_detector(mrl, orc, ctx):
    batch = 64
    E = mrl.LunarLanderV2
    s_h = np.zeros((batch, 192), np.float32)
    orc.orc_ll_reset_batch(s_h, batch, 6)
    b = s_h[:, 8:47].reshape(batch, 3, 13)
    edges_off = 91
    pad_y = float(s_h[0, edges_off + 6 * 5 + 1])           # the helipad edges are flat
    b[:, :, 1] -= (b[:, 0, 1] - pad_y - 0.9)[:, None]       # hull 0.9 above the pad: legs reach it in a few steps
    b[:, :, 0] += (10.0 - b[:, 0, 0])[:, None]
    leg_x = float(b[0, 1, 0])
    _crowd_edges(s_h[::2], edges_off, 4, 6, leg_x, pad_y)
    s = dev(s_h.reshape(-1))
    a, r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch, batch * 8))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, 8), np.float32)
    legs = 0
    for t in range(30):
        act = np.zeros(batch, np.float32)
        a.copy_(dev(act))
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_ll_step_batch(s_h, act, r_h, d_h, o_h, batch, 8)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, 192)
        same_bits(sg, s_h, "state, step %d" % t)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)
        legs += int((o_h[::2, 6] + o_h[::2, 7] > 0).sum())
        s_h[:] = sg
    say("  leg contacts on the crowded pad:", legs)
    assert legs > 20


def test_step_result_is_the_step_in_fresh_buffers(mrl, ctx):
    """VecStepResult (core/vec_env.mojo:25) from step_result equals what step_kernel_gpu writes."""
    E, batch = mrl.PendulumV2, 33
    s1 = torch.zeros(batch * E.STATE_SIZE, device="cuda")
    E.reset_kernel_gpu(ctx, s1, 4)
    s2 = s1.clone()
    act = torch.linspace(-2, 2, batch, device="cuda")
    r, d_, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch * E.OBS_DIM))
    E.step_kernel_gpu(ctx, s1, act, r, d_, o, 1)
    res = E.step_result(ctx, s2, act, 1)
    ctx.synchronize()
    assert isinstance(res, mrl.VecStepResult) and res.observations.shape == (batch, E.OBS_DIM)
    assert torch.equal(res.observations.reshape(-1), o) and torch.equal(res.rewards, r) and torch.equal(res.dones, d_)
    assert torch.equal(s1, s2)
