"""GPU parity: CarRacingV2 (reset with its track generator, step, selective reset, auto-reset) through
the C ABI against the oracle, bit for bit."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
S, OBS = 3040, 13


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def ctx(mrl):
    return mrl.DeviceContext("cuda:0")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def same_bits(a, b, what):
    a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
    bad = a.view(np.uint32) != b.view(np.uint32)
    assert not bad.any(), "%s: %d of %d floats differ, first at %s: %r vs %r" % (
        what, int(bad.sum()), bad.size, np.argwhere(bad)[0], a[bad][0], b[bad][0])


def driver(rng, s_h, t):
    """Actions that keep most cars on the road for a while (gentle steering towards the tile ahead, gas
    while slow), with out-of-range components now and then."""
    n = s_h.shape[0]
    a = np.zeros((n, 3), np.float32)
    a[:, 0] = rng.uniform(-0.3, 0.3, n)
    a[:, 1] = np.where(s_h[:, 12] < 10.0, rng.uniform(-0.2, 1.4, n), -1.0)
    a[:, 2] = np.where(rng.random(n) < 0.05, rng.uniform(-1.5, 1.5, n), -1.0)
    a[rng.random(n) < 0.02, 0] = 2.5
    return a


@pytest.mark.parametrize("batch,seed,form", [(1, 1, 0), (37, 2, 0), (2048, 3, 0), (37, 4, 1), (2048, 5, 1)])
def test_car_racing_reset_and_rollout_parity(mrl, orc, batch, seed, form):
    """form 0: the CPU env's step (the default); form 1: the GPU trait's step_kernel_gpu
    (car_racing_v2.mojo:1556-1716: reward 0.5 * forward speed - 0.01 + tile reward in fp32), selected per
    context with CarRacingV2.set_step_form and in the oracle with orc_cr_set_step_form."""
    say("car racing batch", batch, "step form", form)
    E = mrl.CarRacingV2
    ctx = mrl.DeviceContext("cuda:0")          # a context of its own: the setting belongs to the context
    E.set_step_form(ctx, form)
    orc.orc_cr_set_step_form(form)
    try:
        _rollout_parity(mrl, orc, ctx, E, batch, seed, form)
    finally:
        orc.orc_cr_set_step_form(0)
        ctx.close()


def _rollout_parity(mrl, orc, ctx, E, batch, seed, form):
    s_h = np.zeros((batch, S), np.float32)
    orc.orc_cr_reset_batch(s_h, None, batch, seed)
    s = torch.full((batch * S,), 7.0, device="cuda")          # garbage: the reset must write every float
    E.reset_kernel_gpu(ctx, s, seed)
    ctx.synchronize()
    same_bits(s.cpu().numpy().reshape(batch, S), s_h, "reset")
    a = torch.zeros(batch * 3, device="cuda")
    r, d, o = (torch.zeros(n, device="cuda") for n in (batch, batch, batch * OBS))
    r_h, d_h, o_h = np.zeros(batch, np.float32), np.zeros(batch, np.float32), np.zeros((batch, OBS), np.float32)
    if batch > 100:                       # some rows close to the step limit, some about to leave the playfield
        s_h[::7, 34] = 470; s_h[::11, 13] = 331.0; s_h[::11, 16] = 40.0
        s.copy_(dev(s_h.reshape(-1)))
    rng = np.random.default_rng(seed)
    n_done = new_tiles = 0
    for t in range(64):
        act = driver(rng, s_h, t)
        a.copy_(dev(act.reshape(-1)))
        before = s_h[:, 38].copy()
        E.step_kernel_gpu(ctx, s, a, r, d, o, t)
        orc.orc_cr_step_batch(s_h, act, r_h, d_h, o_h, batch, 8)
        ctx.synchronize()
        sg = s.cpu().numpy().reshape(batch, S)
        same_bits(sg, s_h, "state, step %d" % t)
        same_bits(o.cpu().numpy().reshape(batch, OBS), o_h, "obs, step %d" % t)
        np.testing.assert_array_equal(d.cpu().numpy(), d_h)
        np.testing.assert_array_equal(r.cpu().numpy(), r_h)
        n_done += int(d_h.sum()); new_tiles += int((s_h[:, 38] - before).sum())
        dn = d_h.copy()
        E.selective_reset_kernel_gpu(ctx, s, d, 500 + t)
        orc.orc_cr_reset_batch(s_h, dn.ctypes.data, batch, 500 + t)
        ctx.synchronize()
        same_bits(s.cpu().numpy().reshape(batch, S), s_h, "state after reset, step %d" % t)
        assert d.sum().item() == 0        # the selective reset clears the flags it has served
    say("  finished rows", n_done, "tiles newly visited", new_tiles)
    if batch > 100:
        assert n_done > batch // 8 and new_tiles > batch
    if form == 1:
        with pytest.raises(mrl.MrlError, match="neither"):
            E.set_step_form(ctx, 2)


def test_car_racing_done_rows_stay_untouched(mrl, orc, ctx):
    batch = 64
    E = mrl.CarRacingV2
    s = torch.zeros(batch * S, device="cuda")
    E.reset_kernel_gpu(ctx, s, 9)
    s.view(batch, S)[::2, 36] = 1.0        # done flag
    before = s.clone()
    a = torch.ones(batch * 3, device="cuda")
    r, d, o = (torch.full((n,), 5.0, device="cuda") for n in (batch, batch, batch * OBS))
    E.step_kernel_gpu(ctx, s, a, r, d, o, 0)
    ctx.synchronize()
    assert torch.equal(s.view(batch, S)[::2], before.view(batch, S)[::2])
    assert (r[::2] == 0).all() and (d[::2] == 1).all() and (d[1::2] == 0).all()
    assert not torch.equal(s.view(batch, S)[1::2], before.view(batch, S)[1::2])


def test_car_racing_autoreset_equals_step_then_selective_reset(mrl, ctx):
    batch = 300
    E = mrl.CarRacingV2
    s1 = torch.zeros(batch * S, device="cuda")
    E.reset_kernel_gpu(ctx, s1, 5)
    s1.view(batch, S)[:, 34] = torch.randint(490, 500, (batch,), device="cuda").float()    # near the step limit
    s2 = s1.clone()
    bufs = lambda: tuple(torch.zeros(n, device="cuda") for n in (batch, batch, batch * OBS))
    r1, d1, o1 = bufs(); r2, d2, o2 = bufs()
    g = torch.Generator(device="cuda").manual_seed(1)
    ended = 0
    for t in range(14):
        a = torch.rand(batch * 3, device="cuda", generator=g) * 2 - 1
        E.step_kernel_gpu(ctx, s1, a, r1, d1, o1, t)
        ended += int(d1.sum().item())
        E.selective_reset_kernel_gpu(ctx, s1, d1.clone(), 50 + t)
        E.step_autoreset_kernel_gpu(ctx, s2, a, r2, d2, o2, t, 50 + t)
        ctx.synchronize()
        assert torch.equal(s1, s2) and torch.equal(r1, r2) and torch.equal(d1, d2)
        assert torch.equal(o2.view(batch, OBS), s2.view(batch, S)[:, :OBS])
    assert ended >= batch


def test_continuous_agent_runs_on_car_racing(mrl, ctx):
    agent = mrl.DeepPPOContinuousAgent(obs_dim=13, action_dim=3, hidden_dim=64, rollout_len=32, n_envs=256,
                                       gpu_minibatch_size=1024, num_epochs=2, target_kl=0.0, init_seed=5)
    m = agent.train_gpu(ctx, mrl.CarRacingV2, num_episodes=10**9, max_rollouts=2, seed=3)
    assert m.rollouts == 2 and m.total_steps == 2 * 32 * 256
    assert torch.isfinite(agent.actor.params).all() and torch.isfinite(agent.rb.states).all()
    assert torch.isfinite(agent.rb.r_rewards).all() and agent.rb.states.view(256, S)[:, 34].max().item() >= 1
