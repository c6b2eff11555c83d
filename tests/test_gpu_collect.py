"""mrl_rollout_steps (many collection steps per launch) against the same steps issued one by one."""
import importlib
import sys

import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def mrl():
    return importlib.import_module("mojo-rl_amd")


@pytest.fixture(scope="module")
def ctx(mrl):
    return mrl.DeviceContext("cuda:0")


def _pair(mrl, ctx, N, T, hidden, kind, env="lunar"):
    E = {"lunar": mrl.LunarLanderV2, "lunarc": mrl.LunarLanderV2Continuous, "cartpole": mrl.CartPoleEnv,
         "pendulum": mrl.PendulumV2, "bipedal": mrl.BipedalWalkerV2, "cheetah": mrl.HalfCheetahPlanarV2,
         "car": mrl.CarRacingV2, "hopper": mrl.HopperPlanar, "walker2d": mrl.Walker2dPlanar}[env]
    lin = mrl.LinearReLU if kind == "relu" else mrl.LinearTanh
    head = mrl.StochasticActor(hidden, E.ACTION_DIM) if E.ACTION_DIM else mrl.Linear(hidden, E.NUM_ACTIONS)
    actor = mrl.seq(lin(E.OBS_DIM, hidden), lin(hidden, hidden), head)
    critic = mrl.seq(lin(E.OBS_DIM, hidden), lin(hidden, hidden), mrl.Linear(hidden, 1))
    g = torch.Generator(device="cuda").manual_seed(5)
    ap = (torch.rand(actor.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    cp = (torch.rand(critic.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    out = []
    for _ in range(2):
        rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
        rb.actor_params, rb.critic_params = ap, cp
        E.reset_kernel_gpu(ctx, rb.states, 3)
        # some episodes end inside the range, so that in-place resets and the accounting are covered
        rows = rb.states.view(N, E.STATE_SIZE)
        if env in ("lunar", "lunarc"):
            rows[::3, 188] = 995.0    # step counter close to the limit
        elif env == "cartpole":
            rows[::3, 0] = 2.39       # cart next to the edge of the track, moving outwards
            rows[::3, 1] = 2.0
        elif env == "bipedal":
            rows[::3, 942] = 1995.0   # step counter (first metadata float) close to its limit of 2000
        elif env == "car":
            rows[::3, 34] = 495.0     # step counter (first metadata float) close to its limit of 500
        elif env == "cheetah":
            rows[::3, 245] = 995.0    # step counter (first metadata float) close to its limit of 1000
        elif env in ("hopper", "walker2d"):
            # no step limit in these envs: every third torso starts tilted beyond the health bound (first step
            # ends the episode), the next third high up with the legs folded, so that it falls through the
            # height bound some steps later.  The Float64 state begins behind the observation and a padding float.
            d = rb.states.view(torch.float64).view(N, E.STATE_SIZE // 2)[:, (E.OBS_DIM + 1) // 2:]
            nj = E.ACTION_DIM
            d[::3, 2] = 1.5
            d[1::3, 1] = 1.3
            d[1::3, 15 + 3 * (nj - 3):15 + 3 * (nj - 3) + nj] = -1.0    # joint angles
            rows[::3, 1] = 1.5
        else:
            rows[::3, 4] = 197.0      # step counter close to the limit
        rb.obs.copy_(rows[:, :E.OBS_DIM].reshape(-1))
        out.append(rb)
    return out


@pytest.mark.parametrize("env,N,T,hidden,kind", [
    ("lunar", 8192, 12, 256, "relu"), ("lunar", 1000, 9, 256, "tanh"), ("lunar", 77, 5, 256, "relu"),
    ("lunar", 300, 6, 64, "relu"),            # not fusable: the loop of single steps behind the same call
    # above 8192 envs the single steps run the one-lane-per-env step kernel (rows in global memory,
    # detection inline, accounting and reset by the env's lane) against the fused kernel's 32-row workgroups
    ("lunar", 9001, 8, 256, "relu"), ("lunarc", 9001, 6, 256, "tanh"),
    ("cartpole", 8192, 12, 64, "relu"), ("cartpole", 77, 7, 64, "tanh"),
    ("pendulum", 8192, 12, 64, "tanh"), ("pendulum", 1000, 9, 64, "relu"),
    ("cartpole", 300, 6, 256, "relu"),        # not fusable
    ("lunarc", 8192, 12, 256, "tanh"), ("lunarc", 77, 6, 256, "relu"), ("lunarc", 300, 6, 64, "tanh"),
    # the walkers: legs on the ground from the first step (contacts, joint limits, lidar), falls and
    # step-limit endings with in-place resets inside the launch
    ("bipedal", 4096, 12, 256, "tanh"), ("bipedal", 77, 7, 256, "relu"), ("bipedal", 500, 64, 256, "tanh"),
    ("cheetah", 4096, 12, 256, "tanh"), ("cheetah", 77, 7, 256, "relu"), ("cheetah", 500, 64, 256, "tanh"),
    ("cheetah", 300, 5, 64, "tanh"),          # not fusable
    # CarRacing: tiles are visited from the first step on (the flags an env wrote are read back by later
    # steps of the same launch), truncations rebuild the track inside the launch
    ("car", 4096, 12, 256, "tanh"), ("car", 77, 7, 256, "relu"), ("car", 300, 48, 256, "tanh"),
    ("car", 100, 5, 64, "tanh"),              # not fusable
    # the Float64 planar envs: unhealthy torsos end episodes from the first step on, resets inside the launch
    ("hopper", 4096, 12, 256, "tanh"), ("hopper", 77, 7, 256, "relu"), ("hopper", 500, 64, 256, "tanh"),
    ("walker2d", 4096, 12, 256, "tanh"), ("walker2d", 77, 7, 256, "relu"), ("walker2d", 500, 64, 256, "tanh"),
    ("hopper", 100, 5, 64, "tanh"),           # not fusable
])
def test_rollout_steps_equals_single_steps(mrl, ctx, env, N, T, hidden, kind):
    print("case", env, N, T, hidden, kind, flush=True)
    one, many = _pair(mrl, ctx, N, T, hidden, kind, env)
    s0, ss, r0, rs = 1234567, 2654435761 * N + 7919, 99, 0x9E3779B97F4A7C15
    d1, d2 = one.descriptor(), many.descriptor()
    for t in range(T):
        mrl.ppo.rollout_step(ctx, d1, t, s0 + t * ss, 0, r0 + t * rs)
    # two launches: the second continues from the state the first left in HBM
    k = T // 2
    mrl.ppo.rollout_steps(ctx, d2, 0, k, s0, ss, 0, 0, r0, rs)
    mrl.ppo.rollout_steps(ctx, d2, k, T - k, s0 + k * ss, ss, 0, 0, r0 + k * rs, rs)
    ctx.synchronize()
    for name in ("r_obs", "r_actions", "r_log_probs", "r_values", "r_rewards", "r_dones", "states", "obs",
                 "ep_return", "ep_length"):
        a, b = getattr(one, name), getattr(many, name)
        if name == "states":     # as bit patterns: the halves of the planar envs' doubles include NaN patterns
            a, b = a.view(torch.int32), b.view(torch.int32)
        assert torch.equal(a, b), "%s differs in %d places" % (name, int((a != b).sum()))
    cnt = int(one.done_count.item())
    assert cnt == int(many.done_count.item()) and cnt > 0
    key = lambda rb: sorted(zip(rb.done_returns[:cnt].tolist(), rb.done_lengths[:cnt].tolist()))
    assert key(one) == key(many)


def _low_start(E, N, seed, orc):
    """Rows reset by the oracle, then lowered to just above the terrain with a sideways offset and a
    tilt, so that leg contacts, lander-body crashes, landings and in-place resets all happen within
    a few dozen steps (envs/lunar_lander/lunar_lander_v2.mojo:1097-1255)."""
    import numpy as np
    s_h = np.zeros((N, E.STATE_SIZE), np.float32)
    orc.orc_ll_reset_batch(s_h, N, seed)
    rng = np.random.default_rng(seed)
    b = s_h[:, 8:47].reshape(N, 3, 13)
    b[:, :, 1] -= rng.uniform(7.5, 9.4, N).astype(np.float32)[:, None]
    b[:, :, 0] += rng.uniform(-6, 6, N).astype(np.float32)[:, None]
    b[:, 0, 2] = rng.uniform(-0.4, 0.4, N).astype(np.float32)
    # Every fourth row hovers over the helipad instead: legs folded to their joint limit with the feet
    # 3 mm above the pad -- inside the 1 cm band of the leg-contact observation, no solver contact --
    # and every body moving up at g * dt, which the step's gravity cancels.  A step without engine
    # power leaves such a row at rest on both legs: the +100 landing branch (:1230-1247).
    pad, th = np.float32(400 / 30 / 4), np.float32(0.399)
    leg_y = pad + np.float32(0.2745)
    hov = b[::4]
    hov[:, 0, :3] = (10.0, leg_y + np.float32(10 / 30) + np.cos(th) * np.float32(8 / 30), 0.0)
    for k, sgn in ((1, -1.0), (2, 1.0)):
        hov[:, k, 0] = np.float32(10 + sgn * 20 / 30) + np.float32(sgn) * np.sin(th) * np.float32(8 / 30)
        hov[:, k, 1], hov[:, k, 2] = leg_y, np.float32(-sgn) * th
    hov[:, :, 3:6] = (0.0, 0.2, 0.0)
    return s_h


# up to 4096 envs (16 per CU) run the 16-row kernel, more the 32-row kernel
@pytest.mark.parametrize("env,kind,N", [("lunar", "relu", 2048), ("lunarc", "tanh", 2048), ("lunar", "tanh", 77),
                                        ("lunar", "relu", 4128), ("lunarc", "relu", 4128)])
def test_fused_collection_through_contacts(mrl, ctx, orc, env, kind, N):
    """The fused collection kernel with the envs on the ground: contact detection on the other
    wavefronts, list merge, solver with contacts, crash / landing terminations and resets inside the
    launch.  (1) one-step launches against the oracle fed the kernel's own actions; (2) a 64-step range
    in two launches against the same steps issued one by one, bit for bit."""
    import numpy as np
    print("case contacts", env, kind, N, flush=True)
    T = 64
    E = mrl.LunarLanderV2 if env == "lunar" else mrl.LunarLanderV2Continuous
    cont = env == "lunarc"
    lin = mrl.LinearReLU if kind == "relu" else mrl.LinearTanh
    head = mrl.StochasticActor(256, 2) if cont else mrl.Linear(256, 4)
    actor = mrl.seq(lin(8, 256), lin(256, 256), head)
    critic = mrl.seq(lin(8, 256), lin(256, 256), mrl.Linear(256, 1))
    g = torch.Generator(device="cuda").manual_seed(9)
    ap = (torch.rand(actor.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    cp = (torch.rand(critic.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    s0_h = _low_start(E, N, 21, orc)
    rbs = []
    for _ in range(3):
        rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
        rb.actor_params, rb.critic_params = ap, cp
        rb.states.copy_(torch.from_numpy(s0_h.reshape(-1)).cuda())
        rb.obs.copy_(rb.states.view(N, 192)[:, :8].reshape(-1))
        rbs.append(rb)
    single, fused1, fused = rbs
    assert mrl.ppo.rollout_fused(fused.descriptor()) == 1
    # reset seeds stay below 2^63: the reset rounds the seed through fp32 and converts it back to
    # a signed integer (lunar_lander_v2.mojo:1638), which is only defined in that range
    s0, ss, r0, rs = 424242, 2654435761 * N + 7919, 5, 0x9E3779B97F

    # (1) launches of one step each, checked against the oracle after every step
    s_h = s0_h.copy()
    r_h, d_h, o_h = np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros((N, 8), np.float32)
    d1 = fused1.descriptor()
    crashes = leg_obs = landed = resets = 0
    aw = 2 if cont else 1
    for t in range(T):
        mrl.ppo.rollout_steps(ctx, d1, t, 1, (s0 + t * ss) & 0xFFFFFFFF, 0, 0, 0, (r0 + t * rs) & (2**64 - 1), 0)
        ctx.synchronize()
        acts = fused1.r_actions[t * N * aw:(t + 1) * N * aw].cpu().numpy()
        if cont:
            orc.orc_ll_step_continuous_batch(s_h, np.ascontiguousarray(acts.reshape(N, 2)), r_h, d_h, o_h, N)
        else:
            orc.orc_ll_step_batch(s_h, acts, r_h, d_h, o_h, N, 8)
        np.testing.assert_array_equal(fused1.r_rewards[t * N:(t + 1) * N].cpu().numpy(), r_h, err_msg="reward, step %d" % t)
        np.testing.assert_array_equal(fused1.r_dones[t * N:(t + 1) * N].cpu().numpy(), d_h, err_msg="done, step %d" % t)
        crashes += int((r_h == -100).sum())
        landed += int(((d_h > 0) & (r_h > 50)).sum())
        leg_obs += int((o_h[:, 6] + o_h[:, 7] > 0).sum())
        resets += int(d_h.sum())
        orc.orc_ll_selective_reset_batch(s_h, d_h, N, (r0 + t * rs) & (2**64 - 1))
        sg = fused1.states.cpu().numpy().reshape(N, 192)
        np.testing.assert_allclose(sg, s_h, rtol=1e-5, atol=1e-6, err_msg="state, step %d" % t)
        np.testing.assert_allclose(fused1.obs.cpu().numpy().reshape(N, 8), s_h[:, :8], rtol=1e-5, atol=1e-6)
        s_h[:] = sg
    print("  crashes", crashes, "landings", landed, "leg-contact observations", leg_obs, "resets", resets, flush=True)
    assert crashes > N // 40 and leg_obs > N // 4 and resets >= crashes + landed and landed > N // 64

    # (2) the same range as two launches, against single steps
    dsingle, dfused = single.descriptor(), fused.descriptor()
    for t in range(T):
        mrl.ppo.rollout_step(ctx, dsingle, t, (s0 + t * ss) & 0xFFFFFFFF, 0, (r0 + t * rs) & (2**64 - 1))
    k = 23
    mrl.ppo.rollout_steps(ctx, dfused, 0, k, s0, ss & 0xFFFFFFFF, 0, 0, r0, rs)
    mrl.ppo.rollout_steps(ctx, dfused, k, T - k, (s0 + k * ss) & 0xFFFFFFFF, ss & 0xFFFFFFFF, 0, 0,
                          (r0 + k * rs) & (2**64 - 1), rs)
    ctx.synchronize()
    for name in ("r_obs", "r_actions", "r_log_probs", "r_values", "r_rewards", "r_dones", "states", "obs",
                 "ep_return", "ep_length"):
        a, b, c = getattr(single, name), getattr(fused, name), getattr(fused1, name)
        assert torch.equal(a, b), "%s: fused range differs from single steps in %d places" % (name, int((a != b).sum()))
        assert torch.equal(a, c), "%s: one-step launches differ from single steps in %d places" % (name, int((a != c).sum()))
    cnt = int(single.done_count.item())
    assert cnt == int(fused.done_count.item()) == resets


@pytest.mark.parametrize("env,N", [("lunar", 600), ("lunarc", 600), ("lunar", 4128), ("lunarc", 4128)])
def test_fused_collection_with_wind(mrl, orc, env, N):
    """Wind and turbulence switched on for the context: the fused kernels (16-row form up to 4096 envs,
    32-row form above) against the oracle with the same setting, step by step on the kernel's own
    actions, and the same range as one launch against the single steps, bit for bit.  The rows start
    at different step counts, which is the time the gusts are a function of."""
    import numpy as np
    print("case wind", env, N, flush=True)
    T = 24
    ctx = mrl.DeviceContext("cuda:0")           # a context of its own: the setting belongs to the context
    E = mrl.LunarLanderV2 if env == "lunar" else mrl.LunarLanderV2Continuous
    cont = env == "lunarc"
    head = mrl.StochasticActor(256, 2) if cont else mrl.Linear(256, 4)
    actor = mrl.seq(mrl.LinearTanh(8, 256), mrl.LinearTanh(256, 256), head)
    critic = mrl.seq(mrl.LinearTanh(8, 256), mrl.LinearTanh(256, 256), mrl.Linear(256, 1))
    g = torch.Generator(device="cuda").manual_seed(11)
    ap = (torch.rand(actor.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    cp = (torch.rand(critic.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    s0_h = np.zeros((N, 192), np.float32)
    orc.orc_ll_reset_batch(s0_h, N, 17)
    s0_h[:, 188] = (np.arange(N) * 7) % 900
    rbs = []
    for _ in range(3):
        rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
        rb.actor_params, rb.critic_params = ap, cp
        rb.states.copy_(torch.from_numpy(s0_h.reshape(-1)).cuda())
        rb.obs.copy_(rb.states.view(N, 192)[:, :8].reshape(-1))
        rbs.append(rb)
    calm, single, fused = rbs
    s0, ss, r0, rs = 31337, 2654435761 * N + 7919, 5, 0x9E3779B97F
    aw = 2 if cont else 1
    d0 = calm.descriptor()
    mrl.ppo.rollout_steps(ctx, d0, 0, T, s0, ss & 0xFFFFFFFF, 0, 0, r0, rs)      # before the switch: no wind
    E.set_wind(ctx, True, 15.0, 1.5)
    orc.orc_ll_set_wind(1, 15.0, 1.5)
    try:
        s_h = s0_h.copy()
        r_h, d_h, o_h = np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros((N, 8), np.float32)
        d1 = single.descriptor()
        for t in range(T):
            mrl.ppo.rollout_steps(ctx, d1, t, 1, (s0 + t * ss) & 0xFFFFFFFF, 0, 0, 0, (r0 + t * rs) & (2**64 - 1), 0)
            ctx.synchronize()
            acts = single.r_actions[t * N * aw:(t + 1) * N * aw].cpu().numpy()
            if cont:
                orc.orc_ll_step_continuous_batch(s_h, np.ascontiguousarray(acts.reshape(N, 2)), r_h, d_h, o_h, N)
            else:
                orc.orc_ll_step_batch(s_h, acts, r_h, d_h, o_h, N, 8)
            np.testing.assert_array_equal(single.r_rewards[t * N:(t + 1) * N].cpu().numpy(), r_h, err_msg="reward, step %d" % t)
            np.testing.assert_array_equal(single.r_dones[t * N:(t + 1) * N].cpu().numpy(), d_h, err_msg="done, step %d" % t)
            orc.orc_ll_selective_reset_batch(s_h, d_h, N, (r0 + t * rs) & (2**64 - 1))
            sg = single.states.cpu().numpy().reshape(N, 192)
            np.testing.assert_allclose(sg, s_h, rtol=1e-5, atol=1e-6, err_msg="state, step %d" % t)
            s_h[:] = sg
        mrl.ppo.rollout_steps(ctx, fused.descriptor(), 0, T, s0, ss & 0xFFFFFFFF, 0, 0, r0, rs)
        ctx.synchronize()
    finally:
        orc.orc_ll_set_wind(0, 15.0, 1.5)
    for name in ("r_obs", "r_actions", "r_log_probs", "r_values", "r_rewards", "r_dones", "states", "obs"):
        a, b = getattr(single, name), getattr(fused, name)
        assert torch.equal(a, b), "%s: fused range differs from single steps in %d places" % (name, int((a != b).sum()))
    # the gusts moved the landers: against the calm run the horizontal velocities differ on most rows
    dv = (fused.states.view(N, 192)[:, 11] - calm.states.view(N, 192)[:, 11]).abs()
    print("  rows whose vx differs from the calm run: %d of %d, largest %.3f" % (int((dv > 1e-3).sum()), N, float(dv.max())), flush=True)
    assert int((dv > 1e-3).sum()) > N // 2


@pytest.mark.parametrize("env,kind,N", [("bipedal", "tanh", 512), ("cheetah", "tanh", 512), ("car", "relu", 300),
                                        ("bipedal", "relu", 45), ("car_trait", "tanh", 300)])
def test_fused_walker_collection_against_the_oracle(mrl, orc, env, kind, N):
    """car_trait: CarRacingV2 with the reward and termination arithmetic of the GPU trait's step
    (car_racing_v2.mojo:1556-1716) selected for the context and for the oracle."""
    ctx = mrl.DeviceContext("cuda:0")           # a context of its own: the step form belongs to the context
    trait = env == "car_trait"
    if trait:
        env = "car"
        mrl.CarRacingV2.set_step_form(ctx, mrl.CarRacingV2.STEP_GPU_TRAIT)
        orc.orc_cr_set_step_form(1)
    try:
        _walker_collection_against_the_oracle(mrl, ctx, orc, env, kind, N)
    finally:
        orc.orc_cr_set_step_form(0)
        ctx.close()


def _walker_collection_against_the_oracle(mrl, ctx, orc, env, kind, N):
    """The fused collection kernels of BipedalWalker, HalfCheetah and CarRacingV2 in launches of one step,
    against the oracle fed the kernel's own actions: rewards and done flags exact, the rows (state after
    the in-launch reset of finished envs) and the observation bit for bit; then the same 64 steps in two
    launches give the same buffers."""
    import numpy as np
    print("case walker oracle", env, kind, N, flush=True)
    T = 64
    E, step, reset = {"bipedal": (mrl.BipedalWalkerV2, orc.orc_bw_step_batch, orc.orc_bw_reset_batch),
                      "cheetah": (mrl.HalfCheetahPlanarV2, orc.orc_hc_step_batch, orc.orc_hc_reset_batch),
                      "car": (mrl.CarRacingV2, orc.orc_cr_step_batch, orc.orc_cr_reset_batch)}[env]
    S, OBS, AW = E.STATE_SIZE, E.OBS_DIM, E.ACTION_DIM
    lin = mrl.LinearReLU if kind == "relu" else mrl.LinearTanh
    actor = mrl.seq(lin(OBS, 256), lin(256, 256), mrl.StochasticActor(256, AW))
    critic = mrl.seq(lin(OBS, 256), lin(256, 256), mrl.Linear(256, 1))
    g = torch.Generator(device="cuda").manual_seed(11)
    ap = (torch.rand(actor.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    ap[-AW:] = 0.3                                   # log_std: lively actions, so that walkers fall
    cp = (torch.rand(critic.PARAM_SIZE, device="cuda", generator=g) - 0.5) * 0.3
    s0_h = np.zeros((N, S), np.float32)
    reset(s0_h, None, N, 17)
    meta0 = {"bipedal": 942, "cheetah": 245, "car": 34}[env]
    s0_h[::5, meta0] = {"bipedal": 1990.0, "cheetah": 990.0, "car": 490.0}[env]   # some rows near the step limit
    rbs = []
    for _ in range(2):
        rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
        rb.actor_params, rb.critic_params = ap, cp
        rb.states.copy_(torch.from_numpy(s0_h.reshape(-1)).cuda())
        rb.obs.copy_(rb.states.view(N, S)[:, :OBS].reshape(-1))
        rbs.append(rb)
    fused1, fused = rbs
    assert mrl.ppo.rollout_fused(fused.descriptor()) == 1
    s0, ss, r0, rs = 31337, 2654435761 * N + 7919, 5, 0x9E3779B97F
    s_h = s0_h.copy()
    r_h, d_h, o_h = np.zeros(N, np.float32), np.zeros(N, np.float32), np.zeros((N, OBS), np.float32)
    d1 = fused1.descriptor()
    finished = 0
    for t in range(T):
        mrl.ppo.rollout_steps(ctx, d1, t, 1, (s0 + t * ss) & 0xFFFFFFFF, 0, 0, 0, (r0 + t * rs) & (2**64 - 1), 0)
        ctx.synchronize()
        acts = np.ascontiguousarray(fused1.r_actions[t * N * AW:(t + 1) * N * AW].cpu().numpy().reshape(N, AW))
        step(s_h, acts, r_h, d_h, o_h, N, 8)
        np.testing.assert_array_equal(fused1.r_rewards[t * N:(t + 1) * N].cpu().numpy(), r_h, err_msg="reward, step %d" % t)
        np.testing.assert_array_equal(fused1.r_dones[t * N:(t + 1) * N].cpu().numpy(), d_h, err_msg="done, step %d" % t)
        finished += int(d_h.sum())
        flags = d_h.copy()                      # kept alive over the call that reads it through a raw pointer
        reset(s_h, flags.ctypes.data, N, (r0 + t * rs) & (2**64 - 1))
        sg = fused1.states.cpu().numpy().reshape(N, S)
        assert np.array_equal(sg.view(np.uint32), s_h.view(np.uint32)), "state, step %d: %d floats differ" % (
            t, int((sg.view(np.uint32) != s_h.view(np.uint32)).sum()))
        assert np.array_equal(fused1.obs.cpu().numpy().reshape(N, OBS).view(np.uint32), s_h[:, :OBS].view(np.uint32))
    print("  finished episodes", finished, flush=True)
    assert finished >= N // 5
    dfused = fused.descriptor()
    k = 29
    mrl.ppo.rollout_steps(ctx, dfused, 0, k, s0, ss & 0xFFFFFFFF, 0, 0, r0, rs)
    mrl.ppo.rollout_steps(ctx, dfused, k, T - k, (s0 + k * ss) & 0xFFFFFFFF, ss & 0xFFFFFFFF, 0, 0,
                          (r0 + k * rs) & (2**64 - 1), rs)
    ctx.synchronize()
    for name in ("r_obs", "r_actions", "r_log_probs", "r_values", "r_rewards", "r_dones", "states", "obs",
                 "ep_return", "ep_length"):
        a, b = getattr(fused1, name), getattr(fused, name)
        assert torch.equal(a, b), "%s: the 64-step range differs from one-step launches in %d places" % (name, int((a != b).sum()))
    assert int(fused.done_count.item()) == finished


@pytest.mark.parametrize("env", ["lunar", "bipedal", "cheetah"])
def test_barrier_wait_gives_up_and_reports(mrl, env):
    """The wavefront-group barriers inside the fused collection kernels (LunarLander: critic and contact
    detection beside the solver; the walkers: actor ahead of the env step, critic beside it) are bounded:
    with a limit of one poll some wait gives up, the kernel still ends normally, and the next synchronize
    reports it once.  With the default limit the same launch then runs clean."""
    ctx = mrl.DeviceContext("cuda:0")
    N, T = 2048, 4
    one, many = _pair(mrl, ctx, N, T, 256, "relu", env)
    s0, ss = 99, 7919
    ctx.set_spin_limit(1)
    before, obs_before = many.states.clone(), many.obs.clone()
    mrl.ppo.rollout_steps(ctx, many.descriptor(), 0, T, s0, ss, 0, 0, 5, 1)
    with pytest.raises(mrl.MrlError, match="internal barriers"):
        ctx.synchronize()
    ctx.synchronize()                       # reported once, then cleared
    # a workgroup that gave up stores nothing: its rows and observations are those from before the launch
    S = many.env.STATE_SIZE
    kept = (many.states.view(N, S) == before.view(N, S)).all(1)
    obs_kept = (many.obs.view(N, -1) == obs_before.view(N, -1)).all(1)
    print("  rows left as they were:", int(kept.sum()), "of", N, flush=True)
    assert int(kept.sum()) >= 16 and bool((obs_kept | ~kept).all())
    assert bool(torch.isfinite(many.states).all())
    ctx.set_spin_limit(0)
    one, many = _pair(mrl, ctx, N, T, 256, "relu", env)
    d1, d2 = one.descriptor(), many.descriptor()
    for t in range(T):
        mrl.ppo.rollout_step(ctx, d1, t, s0 + t * ss, 0, 5 + t)
    mrl.ppo.rollout_steps(ctx, d2, 0, T, s0, ss, 0, 0, 5, 1)
    ctx.synchronize()
    assert torch.equal(one.states, many.states) and torch.equal(one.r_rewards, many.r_rewards)
    ctx.close()
