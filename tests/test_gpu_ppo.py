"""GPU parity: PPO pieces through the C ABI against the CPU oracle.

Integer-like outputs (sampled actions) and pure fp32 per-element formulas whose only library
calls are exp/log are compared at 1e-5 relative; reductions (normalisation, grad norm) at 1e-5
relative to the oracle's serial fp32 sums; GAE and Adam are per-element chains: 1e-6."""
import ctypes

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def say(*a):
    print(*a, flush=True)


@pytest.fixture(scope="module")
def ctx(mrl):
    return mrl.DeviceContext("cuda:0")


def d(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def h(t):
    return t.cpu().numpy()


def test_sample_categorical(mrl, orc, ctx):
    rng = np.random.default_rng(0)
    n, A = 8192, 4
    logits = rng.normal(size=(n, A)).astype(np.float32) * 2
    a_h, lp_h = np.zeros(n, np.float32), np.zeros(n, np.float32)
    orc.orc_sample_categorical(logits, n, A, 987654321, a_h, lp_h)
    a, lp = torch.zeros(n, device="cuda"), torch.zeros(n, device="cuda")
    mrl.ppo.sample_actions(ctx, d(logits.reshape(-1)), a, lp, 987654321)
    ctx.synchronize()
    # same fp32 operations in the same order, exp and log correctly rounded on both sides:
    # every action and every log-probability is the oracle's, bit for bit
    np.testing.assert_array_equal(h(a), a_h)
    np.testing.assert_array_equal(h(lp), lp_h)
    assert set(np.unique(h(a))) == {0.0, 1.0, 2.0, 3.0}


def test_sample_gaussian(mrl, orc, ctx):
    rng = np.random.default_rng(1)
    n, A = 4096, 6
    out = np.concatenate([rng.normal(size=(n, A)), rng.uniform(-6, 3, (n, A))], 1).astype(np.float32)
    a_h, lp_h = np.zeros((n, A), np.float32), np.zeros(n, np.float32)
    orc.orc_sample_gaussian(out, n, A, 4242, a_h, lp_h)
    a, lp = torch.zeros(n * A, device="cuda"), torch.zeros(n, device="cuda")
    mrl.ppo.sample_continuous_actions(ctx, d(out.reshape(-1)), a, lp, 4242)
    ctx.synchronize()
    np.testing.assert_array_equal(h(a).reshape(n, A), a_h)
    np.testing.assert_array_equal(h(lp), lp_h)


def test_add_obs_noise(mrl, orc, ctx):
    rng = np.random.default_rng(12)
    for n, D, std, seed in ((4096, 24, 0.05, 123456789), (33, 3, 1.5, 4000000000), (1, 8, 0.1, 7)):
        obs = rng.normal(size=(n, D)).astype(np.float32)
        want = obs.copy()
        orc.orc_add_obs_noise(want, n, D, std, seed)
        x = d(obs.reshape(-1))
        mrl.ppo.add_obs_noise(ctx, x, n, std, seed)
        ctx.synchronize()
        np.testing.assert_array_equal(h(x).reshape(n, D), want)
        assert np.abs(want - obs).max() > 0
    x0 = x.clone()
    mrl.ppo.add_obs_noise(ctx, x, 1, 0.0, 7)             # std <= 0: nothing happens
    ctx.synchronize()
    assert torch.equal(x, x0)


@pytest.mark.parametrize("T,N", [(1, 1), (7, 65), (16, 3), (37, 130), (1000, 300), (512, 4096)])
def test_gae(mrl, orc, ctx, T, N):
    say("gae", T, N)
    rng = np.random.default_rng(2)
    r = rng.normal(size=T * N).astype(np.float32); v = rng.normal(size=T * N).astype(np.float32)
    dn = (rng.random(T * N) < 0.02).astype(np.float32); boot = rng.normal(size=N).astype(np.float32)
    adv_h, ret_h = np.zeros(T * N, np.float32), np.zeros(T * N, np.float32)
    orc.orc_gae(T, N, r, v, dn, boot, 0.99, 0.95, adv_h, ret_h)
    adv, ret = torch.zeros(T * N, device="cuda"), torch.zeros(T * N, device="cuda")
    mrl.ppo.compute_gae(ctx, d(r), d(v), d(dn), d(boot), 0.99, 0.95, adv, ret)
    ctx.synchronize()
    np.testing.assert_array_equal(h(adv), adv_h)       # same fp32 operations in the same order
    np.testing.assert_array_equal(h(ret), ret_h)


@pytest.mark.parametrize("n", [1, 1000, 4096, 512 * 4096])
def test_normalize_advantages(mrl, orc, ctx, n):
    rng = np.random.default_rng(3)
    a = rng.normal(1.5, 2.5, n).astype(np.float32)
    a64 = a.astype(np.float64)
    want = (a64 - a64.mean()) / (np.sqrt(a64.var() + 1e-8) + 1e-8)
    x = d(a)
    mrl.ppo.normalize_advantages(ctx, x)
    ctx.synchronize()
    np.testing.assert_allclose(h(x), want, rtol=1e-4, atol=2e-5)
    if n <= 4096:                                      # the oracle's serial fp32 sums, where they are still accurate
        b = a.copy(); orc.orc_normalize_minibatch_fused(b, n)
        np.testing.assert_allclose(h(x), b, rtol=1e-4, atol=2e-5)


def test_gather_minibatch(mrl, ctx):
    rng = np.random.default_rng(4)
    TN, OBS, MB = 5000, 8, 1024
    bufs = [rng.normal(size=TN * OBS).astype(np.float32)] + [rng.normal(size=TN).astype(np.float32) for _ in range(5)]
    idx = rng.permutation(TN)[:MB].astype(np.int32)
    roll = [d(b) for b in bufs]
    mbs = [torch.zeros(MB * OBS, device="cuda")] + [torch.zeros(MB, device="cuda") for _ in range(5)]
    mrl.ppo.gather_minibatch(ctx, d(idx), roll, mbs, OBS, 1)
    ctx.synchronize()
    np.testing.assert_array_equal(h(mbs[0]).reshape(MB, OBS), bufs[0].reshape(TN, OBS)[idx])
    for k in range(1, 6):
        np.testing.assert_array_equal(h(mbs[k]), bufs[k][idx])


def test_actor_grad_discrete(mrl, orc, ctx):
    rng = np.random.default_rng(5)
    mb, A = 4096, 4
    logits = rng.normal(size=(mb, A)).astype(np.float32)
    acts = rng.integers(0, A, mb).astype(np.float32); adv = rng.normal(size=mb).astype(np.float32)
    old = (np.log(1.0 / A) + rng.uniform(-0.6, 0.6, mb)).astype(np.float32)
    g_h, kl_h = np.zeros((mb, A), np.float32), np.zeros(mb, np.float32)
    orc.orc_ppo_actor_grad_discrete(logits, old, adv, acts, mb, A, 0.2, 0.01, g_h, kl_h)
    g, kl = torch.zeros(mb * A, device="cuda"), torch.zeros(mb, device="cuda")
    mrl.ppo.ppo_actor_grad_with_kl(ctx, g, kl, d(logits.reshape(-1)), d(old), d(adv), d(acts), 0.2, 0.01)
    ctx.synchronize()
    gg = h(g).reshape(mb, A)
    np.testing.assert_array_equal(gg, g_h)             # incl. which rows the clip test zeroes
    np.testing.assert_array_equal(h(kl), kl_h)
    assert 0.05 < (g_h == 0).all(1).mean() < 0.95      # both branches exercised


def test_actor_grad_gaussian(mrl, orc, ctx):
    rng = np.random.default_rng(6)
    mb, A = 4096, 6
    out = np.concatenate([rng.normal(size=(mb, A)), rng.uniform(-1.5, 0.5, (mb, A))], 1).astype(np.float32)
    acts = (out[:, :A] + rng.normal(size=(mb, A)) * np.exp(out[:, A:])).astype(np.float32)
    adv = rng.normal(size=mb).astype(np.float32)
    z = (acts - out[:, :A]) / (np.exp(out[:, A:]) + 1e-6)
    old = ((-0.5 * (np.log(2 * np.pi) + 2 * out[:, A:] + z * z)).sum(1) + rng.uniform(-0.4, 0.4, mb)).astype(np.float32)
    g_h, kl_h = np.zeros((mb, 2 * A), np.float32), np.zeros(mb, np.float32)
    orc.orc_ppo_actor_grad_gaussian(out, old, adv, acts, mb, A, 0.2, 0.01, g_h, kl_h)
    g, kl = torch.zeros(mb * 2 * A, device="cuda"), torch.zeros(mb, device="cuda")
    mrl.ppo.ppo_continuous_actor_grad(ctx, g, kl, d(out.reshape(-1)), d(old), d(adv), d(acts.reshape(-1)), 0.2, 0.01)
    ctx.synchronize()
    gg = h(g).reshape(mb, 2 * A)
    np.testing.assert_array_equal(gg, g_h)
    np.testing.assert_array_equal(h(kl), kl_h)
    assert 0.05 < (g_h == 0).all(1).mean() < 0.95


@pytest.mark.parametrize("conv,clipped", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_critic_grad(mrl, orc, ctx, conv, clipped):
    rng = np.random.default_rng(7)
    mb = 4096
    v = rng.normal(size=mb).astype(np.float32); vo = (v + rng.normal(size=mb) * 0.3).astype(np.float32)
    ret = rng.normal(size=mb).astype(np.float32)
    g_h = np.zeros(mb, np.float32)
    orc.orc_ppo_critic_grad(v, vo, ret, mb, conv, clipped, 0.5, 0.2, g_h)
    g = torch.zeros(mb, device="cuda")
    mrl.ppo.ppo_critic_grad(ctx, g, d(v), d(ret), 0.5, d(vo) if clipped else None, 0.2, continuous=bool(conv))
    ctx.synchronize()
    np.testing.assert_array_equal(h(g), g_h)


def test_clip_grad_norm(mrl, orc, ctx):
    rng = np.random.default_rng(8)
    for n, scale in ((69124, 1.0), (69124, 1e-4), (5, 3.0)):
        g0 = (rng.normal(size=n) * scale).astype(np.float32)
        g_h = g0.copy(); orc.orc_clip_grad_norm(g_h, n, 0.5)
        g = d(g0)
        mrl.ppo.clip_grad_norm(ctx, g, 0.5)
        ctx.synchronize()
        np.testing.assert_allclose(h(g), g_h, rtol=1e-5, atol=1e-12)
        assert np.linalg.norm(h(g).astype(np.float64)) <= 0.5 * (1 + 1e-5)


def test_adam_three_steps(mrl, orc, ctx):
    rng = np.random.default_rng(9)
    n = 69124
    p0 = rng.normal(size=n).astype(np.float32)
    p_h, st_h = p0.copy(), np.zeros(2 * n, np.float32)
    p, st = d(p0), torch.zeros(2 * n, device="cuda")
    opt = mrl.Adam(lr=3e-4)
    for t in range(1, 4):
        g = rng.normal(size=n).astype(np.float32) * 0.01
        orc.orc_adam_step(p_h, g, st_h, n, t, 3e-4, 0.9, 0.999, 1e-8)
        opt.step_gpu(ctx, p, d(g), st)
        ctx.synchronize()
        np.testing.assert_allclose(h(p), p_h, rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(h(st), st_h, rtol=1e-6, atol=1e-12)
    assert opt.t == 3


def test_clamp_log_std(mrl, ctx):
    p = torch.tensor([0.0, 1.0, -9.0, 0.3, 5.0], device="cuda")
    mrl.ppo.clamp_log_std_params(ctx, p, 2, 3)
    ctx.synchronize()
    assert p.tolist() == [0.0, 1.0, -5.0, pytest.approx(0.3), 2.0]


def test_rollout_step_equals_its_parts(mrl, ctx):
    """The fused collection step against the same sequence issued call by call
    (forward, sample, store, step, selective reset, accounting).  The fused policy kernel sums
    in a different order than the layer-by-layer kernels, so values / log-probs are compared at
    the MLP tolerance and the env is then stepped with the fused path's own actions."""
    torch.manual_seed(0)
    N, T = 1000, 6
    E = mrl.LunarLanderV2
    actor = mrl.seq(mrl.LinearReLU(8, 256), mrl.LinearReLU(256, 256), mrl.Linear(256, 4))
    critic = mrl.seq(mrl.LinearReLU(8, 256), mrl.LinearReLU(256, 256), mrl.Linear(256, 1))
    ap = (torch.rand(actor.PARAM_SIZE, device="cuda") - 0.5) * 0.3
    cp = (torch.rand(critic.PARAM_SIZE, device="cuda") - 0.5) * 0.3
    rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
    rb.actor_params, rb.critic_params = ap, cp
    E.reset_kernel_gpu(ctx, rb.states, 3)
    rb.states.view(N, 192)[:, 188] = torch.randint(994, 1000, (N,), device="cuda").float()   # episodes end soon
    rb.obs.copy_(rb.states.view(N, 192)[:, :8].reshape(-1))
    s2, o2 = rb.states.clone(), rb.obs.clone()
    desc = rb.descriptor()
    z = lambda n: torch.zeros(n, device="cuda")
    logits, values, acts, lps, rew, dn = z(N * 4), z(N), z(N), z(N), z(N), z(N)
    ep_r, ep_l, finished = z(N), z(N), []
    for t in range(T):
        mrl.ppo.rollout_step(ctx, desc, t, 100 + t, 0, 500 + t)
        actor.forward_gpu_no_cache_ws(ctx, logits, o2, ap)
        critic.forward_gpu_no_cache_ws(ctx, values, o2, cp)
        mrl.ppo.sample_actions(ctx, logits, acts, lps, 100 + t)
        ctx.synchronize()
        sl = slice(t * N, (t + 1) * N)
        assert torch.equal(rb.r_obs[t * N * 8:(t + 1) * N * 8], o2)
        same = rb.r_actions[sl] == acts
        assert same.float().mean() > 0.995
        torch.testing.assert_close(rb.r_log_probs[sl][same], lps[same], rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(rb.r_values[sl], values, rtol=1e-4, atol=1e-5)
        acts.copy_(rb.r_actions[sl])
        E.step_kernel_gpu(ctx, s2, acts, rew, dn, o2, 0)
        ep_r += rew; ep_l += 1
        ctx.synchronize()
        assert torch.equal(rb.r_rewards[sl], rew) and torch.equal(rb.r_dones[sl], dn)
        fin = dn > 0.5
        finished += list(zip(ep_r[fin].tolist(), ep_l[fin].tolist()))
        ep_r[fin] = 0; ep_l[fin] = 0
        E.selective_reset_kernel_gpu(ctx, s2, dn, 500 + t)
        o2.copy_(s2.view(N, 192)[:, :8].reshape(-1))
        ctx.synchronize()
        assert torch.equal(rb.states, s2) and torch.equal(rb.obs, o2)
        assert torch.equal(rb.ep_return, ep_r) and torch.equal(rb.ep_length, ep_l)
    cnt = int(rb.done_count.item())
    assert cnt == len(finished) and cnt > N // 2
    got = sorted(zip(rb.done_returns[:cnt].tolist(), rb.done_lengths[:cnt].tolist()))
    assert got == sorted(finished)


@pytest.mark.parametrize("hidden,kind,obs_dim,na,n", [(256, "relu", 8, 4, 8192), (256, "tanh", 24, 6, 333),
                                                       (64, "relu", 4, 2, 4096), (64, "tanh", 3, 3, 31)])
def test_fused_policy_kernel_against_layerwise_path_and_oracle(mrl, orc, orcmod, ctx, hidden, kind, obs_dim, na, n):
    """Fused policy/value/sampling kernel (via the rollout step of a do-nothing-else harness) against
    the oracle's serial fp32 forward: logits are not exposed, so values and log-probs are the probes."""
    say("fused policy", hidden, kind, n)
    Lay = mrl.LinearReLU if kind == "relu" else mrl.LinearTanh
    k = 1 if kind == "relu" else 2
    actor = mrl.seq(Lay(obs_dim, hidden), Lay(hidden, hidden), mrl.Linear(hidden, na))
    critic = mrl.seq(Lay(obs_dim, hidden), Lay(hidden, hidden), mrl.Linear(hidden, 1))
    rng = np.random.default_rng(hidden + n)
    ap = rng.uniform(-0.15, 0.15, actor.PARAM_SIZE).astype(np.float32)
    cp = rng.uniform(-0.15, 0.15, critic.PARAM_SIZE).astype(np.float32)
    obs = rng.normal(size=(n, obs_dim)).astype(np.float32)
    la = orcmod.layers([(k, obs_dim, hidden), (k, hidden, hidden), (0, hidden, na)])
    lc = orcmod.layers([(k, obs_dim, hidden), (k, hidden, hidden), (0, hidden, 1)])
    logits_h, values_h = np.zeros((n, na), np.float32), np.zeros((n, 1), np.float32)
    orc.orc_mlp_forward(la, 3, n, obs, ap, logits_h, None)
    orc.orc_mlp_forward(lc, 3, n, obs, cp, values_h, None)
    a_h, lp_h = np.zeros(n, np.float32), np.zeros(n, np.float32)
    orc.orc_sample_categorical(logits_h, n, na, 77, a_h, lp_h)
    out = [torch.zeros(m, device="cuda") for m in (n, n * obs_dim, n, n, n)]
    obs_d, ap_d, cp_d = d(obs.reshape(-1)), d(ap), d(cp)      # keep the device copies alive
    mrl._lib.call("mrl_policy_step_discrete", ctx.handle, ctypes.byref(actor.desc), ctypes.byref(critic.desc), n,
                  obs_d.data_ptr(), ap_d.data_ptr(), cp_d.data_ptr(), 77, *[o.data_ptr() for o in out])
    ctx.synchronize()
    actions, r_obs, r_actions, r_logp, r_values = (h(o) for o in out)
    np.testing.assert_array_equal(r_obs.reshape(n, obs_dim), obs)
    np.testing.assert_array_equal(actions, r_actions)
    np.testing.assert_allclose(r_values, values_h[:, 0], rtol=1e-4, atol=1e-5)
    # the kernel's logits differ from the oracle's serial sums at the MLP tolerance, so a draw may
    # land on the other side of a CDF boundary -- but only where u is that close to one
    same = r_actions == a_h
    assert same.mean() > 0.995, same.mean()
    np.testing.assert_allclose(r_logp[same], lp_h[same], rtol=1e-4, atol=1e-5)
    if not same.all():
        rows = np.nonzero(~same)[0]
        p64 = np.exp(logits_h[rows].astype(np.float64) - logits_h[rows].max(1, keepdims=True))
        cdf = np.cumsum(p64 / p64.sum(1, keepdims=True), 1)
        x = (np.uint32(77) ^ (rows.astype(np.uint64) * 2654435761 & 0xFFFFFFFF).astype(np.uint32)).astype(np.uint64)
        for _ in range(2):               # seeding step, then the draw (deep_rl/gpu/random.mojo:11-29)
            x ^= (x << np.uint64(13)) & np.uint64(0xFFFFFFFF); x ^= x >> np.uint64(17); x ^= (x << np.uint64(5)) & np.uint64(0xFFFFFFFF)
        u = x.astype(np.float64) / 4294967295.0
        assert np.abs(cdf - u[:, None]).min(1).max() < 2e-5
        assert np.abs(r_actions[rows] - a_h[rows]).max() == 1.0      # the neighbouring action, nothing else


@pytest.mark.parametrize("hidden,kind,obs_dim,A,n", [(256, "tanh", 17, 6, 4096), (256, "relu", 24, 4, 333),
                                                      (64, "tanh", 3, 1, 16384), (64, "relu", 5, 8, 31)])
def test_fused_gaussian_policy_kernel_against_oracle(mrl, orc, orcmod, ctx, hidden, kind, obs_dim, A, n):
    """Fused actor(StochasticActor head) + critic + Gaussian sampling + stores against the oracle's
    forward and sampler.  The noise comes from the same Philox streams, so action = mean + std * z
    differs from the oracle's only through the mean: MLP tolerance."""
    say("fused gaussian policy", hidden, kind, n)
    Lay = mrl.LinearReLU if kind == "relu" else mrl.LinearTanh
    k = 1 if kind == "relu" else 2
    actor = mrl.seq(Lay(obs_dim, hidden), Lay(hidden, hidden), mrl.StochasticActor(hidden, A))
    critic = mrl.seq(Lay(obs_dim, hidden), Lay(hidden, hidden), mrl.Linear(hidden, 1))
    rng = np.random.default_rng(hidden + n)
    ap = rng.uniform(-0.15, 0.15, actor.PARAM_SIZE).astype(np.float32)
    ap[-A:] = rng.uniform(-6.0, 2.5, A)          # log_std, partly outside the clamp range
    cp = rng.uniform(-0.15, 0.15, critic.PARAM_SIZE).astype(np.float32)
    obs = rng.normal(size=(n, obs_dim)).astype(np.float32)
    la = orcmod.layers([(k, obs_dim, hidden), (k, hidden, hidden), (3, hidden, A)])
    lc = orcmod.layers([(k, obs_dim, hidden), (k, hidden, hidden), (0, hidden, 1)])
    out_h, values_h = np.zeros((n, 2 * A), np.float32), np.zeros((n, 1), np.float32)
    orc.orc_mlp_forward(la, 3, n, obs, ap, out_h, None)
    orc.orc_mlp_forward(lc, 3, n, obs, cp, values_h, None)
    a_h, lp_h = np.zeros((n, A), np.float32), np.zeros(n, np.float32)
    orc.orc_sample_gaussian(out_h, n, A, 4242, a_h, lp_h)
    out = [torch.zeros(m, device="cuda") for m in (n * A, n * obs_dim, n * A, n, n)]
    obs_d, ap_d, cp_d = d(obs.reshape(-1)), d(ap), d(cp)
    mrl._lib.call("mrl_policy_step_gaussian", ctx.handle, ctypes.byref(actor.desc), ctypes.byref(critic.desc), n,
                  obs_d.data_ptr(), ap_d.data_ptr(), cp_d.data_ptr(), 4242, *[o.data_ptr() for o in out])
    ctx.synchronize()
    actions, r_obs, r_actions, r_logp, r_values = (h(o) for o in out)
    np.testing.assert_array_equal(r_obs.reshape(n, obs_dim), obs)
    np.testing.assert_array_equal(actions, r_actions)
    np.testing.assert_allclose(r_values, values_h[:, 0], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(actions.reshape(n, A), a_h, rtol=1e-4, atol=2e-5)
    # log-prob: ((a - mean) / std)^2 amplifies the mean's rounding by 1/std (std down to e^-5)
    np.testing.assert_allclose(r_logp, lp_h, rtol=1e-3, atol=2e-2)
    wide = ap[-A:].min() > -2.0
    if wide:
        np.testing.assert_allclose(r_logp, lp_h, rtol=1e-4, atol=1e-3)


def test_gaussian_policy_step_layerwise_path(mrl, orc, orcmod, ctx):
    """A shape the fused kernel does not cover (hidden 128) takes the layer-by-layer path."""
    n, obs_dim, hidden, A = 500, 11, 128, 3
    actor = mrl.seq(mrl.LinearTanh(obs_dim, hidden), mrl.LinearTanh(hidden, hidden), mrl.StochasticActor(hidden, A))
    critic = mrl.seq(mrl.LinearTanh(obs_dim, hidden), mrl.LinearTanh(hidden, hidden), mrl.Linear(hidden, 1))
    rng = np.random.default_rng(5)
    ap = rng.uniform(-0.15, 0.15, actor.PARAM_SIZE).astype(np.float32)
    cp = rng.uniform(-0.15, 0.15, critic.PARAM_SIZE).astype(np.float32)
    obs = rng.normal(size=(n, obs_dim)).astype(np.float32)
    la = orcmod.layers([(2, obs_dim, hidden), (2, hidden, hidden), (3, hidden, A)])
    lc = orcmod.layers([(2, obs_dim, hidden), (2, hidden, hidden), (0, hidden, 1)])
    out_h, values_h = np.zeros((n, 2 * A), np.float32), np.zeros((n, 1), np.float32)
    orc.orc_mlp_forward(la, 3, n, obs, ap, out_h, None)
    orc.orc_mlp_forward(lc, 3, n, obs, cp, values_h, None)
    a_h, lp_h = np.zeros((n, A), np.float32), np.zeros(n, np.float32)
    orc.orc_sample_gaussian(out_h, n, A, 9, a_h, lp_h)
    out = [torch.zeros(m, device="cuda") for m in (n * A, n * obs_dim, n * A, n, n)]
    obs_d, ap_d, cp_d = d(obs.reshape(-1)), d(ap), d(cp)
    mrl._lib.call("mrl_policy_step_gaussian", ctx.handle, ctypes.byref(actor.desc), ctypes.byref(critic.desc), n,
                  obs_d.data_ptr(), ap_d.data_ptr(), cp_d.data_ptr(), 9, *[o.data_ptr() for o in out])
    ctx.synchronize()
    actions, r_obs, r_actions, r_logp, r_values = (h(o) for o in out)
    np.testing.assert_array_equal(r_obs.reshape(n, obs_dim), obs)
    np.testing.assert_allclose(actions.reshape(n, A), a_h, rtol=1e-4, atol=2e-5)
    np.testing.assert_allclose(r_values, values_h[:, 0], rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(r_logp, lp_h, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("env_name,N", [("PendulumV2", 1000), ("HalfCheetahPlanarV2", 300)])
def test_continuous_rollout_step_equals_its_parts(mrl, ctx, env_name, N):
    """mrl_rollout_step for a continuous agent against forward + sample + step + selective reset."""
    torch.manual_seed(1)
    T = 4
    E = getattr(mrl, env_name)
    od, A, S = E.OBS_DIM, E.ACTION_DIM, E.STATE_SIZE
    actor = mrl.seq(mrl.LinearTanh(od, 64), mrl.LinearTanh(64, 64), mrl.StochasticActor(64, A))
    critic = mrl.seq(mrl.LinearTanh(od, 64), mrl.LinearTanh(64, 64), mrl.Linear(64, 1))
    ap = (torch.rand(actor.PARAM_SIZE, device="cuda") - 0.5) * 0.3
    cp = (torch.rand(critic.PARAM_SIZE, device="cuda") - 0.5) * 0.3
    rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
    assert rb.continuous and rb.act_width == A
    rb.actor_params, rb.critic_params = ap, cp
    E.reset_kernel_gpu(ctx, rb.states, 3)
    rb.obs.copy_(rb.states.view(N, S)[:, :od].reshape(-1))
    s2, o2 = rb.states.clone(), rb.obs.clone()
    desc = rb.descriptor()
    z = lambda n: torch.zeros(n, device="cuda")
    head, values, acts, lps, rew, dn = z(N * 2 * A), z(N), z(N * A), z(N), z(N), z(N)
    for t in range(T):
        mrl.ppo.rollout_step(ctx, desc, t, 100 + t, 0, 500 + t)
        actor.forward_gpu_no_cache_ws(ctx, head, o2, ap)
        critic.forward_gpu_no_cache_ws(ctx, values, o2, cp)
        mrl.ppo.sample_continuous_actions(ctx, head, acts, lps, 100 + t)
        ctx.synchronize()
        sl = slice(t * N, (t + 1) * N)
        assert torch.equal(rb.r_obs[t * N * od:(t + 1) * N * od], o2)
        torch.testing.assert_close(rb.r_actions[t * N * A:(t + 1) * N * A], acts, rtol=1e-4, atol=2e-5)
        torch.testing.assert_close(rb.r_log_probs[sl], lps, rtol=1e-4, atol=1e-3)
        torch.testing.assert_close(rb.r_values[sl], values, rtol=1e-4, atol=1e-5)
        acts.copy_(rb.r_actions[t * N * A:(t + 1) * N * A])
        E.step_kernel_gpu(ctx, s2, acts, rew, dn, o2, 0)
        ctx.synchronize()
        assert torch.equal(rb.r_rewards[sl], rew) and torch.equal(rb.r_dones[sl], dn)
        E.selective_reset_kernel_gpu(ctx, s2, dn, 500 + t)
        o2.copy_(s2.view(N, S)[:, :od].reshape(-1))
        ctx.synchronize()
        assert torch.equal(rb.states, s2) and torch.equal(rb.obs, o2)


def test_running_mean_std(mrl, orc, orcmod, ctx):
    rng = np.random.default_rng(3)
    rms_h = orcmod.Rms(0.0, 0.0, 0.0)
    rms = mrl.ppo.RunningMeanStd(ctx)
    for n, scale, shift in ((1, 1.0, 0.0), (4096 * 50, 3.0, -2.0), (1000, 0.1, 7.0)):
        x = (rng.normal(size=n) * scale + shift).astype(np.float32)
        xd = d(x)
        orc.orc_rms_update(ctypes.byref(rms_h), x, n)
        rms.update(xd)
        st = h(rms.state)
        np.testing.assert_allclose(st, [rms_h.count, rms_h.mean, rms_h.var_sum], rtol=1e-12, atol=1e-12)
        y = x.copy()
        orc.orc_rms_normalize(ctypes.byref(rms_h), y, n)
        rms.normalize(xd)
        np.testing.assert_allclose(h(xd), y, rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("n", [1, 2, 5, 1000, 4096, 65537, 4096 * 1000])
def test_permutation_is_a_permutation(mrl, ctx, n):
    idx = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    mrl.ppo.permutation(ctx, idx, 12345)
    first = idx.clone()
    assert torch.equal(torch.sort(idx.long()).values, torch.arange(n, device="cuda"))
    mrl.ppo.permutation(ctx, idx, 12345)
    assert torch.equal(idx, first)                      # deterministic in the seed
    if n >= 1000:
        mrl.ppo.permutation(ctx, idx, 12346)
        assert (idx == first).float().mean() < 0.01     # another seed, another permutation
        # no structure left from the identity: displacement |p(i) - i| of a random permutation
        # has mean n/3, and each tenth of the range receives a tenth of the first tenth
        # (tolerances: 4.5 standard deviations of the statistic under a uniform permutation)
        disp = (first.double() - torch.arange(n, device="cuda").double()).abs().mean().item()
        assert abs(disp / n - 1 / 3) < 4.5 * 0.236 / n ** 0.5 + 1e-3
        head = first[: n // 10].long() * 10 // n
        counts = torch.bincount(head, minlength=10).double()
        assert (counts / counts.sum() - 0.1).abs().max() < 4.5 * (0.09 / (n // 10)) ** 0.5


@pytest.mark.parametrize("n", [1, 2, 3, 5, 8, 1000, 4096, 65537, 4096 * 1000])
def test_shuffle_indices_is_the_reference_fisher_yates(mrl, orc, ctx, n):
    """mrl_permutation_from_uniforms against the oracle's serial Fisher-Yates
    (core/utils/shuffle.mojo:21-48) on the same draws: the same permutation index for index.  The
    draws include exact 0.0 and values one ulp below 1 (the last bin), and 1.0 itself at small n
    (the loop's `if j > i` clamp)."""
    rng = np.random.default_rng(n)
    u = rng.random(max(n - 1, 1))
    if n > 8:
        u[rng.integers(0, n - 1, 16)] = 0.0
        u[rng.integers(0, n - 1, 16)] = np.nextafter(1.0, 0.0)
        u[rng.integers(0, n - 1, 4)] = 1.0
    elif n > 2:
        u[0] = 1.0
    want = np.zeros(n, np.int32)
    orc.orc_shuffle_indices(n, u, want)
    idx = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    ws = torch.full((2 * n + 1,), 7, dtype=torch.int32, device="cuda")     # dirty scratch
    mrl.ppo.shuffle_indices(ctx, idx, d(u), ws)
    np.testing.assert_array_equal(h(idx), want)
    mrl.ppo.shuffle_indices(ctx, idx, d(u), ws)                                # and again over its own leftovers
    np.testing.assert_array_equal(h(idx), want)
    assert sorted(want.tolist()) == list(range(n))


def test_kl_check_flag(mrl, ctx):
    kl = torch.full((4096,), 0.01, device="cuda")
    flag = torch.zeros(2, dtype=torch.int32, device="cuda")
    mrl.ppo.kl_check(ctx, kl, 0.015, flag)
    assert flag[0].item() == 0
    assert abs(flag[1:2].view(torch.float32).item() - 0.01) < 1e-7
    kl[:2048] = 0.03
    mrl.ppo.kl_check(ctx, kl, 0.015, flag)
    assert flag[0].item() == 1
    kl.fill_(0.0)
    mrl.ppo.kl_check(ctx, kl, 0.015, flag)
    assert flag[0].item() == 1 and flag[1:2].view(torch.float32).item() == 0.0   # sticky


def test_init_uniform_and_network(mrl, orc, ctx):
    n = 1003
    p = torch.zeros(n, device="cuda")
    mrl._lib.call("mrl_init_uniform", ctx.handle, p.data_ptr(), n, -0.5, 1.5, 99)
    got = h(p)
    want = np.zeros(n + 1, np.float32)
    u = np.zeros(4, np.float32)
    for q in range((n + 3) // 4):
        orc.orc_philox_uniform4(99, q, 0, u)
        want[4 * q:4 * q + 4] = np.float32(-0.5) + u * np.float32(2.0)
    np.testing.assert_array_equal(got, want[:n])
    model = mrl.seq(mrl.LinearReLU(8, 256), mrl.LinearReLU(256, 256), mrl.Linear(256, 4))
    net = mrl.Network(ctx, model, mrl.Adam(lr=3e-4), mrl.Xavier(seed=1))
    w = h(net.params)
    b = (2.0 / (8 + 4)) ** 0.5
    assert w.shape == (69124,) and np.abs(w).max() <= b and np.abs(w).max() > 0.99 * b
    assert abs(w.mean()) < 0.01 * b * 3 and abs(w.std() - b / 3 ** 0.5) < 0.01 * b
    assert net.grads.abs().sum().item() == 0 and net.optimizer_state.numel() == 2 * 69124
    amodel = mrl.seq(mrl.LinearTanh(17, 256), mrl.LinearTanh(256, 256), mrl.StochasticActor(256, 6))
    anet = mrl.Network(ctx, amodel, mrl.Adam(lr=3e-4), mrl.Kaiming(seed=2))
    off = 17 * 256 + 256 + 256 * 256 + 256
    mrl.init_params_small(ctx, anet.params, off, 256, 6, seed=3)
    a = h(anet.params)
    assert np.abs(a[:off]).max() <= (2.0 / 17) ** 0.5
    assert np.abs(a[off:off + 256 * 6]).max() <= 0.01 and np.all(a[off + 1536:off + 1542] == 0.0)
    assert np.all(a[-6:] == np.float32(-0.5))


@pytest.mark.parametrize("H", [64, 128])     # 64: actor and critic share fused launches; 128: layer-by-layer path
def test_continuous_update_minibatch_against_oracle(mrl, orc, orcmod, ctx, H):
    """One ContinuousUpdate minibatch (gather, per-minibatch normalisation, actor forward, Gaussian
    loss gradient, backward, clip, Adam, log_std clamp, critic forward, gradient, backward, clip,
    Adam) against the same sequence on the oracle."""
    rng = np.random.default_rng(11)
    N, T, MB = 64, 8, 256
    E = mrl.HalfCheetahPlanarV2
    od, A = E.OBS_DIM, E.ACTION_DIM
    actor = mrl.seq(mrl.LinearTanh(od, H), mrl.LinearTanh(H, H), mrl.StochasticActor(H, A))
    critic = mrl.seq(mrl.LinearTanh(od, H), mrl.LinearTanh(H, H), mrl.Linear(H, 1))
    la = orcmod.layers([(2, od, H), (2, H, H), (3, H, A)])
    lc = orcmod.layers([(2, od, H), (2, H, H), (0, H, 1)])
    ap = rng.uniform(-0.2, 0.2, actor.PARAM_SIZE).astype(np.float32)
    ap[-A:] = -0.5
    cp = rng.uniform(-0.2, 0.2, critic.PARAM_SIZE).astype(np.float32)
    rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
    rb.actor_params, rb.critic_params = d(ap), d(cp)
    total = N * T
    r_obs = rng.normal(size=(total, od)).astype(np.float32)
    # behaviour policy = current policy: old log-probs from the oracle's own sampler
    out0 = np.zeros((total, 2 * A), np.float32)
    orc.orc_mlp_forward(la, 3, total, r_obs, ap, out0, None)
    r_act, r_lp = np.zeros((total, A), np.float32), np.zeros(total, np.float32)
    orc.orc_sample_gaussian(out0, total, A, 5, r_act, r_lp)
    r_lp += rng.normal(size=total).astype(np.float32) * 0.05     # ratio != 1
    r_val = rng.normal(size=total).astype(np.float32)
    adv = rng.normal(size=total).astype(np.float32)
    ret = (r_val + adv).astype(np.float32)
    rb.r_obs.copy_(d(r_obs.reshape(-1))); rb.r_actions.copy_(d(r_act.reshape(-1)))
    rb.r_log_probs.copy_(d(r_lp)); rb.r_values.copy_(d(r_val))
    aopt, copt = mrl.Adam(lr=3e-4), mrl.Adam(lr=1e-3)
    upd = mrl.ppo.ContinuousUpdate(ctx, rb, MB, aopt, copt, target_kl=0.0)
    upd.advantages.copy_(d(adv)); upd.returns.copy_(d(ret))
    idx = rng.permutation(total)[:MB].astype(np.int32)
    upd.minibatch_step(d(idx))
    ctx.synchronize()
    # oracle
    mo, ma, madv = r_obs[idx], r_act[idx], adv[idx].copy()
    orc.orc_normalize_minibatch_host(madv, MB)
    cache = np.zeros(MB * actor.CACHE_SIZE, np.float32)
    out = np.zeros((MB, 2 * A), np.float32)
    orc.orc_mlp_forward(la, 3, MB, mo, ap, out, cache.ctypes.data)
    g_out, kl = np.zeros((MB, 2 * A), np.float32), np.zeros(MB, np.float32)
    orc.orc_ppo_actor_grad_gaussian(out, r_lp[idx], madv, ma, MB, A, 0.2, 0.01, g_out, kl)
    ga = np.zeros(actor.PARAM_SIZE, np.float32)
    orc.orc_mlp_backward(la, 3, MB, g_out, ap, cache, ga, None)
    orc.orc_clip_grad_norm(ga, ga.size, 0.5)
    st = np.zeros(2 * ga.size, np.float32)
    ap2 = ap.copy()
    orc.orc_adam_step(ap2, ga, st, ga.size, 1, 3e-4, 0.9, 0.999, 1e-8)
    orc.orc_clamp_log_std(ap2, ap2.size - A, A)
    np.testing.assert_allclose(h(upd.kl), kl, rtol=1e-3, atol=1e-5)
    np.testing.assert_allclose(h(upd.actor_grads), ga, rtol=1e-3, atol=1e-6)
    # the first Adam step is lr * g / (|g| + eps): for a gradient entry near eps = 1e-8 the step
    # follows the entry's absolute rounding error, so parameters are compared to a few % of lr
    np.testing.assert_allclose(h(rb.actor_params), ap2, rtol=1e-5, atol=0.03 * 3e-4)
    ccache = np.zeros(MB * critic.CACHE_SIZE, np.float32)
    v = np.zeros((MB, 1), np.float32)
    orc.orc_mlp_forward(lc, 3, MB, mo, cp, v, ccache.ctypes.data)
    gv = np.zeros(MB, np.float32)
    orc.orc_ppo_critic_grad(v.reshape(-1), r_val[idx], ret[idx], MB, 1, 1, 0.5, 0.2, gv)
    gc = np.zeros(critic.PARAM_SIZE, np.float32)
    orc.orc_mlp_backward(lc, 3, MB, gv.reshape(MB, 1), cp, ccache, gc, None)
    orc.orc_clip_grad_norm(gc, gc.size, 0.5)
    st = np.zeros(2 * gc.size, np.float32)
    cp2 = cp.copy()
    orc.orc_adam_step(cp2, gc, st, gc.size, 1, 1e-3, 0.9, 0.999, 1e-8)
    np.testing.assert_allclose(h(upd.critic_grads), gc, rtol=1e-3, atol=1e-6)
    np.testing.assert_allclose(h(rb.critic_params), cp2, rtol=1e-5, atol=0.03 * 1e-3)


def _f64_param_grads(spec, params, x, g_out):
    """Parameter gradients of sum(out * g_out) for an MLP given as [(kind, in, out)] (kinds as
    mrl_layer_kind) with params [W | b] per layer (+ log_std), evaluated by torch autograd in
    float64 on the CPU: the value both fp32 summation orders (the oracle's serial loops, the
    kernels' tiles) are rounding errors away from."""
    p = torch.tensor(params, dtype=torch.float64, requires_grad=True)
    cur, off = torch.tensor(x, dtype=torch.float64), 0
    for kind, i, o in spec:
        W = p[off:off + i * o].view(i, o); off += i * o
        b = p[off:off + o]; off += o
        cur = cur @ W + b
        if kind == 1:
            cur = torch.relu(cur)
        elif kind == 2:
            cur = torch.tanh(cur)
        elif kind == 3:
            ls = p[off:off + o]; off += o
            cur = torch.cat([cur, torch.clamp(ls, -5.0, 2.0).expand(cur.shape[0], o)], 1)
    (cur * torch.tensor(g_out, dtype=torch.float64)).sum().backward()
    return p.grad.numpy()


def _clip64(g, max_norm):
    n = np.sqrt((g * g).sum())
    return g * (max_norm / (n + 1e-8)) if n > max_norm else g


@pytest.mark.parametrize("env_name,kind", [("LunarLanderV2", "relu"), ("HalfCheetahPlanarV2", "tanh")])
def test_fused_update_minibatch_against_oracle_at_bench_size(mrl, orc, orcmod, ctx, env_name, kind):
    """mrl_ppo_update_minibatch at the sizes bench.py times (hidden width 256, minibatch 4096; the
    discrete 8-256-256-4 ReLU nets of the LunarLander agent and the Gaussian 17-256-256-6 tanh nets of
    the HalfCheetah agent) against the oracle's sequence forward -> loss gradient -> backward -> clip
    -> Adam (-> log_std clamp), deep_agents/ppo/ppo.mojo:2438-2727 and ppo_continuous.mojo:3000-3260.
    Bar: KL, loss gradients and parameter gradients within 1e-4 of the tensor's scale.  The float64
    value of the parameter gradients is evaluated as well, so that the test states how far each
    fp32 summation order is from it."""
    say("case", env_name, kind)
    rng = np.random.default_rng(23)
    E = getattr(mrl, env_name)
    cont = E.NUM_ACTIONS == 0
    od = E.OBS_DIM
    A = E.ACTION_DIM if cont else E.NUM_ACTIONS
    H, MB, N, T = 256, 4096, 1024, 8
    hk = 1 if kind == "relu" else 2
    lin = mrl.LinearReLU if kind == "relu" else mrl.LinearTanh
    head = mrl.StochasticActor(H, A) if cont else mrl.Linear(H, A)
    actor = mrl.seq(lin(od, H), lin(H, H), head)
    critic = mrl.seq(lin(od, H), lin(H, H), mrl.Linear(H, 1))
    spec_a = [(hk, od, H), (hk, H, H), (3 if cont else 0, H, A)]
    spec_c = [(hk, od, H), (hk, H, H), (0, H, 1)]
    la, lc = orcmod.layers(spec_a), orcmod.layers(spec_c)
    hd = actor.OUT_DIM
    # the reference's initialisation scales: Kaiming U(+-sqrt(2/fan_in)) / Xavier over the net's dims
    bound = (2.0 / od) ** 0.5 if cont else (2.0 / (od + A)) ** 0.5
    ap = rng.uniform(-bound, bound, actor.PARAM_SIZE).astype(np.float32) * 0.5
    cp = rng.uniform(-bound, bound, critic.PARAM_SIZE).astype(np.float32) * 0.5
    if cont:
        ap[-A:] = -0.5
    total, aw = N * T, (A if cont else 1)
    r_obs = rng.normal(size=(total, od)).astype(np.float32)
    out0 = np.zeros((total, hd), np.float32)
    orc.orc_mlp_forward(la, 3, total, r_obs, ap, out0, None)
    r_lp = np.zeros(total, np.float32)
    if cont:
        r_act = np.zeros((total, A), np.float32)
        orc.orc_sample_gaussian(out0, total, A, 5, r_act, r_lp)
    else:
        r_act = np.zeros(total, np.float32)
        orc.orc_sample_categorical(out0, total, A, 5, r_act, r_lp)
    r_lp += rng.normal(size=total).astype(np.float32) * 0.1      # ratios on both sides of the clip range
    r_val = rng.normal(size=total).astype(np.float32)
    adv = (rng.normal(size=total) * 2.0 + 0.3).astype(np.float32)
    ret = (r_val + rng.normal(size=total) * 0.5).astype(np.float32)
    rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
    rb.actor_params, rb.critic_params = d(ap), d(cp)
    rb.r_obs.copy_(d(r_obs.reshape(-1))); rb.r_actions.copy_(d(r_act.reshape(-1)))
    rb.r_log_probs.copy_(d(r_lp)); rb.r_values.copy_(d(r_val))
    a_lr, c_lr = 3e-4, 1e-3
    max_norm = 0.5 if cont else 0.1          # below the raw gradient norm: the clip is active
    cls = mrl.ppo.ContinuousUpdate if cont else mrl.ppo.DiscreteUpdate
    upd = cls(ctx, rb, MB, mrl.Adam(lr=a_lr), mrl.Adam(lr=c_lr), target_kl=0.0, max_grad_norm=max_norm)
    upd.advantages.copy_(d(adv)); upd.returns.copy_(d(ret))
    idx = rng.permutation(total)[:MB].astype(np.int32)
    upd.minibatch_step(d(idx))
    ctx.synchronize()

    # ---- the oracle's sequence
    mo, ma, madv = np.ascontiguousarray(r_obs[idx]), np.ascontiguousarray(r_act[idx]), adv[idx].copy()
    orc.orc_normalize_minibatch_host(madv, MB)
    cache = np.zeros(MB * actor.CACHE_SIZE, np.float32)
    out = np.zeros((MB, hd), np.float32)
    orc.orc_mlp_forward(la, 3, MB, mo, ap, out, cache.ctypes.data)
    g_out, kl = np.zeros((MB, hd), np.float32), np.zeros(MB, np.float32)
    if cont:
        orc.orc_ppo_actor_grad_gaussian(out, r_lp[idx], madv, ma, MB, A, 0.2, 0.01, g_out, kl)
    else:
        orc.orc_ppo_actor_grad_discrete(out, r_lp[idx], madv, ma, MB, A, 0.2, 0.01, g_out, kl)
    ga = np.zeros(actor.PARAM_SIZE, np.float32)
    orc.orc_mlp_backward(la, 3, MB, g_out, ap, cache, ga, None)
    ga_raw = ga.copy()
    orc.orc_clip_grad_norm(ga, ga.size, max_norm)
    ap2, st = ap.copy(), np.zeros(2 * ga.size, np.float32)
    orc.orc_adam_step(ap2, ga, st, ga.size, 1, a_lr, 0.9, 0.999, 1e-8)
    if cont:
        orc.orc_clamp_log_std(ap2, ap2.size - A, A)
    ccache = np.zeros(MB * critic.CACHE_SIZE, np.float32)
    v = np.zeros((MB, 1), np.float32)
    orc.orc_mlp_forward(lc, 3, MB, mo, cp, v, ccache.ctypes.data)
    gv = np.zeros(MB, np.float32)
    orc.orc_ppo_critic_grad(v.reshape(-1), r_val[idx], ret[idx], MB, 1 if cont else 0, 1, 0.5, 0.2, gv)
    gc = np.zeros(critic.PARAM_SIZE, np.float32)
    orc.orc_mlp_backward(lc, 3, MB, gv.reshape(MB, 1), cp, ccache, gc, None)
    orc.orc_clip_grad_norm(gc, gc.size, max_norm)
    cp2, st = cp.copy(), np.zeros(2 * gc.size, np.float32)
    orc.orc_adam_step(cp2, gc, st, gc.size, 1, c_lr, 0.9, 0.999, 1e-8)

    def rel(a, b):          # largest difference in units of the tensor's scale
        return float(np.abs(a.astype(np.float64) - b).max() / np.abs(b).max())

    clipped_rows = int((np.abs(g_out).sum(1) == 0).sum()) if not cont else -1
    say("  rows with the ratio outside the clip range (discrete):", clipped_rows, "of", MB)
    assert rel(h(upd.actor_out).reshape(MB, hd), out) < 1e-4
    assert rel(h(upd.values), v.reshape(-1)) < 1e-4
    assert rel(h(upd.kl), kl) < 1e-4
    assert rel(h(upd.g_actor_out).reshape(MB, hd), g_out) < 1e-4
    assert rel(h(upd.g_values), gv) < 1e-4
    # parameter gradients: GPU vs oracle, and both against float64 autograd fed the oracle's loss gradients
    ga64 = _clip64(_f64_param_grads(spec_a, ap, mo, g_out), max_norm)
    gc64 = _clip64(_f64_param_grads(spec_c, cp, mo, gv.reshape(MB, 1)), max_norm)
    e = {"actor gpu-oracle": rel(h(upd.actor_grads), ga), "actor gpu-f64": rel(h(upd.actor_grads), ga64),
         "actor oracle-f64": rel(ga, ga64), "critic gpu-oracle": rel(h(upd.critic_grads), gc),
         "critic gpu-f64": rel(h(upd.critic_grads), gc64), "critic oracle-f64": rel(gc, gc64)}
    say("  parameter-gradient error / tensor scale:", {k: "%.2e" % x for k, x in e.items()})
    assert all(x < 1e-4 for x in e.values()), e
    # per layer block as well (a thin layer's error must not hide behind a wide layer's scale)
    off = 0
    for kind_, i, o in spec_a:
        n = i * o + o + (o if kind_ == 3 else 0)
        assert rel(h(upd.actor_grads)[off:off + n], ga[off:off + n]) < 1e-4, ("actor layer", i, o)
        off += n
    off = 0
    for kind_, i, o in spec_c:
        n = i * o + o
        assert rel(h(upd.critic_grads)[off:off + n], gc[off:off + n]) < 1e-4, ("critic layer", i, o)
        off += n
    assert float(np.sqrt((ga_raw.astype(np.float64) ** 2).sum())) > max_norm
    # Adam's first step is lr * g / (|g| + eps): entries near eps follow their own rounding error, so
    # the step is compared to 3 % of lr and, for entries that are not tiny, to 1e-3 of lr
    for got, want, p0, g, lr in ((h(rb.actor_params), ap2, ap, ga, a_lr), (h(rb.critic_params), cp2, cp, gc, c_lr)):
        np.testing.assert_allclose(got, want, rtol=0, atol=0.03 * lr)
        big = np.abs(g) > 1e-5
        np.testing.assert_allclose((got - p0)[big], (want - p0)[big], rtol=0, atol=1e-3 * lr + 1e-7)


@pytest.mark.parametrize("env_name,kind", [("LunarLanderV2", "relu"), ("HalfCheetahPlanarV2", "tanh")])
def test_update_epoch_trajectory_against_oracle(mrl, orc, orcmod, ctx, env_name, kind):
    """The update path that bench.py times -- PPOUpdate.run_epoch -> mrl_ppo_update_epoch: one
    adv_stats launch ahead, then minibatches with Adam step counts t0 + k + 1 -- over four
    consecutive minibatches of one permutation at hidden width 256 and minibatch 4096, against the
    oracle's sequence (deep_agents/ppo/ppo.mojo:2438-2727, ppo_continuous.mojo:3000-3260) carried
    through the same four steps with its own parameters and Adam state.  Per minibatch k: the
    advantage statistics, the per-sample KL and loss gradients, the clipped parameter gradients
    (1e-4 of the tensor's scale) and the parameters after Adam step t = k (a fraction of lr)."""
    say("case", env_name, kind)
    rng = np.random.default_rng(31)
    E = getattr(mrl, env_name)
    cont = E.NUM_ACTIONS == 0
    od = E.OBS_DIM
    A = E.ACTION_DIM if cont else E.NUM_ACTIONS
    H, MB, N, T, K = 256, 4096, 2048, 8, 4
    hk = 1 if kind == "relu" else 2
    lin = mrl.LinearReLU if kind == "relu" else mrl.LinearTanh
    head = mrl.StochasticActor(H, A) if cont else mrl.Linear(H, A)
    actor = mrl.seq(lin(od, H), lin(H, H), head)
    critic = mrl.seq(lin(od, H), lin(H, H), mrl.Linear(H, 1))
    spec_a = [(hk, od, H), (hk, H, H), (3 if cont else 0, H, A)]
    spec_c = [(hk, od, H), (hk, H, H), (0, H, 1)]
    la, lc = orcmod.layers(spec_a), orcmod.layers(spec_c)
    hd = actor.OUT_DIM
    bound = (2.0 / od) ** 0.5 if cont else (2.0 / (od + A)) ** 0.5
    ap0 = rng.uniform(-bound, bound, actor.PARAM_SIZE).astype(np.float32) * 0.5
    cp0 = rng.uniform(-bound, bound, critic.PARAM_SIZE).astype(np.float32) * 0.5
    if cont:
        ap0[-A:] = -0.5
    total = N * T
    assert total == K * MB
    r_obs = rng.normal(size=(total, od)).astype(np.float32)
    out0 = np.zeros((total, hd), np.float32)
    orc.orc_mlp_forward(la, 3, total, r_obs, ap0, out0, None)
    r_lp = np.zeros(total, np.float32)
    if cont:
        r_act = np.zeros((total, A), np.float32)
        orc.orc_sample_gaussian(out0, total, A, 5, r_act, r_lp)
    else:
        r_act = np.zeros(total, np.float32)
        orc.orc_sample_categorical(out0, total, A, 5, r_act, r_lp)
    r_lp += rng.normal(size=total).astype(np.float32) * 0.1
    r_val = rng.normal(size=total).astype(np.float32)
    # every minibatch with its own mean and spread, so that statistics of the wrong minibatch show
    adv = (rng.normal(size=total) * rng.uniform(0.5, 3.0, total // 64).repeat(64) + 0.3).astype(np.float32)
    ret = (r_val + rng.normal(size=total) * 0.5).astype(np.float32)
    perm = rng.permutation(total).astype(np.int32)
    a_lr, c_lr = 3e-4, 1e-3
    max_norm = 0.5 if cont else 0.1
    cls = mrl.ppo.ContinuousUpdate if cont else mrl.ppo.DiscreteUpdate

    # ---- GPU: k minibatches from the same start, k = 1 .. K (what run_epoch leaves after each)
    gpu = []
    for k in range(1, K + 1):
        rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
        rb.actor_params, rb.critic_params = d(ap0), d(cp0)
        rb.r_obs.copy_(d(r_obs.reshape(-1))); rb.r_actions.copy_(d(r_act.reshape(-1)))
        rb.r_log_probs.copy_(d(r_lp)); rb.r_values.copy_(d(r_val))
        aopt, copt = mrl.Adam(lr=a_lr), mrl.Adam(lr=c_lr)
        upd = cls(ctx, rb, MB, aopt, copt, target_kl=0.0, max_grad_norm=max_norm)
        upd.advantages.copy_(d(adv)); upd.returns.copy_(d(ret))
        upd.run_epoch(d(perm[:k * MB]))
        ctx.synchronize()
        assert aopt.t == k and copt.t == k
        gpu.append(dict(ap=h(rb.actor_params), cp=h(rb.critic_params), ga=h(upd.actor_grads), gc=h(upd.critic_grads),
                        kl=h(upd.kl), g_out=h(upd.g_actor_out).reshape(MB, hd), gv=h(upd.g_values),
                        a_st=h(upd.actor_state), c_st=h(upd.critic_state)))
    stats = torch.zeros(2 * K, device="cuda")
    mrl.ppo.minibatch_adv_stats(ctx, d(perm), d(adv), MB, stats)
    stats = h(stats).reshape(K, 2)

    # ---- oracle: the same four steps in sequence
    def rel(a, b):
        return float(np.abs(a.astype(np.float64) - b).max() / np.abs(b).max())

    ap, cp = ap0.copy(), cp0.copy()
    a_st, c_st = np.zeros(2 * ap.size, np.float32), np.zeros(2 * cp.size, np.float32)
    clipped_steps = 0
    for k in range(1, K + 1):
        idx = perm[(k - 1) * MB:k * MB]
        mo, ma, madv = np.ascontiguousarray(r_obs[idx]), np.ascontiguousarray(r_act[idx]), adv[idx].copy()
        raw = madv.copy()
        orc.orc_normalize_minibatch_host(madv, MB)
        # advantage statistics: the kernel's (mean, sqrt(var + 1e-8)) reproduce the oracle's normalised values
        mean64, std64 = raw.astype(np.float64).mean(), raw.astype(np.float64).std()
        assert abs(stats[k - 1, 0] - mean64) < 1e-5 * (abs(mean64) + std64)
        assert abs(stats[k - 1, 1] - np.sqrt(std64 ** 2 + 1e-8)) < 1e-5 * std64
        np.testing.assert_allclose((raw - stats[k - 1, 0]) / (stats[k - 1, 1] + np.float32(1e-8)), madv,
                                   rtol=0, atol=2e-5)
        cache = np.zeros(MB * actor.CACHE_SIZE, np.float32)
        out = np.zeros((MB, hd), np.float32)
        orc.orc_mlp_forward(la, 3, MB, mo, ap, out, cache.ctypes.data)
        g_out, kl = np.zeros((MB, hd), np.float32), np.zeros(MB, np.float32)
        if cont:
            orc.orc_ppo_actor_grad_gaussian(out, r_lp[idx], madv, ma, MB, A, 0.2, 0.01, g_out, kl)
        else:
            orc.orc_ppo_actor_grad_discrete(out, r_lp[idx], madv, ma, MB, A, 0.2, 0.01, g_out, kl)
        ga = np.zeros(actor.PARAM_SIZE, np.float32)
        orc.orc_mlp_backward(la, 3, MB, g_out, ap, cache, ga, None)
        clipped_steps += float(np.sqrt((ga.astype(np.float64) ** 2).sum())) > max_norm
        orc.orc_clip_grad_norm(ga, ga.size, max_norm)
        ap_prev, cp_prev = ap.copy(), cp.copy()
        orc.orc_adam_step(ap, ga, a_st, ga.size, k, a_lr, 0.9, 0.999, 1e-8)
        if cont:
            orc.orc_clamp_log_std(ap, ap.size - A, A)
        ccache = np.zeros(MB * critic.CACHE_SIZE, np.float32)
        v = np.zeros((MB, 1), np.float32)
        orc.orc_mlp_forward(lc, 3, MB, mo, cp, v, ccache.ctypes.data)
        gv = np.zeros(MB, np.float32)
        orc.orc_ppo_critic_grad(v.reshape(-1), r_val[idx], ret[idx], MB, 1 if cont else 0, 1, 0.5, 0.2, gv)
        gc = np.zeros(critic.PARAM_SIZE, np.float32)
        orc.orc_mlp_backward(lc, 3, MB, gv.reshape(MB, 1), cp, ccache, gc, None)
        orc.orc_clip_grad_norm(gc, gc.size, max_norm)
        orc.orc_adam_step(cp, gc, c_st, gc.size, k, c_lr, 0.9, 0.999, 1e-8)

        g = gpu[k - 1]
        e = {"kl": rel(g["kl"], kl), "g_out": rel(g["g_out"], g_out), "gv": rel(g["gv"], gv),
             "actor grads": rel(g["ga"], ga), "critic grads": rel(g["gc"], gc),
             "actor m": rel(g["a_st"][0::2], a_st[0::2]), "critic m": rel(g["c_st"][0::2], c_st[0::2]),
             "actor v": rel(g["a_st"][1::2], a_st[1::2]), "critic v": rel(g["c_st"][1::2], c_st[1::2])}
        say("  minibatch", k, {n_: "%.1e" % x for n_, x in e.items()})
        assert all(x < 1e-4 for x in e.values()), (k, e)
        # parameters after Adam step t = k.  A step is lr * m_hat / (sqrt(v_hat) + eps), so a gradient
        # error dg (the bar above: 1e-4 of the gradient's scale) moves an entry's step by about
        # lr * dg / sqrt(v_hat) through m_hat and as much again through v_hat: nothing for entries with a
        # solid second moment, the whole step for entries whose gradients sit near eps.  Per entry and
        # step taken: lr * min(10 %, 2e-4 * scale / sqrt(v_hat)).
        for got, want, prev, grad, st, lr in ((g["ap"], ap, ap_prev, ga, a_st, a_lr), (g["cp"], cp, cp_prev, gc, c_st, c_lr)):
            v_hat = st[1::2].astype(np.float64) / (1.0 - 0.999 ** k)
            bound = np.minimum(0.1, 2e-4 * np.abs(grad).max() / (np.sqrt(v_hat) + 1e-12))
            diff = np.abs(got.astype(np.float64) - want)
            assert (diff <= k * lr * bound + 2e-7).all(), (k, float((diff / (k * lr * bound + 2e-7)).max()))
            say("    Adam step %d: largest difference / allowance %.2f, median allowance %.3f of lr" % (
                k, float((diff / (k * lr * bound + 2e-7)).max()), float(np.median(bound))))
            assert np.abs(want - prev).max() > 0.5 * lr                   # a step was taken
    say("  minibatches whose actor gradient was clipped:", clipped_steps, "of", K)
    assert clipped_steps >= 1                   # the clip ran under the comparison at least once
    if cont:
        assert np.all(gpu[-1]["ap"][-A:] >= -5.0) and np.all(gpu[-1]["ap"][-A:] <= 2.0)


def test_update_driver_runs_epochs_and_stops_on_kl(mrl, ctx):
    """PPOUpdate.update end to end on a small LunarLander rollout: permutation drawn on the device,
    the KL flag raised on the device stops the epochs, parameters stay finite."""
    N, T, MB = 256, 16, 512
    E = mrl.LunarLanderV2
    actor = mrl.seq(mrl.LinearReLU(8, 64), mrl.LinearReLU(64, 64), mrl.Linear(64, 4))
    critic = mrl.seq(mrl.LinearReLU(8, 64), mrl.LinearReLU(64, 64), mrl.Linear(64, 1))
    anet = mrl.Network(ctx, actor, mrl.Adam(lr=3e-4), mrl.Xavier(seed=1))
    cnet = mrl.Network(ctx, critic, mrl.Adam(lr=1e-3), mrl.Xavier(seed=2))
    rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
    rb.actor_params, rb.critic_params = anet.params, cnet.params
    E.reset_kernel_gpu(ctx, rb.states, 5)
    rb.obs.copy_(rb.states.view(N, 192)[:, :8].reshape(-1))
    desc = rb.descriptor()
    for t in range(T):
        mrl.ppo.rollout_step(ctx, desc, t, 10 + t, 0, 900 + t)
    upd = mrl.ppo.DiscreteUpdate(ctx, rb, MB, anet.optimizer, cnet.optimizer, target_kl=0.0)
    before = anet.params.clone()
    assert upd.update(2, seed=4) == 2
    assert anet.optimizer.t == 2 * (N * T // MB)
    assert torch.isfinite(anet.params).all() and not torch.equal(before, anet.params)
    # a huge learning rate moves the policy far in one epoch: the device flag must stop the update
    anet.optimizer.lr = 0.5
    upd2 = mrl.ppo.DiscreteUpdate(ctx, rb, MB, anet.optimizer, cnet.optimizer, target_kl=1e-4)
    ran = upd2.update(10, seed=5)
    stopped, mean_kl = upd2.kl_stopped()
    assert stopped and ran < 10 and mean_kl > 1e-4
    applied = int(upd2.kl_flag[2].item())
    assert applied < ran * (N * T // MB)
    assert anet.optimizer.t == 2 * (N * T // MB) + applied == cnet.optimizer.t
    # nothing moves once the stop has fired
    frozen = anet.params.clone()
    upd2.minibatch_step(upd2.indices[:MB])
    ctx.synchronize()
    assert torch.equal(frozen, anet.params)


@pytest.mark.parametrize("env_name,kind,MB,HID", [("LunarLanderV2", "relu", 4096, 256), ("LunarLanderV2", "tanh", 1000, 256),
                                                  ("HalfCheetahPlanarV2", "tanh", 777, 256),
                                                  # hidden width 64: the fused kernel also leaves the hidden layer's
                                                  # weight gradient per row tile (no weight-gradient launch)
                                                  ("CartPoleEnv", "tanh", 4096, 64), ("PendulumV2", "tanh", 1000, 64),
                                                  ("CartPoleEnv", "relu", 777, 64)])
def test_fused_update_minibatch_equals_its_parts(mrl, ctx, env_name, kind, MB, HID):
    """mrl_ppo_update_minibatch on nets of hidden width 256 or 64 (one kernel takes a row tile forward,
    through the loss and back) against the same minibatch issued call by call: gather,
    normalise, forward with cache, loss gradients, backward, clip, Adam.  The fused kernel sums
    in a different order, hence MLP tolerances on the gradients."""
    say("case", env_name, kind, MB, HID)
    E = getattr(mrl, env_name)
    cont = E.NUM_ACTIONS == 0
    lin = mrl.LinearReLU if kind == "relu" else mrl.LinearTanh
    A = E.ACTION_DIM if cont else E.NUM_ACTIONS
    head = mrl.StochasticActor(HID, A) if cont else mrl.Linear(HID, A)
    actor = mrl.seq(lin(E.OBS_DIM, HID), lin(HID, HID), head)
    critic = mrl.seq(lin(E.OBS_DIM, HID), lin(HID, HID), mrl.Linear(HID, 1))
    N, T = 512, 8
    g = torch.Generator(device="cuda").manual_seed(11)
    rnd = lambda n, s=1.0: (torch.rand(n, device="cuda", generator=g) - 0.5) * 2 * s
    rb = mrl.ppo.RolloutBuffers(ctx, E, actor, critic, N, T)
    rb.actor_params, rb.critic_params = rnd(actor.PARAM_SIZE, 0.15), rnd(critic.PARAM_SIZE, 0.15)
    total, aw = N * T, rb.act_width
    rb.r_obs.copy_(rnd(total * E.OBS_DIM))
    rb.r_actions.copy_(rnd(total * aw) if cont else torch.randint(0, A, (total,), device="cuda", generator=g).float())
    rb.r_log_probs.copy_(rnd(total, 0.3) - (2.0 if cont else 1.2))
    rb.r_values.copy_(rnd(total))
    aopt, copt = mrl.Adam(lr=3e-4), mrl.Adam(lr=1e-3)
    cls = mrl.ppo.ContinuousUpdate if cont else mrl.ppo.DiscreteUpdate
    upd = cls(ctx, rb, MB, aopt, copt, target_kl=0.0)
    upd.advantages.copy_(rnd(total, 2.0) + 0.3)
    upd.returns.copy_(rnd(total))
    idx = torch.randperm(total, device="cuda", generator=g)[:MB].to(torch.int32)
    ap0, cp0 = rb.actor_params.clone(), rb.critic_params.clone()
    upd.minibatch_step(idx)
    ctx.synchronize()

    # ---- the same minibatch, call by call, on copies
    z = lambda n: torch.zeros(n, device="cuda")
    hd = actor.OUT_DIM
    mb = (z(MB * E.OBS_DIM), z(MB * aw), z(MB), z(MB), z(MB), z(MB))
    mrl.ppo.gather_minibatch(ctx, idx, (rb.r_obs, rb.r_actions, upd.advantages, upd.returns, rb.r_log_probs, rb.r_values),
                             mb, E.OBS_DIM, aw)
    m_obs, m_act, m_adv, m_ret, m_lp, m_val = mb
    mrl.ppo.normalize_advantages(ctx, m_adv)
    a_out, vals = z(MB * hd), z(MB)
    a_cache, c_cache = z(MB * actor.CACHE_SIZE), z(MB * critic.CACHE_SIZE)
    actor.forward_gpu_ws(ctx, a_out, m_obs, ap0, a_cache)
    critic.forward_gpu_ws(ctx, vals, m_obs, cp0, c_cache)
    g_out, kl, g_val = z(MB * hd), z(MB), z(MB)
    if cont:
        mrl.ppo.ppo_continuous_actor_grad(ctx, g_out, kl, a_out, m_lp, m_adv, m_act, 0.2, 0.01)
    else:
        mrl.ppo.ppo_actor_grad_with_kl(ctx, g_out, kl, a_out, m_lp, m_adv, m_act, 0.2, 0.01)
    mrl.ppo.ppo_critic_grad(ctx, g_val, vals, m_ret, 0.5, old_values=m_val, clip_epsilon=0.2, continuous=cont)
    ga, gc = z(actor.PARAM_SIZE), z(critic.PARAM_SIZE)
    actor.backward_gpu_ws(ctx, None, g_out, ap0, a_cache, ga)
    critic.backward_gpu_ws(ctx, None, g_val, cp0, c_cache, gc)
    mrl.ppo.clip_grad_norm(ctx, ga, 0.5)
    mrl.ppo.clip_grad_norm(ctx, gc, 0.5)
    ap1, cp1 = ap0.clone(), cp0.clone()
    mrl.Adam(lr=3e-4).step_gpu(ctx, ap1, ga, z(2 * actor.PARAM_SIZE))
    mrl.Adam(lr=1e-3).step_gpu(ctx, cp1, gc, z(2 * critic.PARAM_SIZE))
    if cont:
        mrl.ppo.clamp_log_std_params(ctx, ap1, actor.PARAM_SIZE - A, A)
    ctx.synchronize()

    torch.testing.assert_close(upd.actor_out, a_out, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(upd.values, vals, rtol=1e-4, atol=1e-5)
    torch.testing.assert_close(upd.kl, kl, rtol=1e-3, atol=1e-5)
    torch.testing.assert_close(upd.g_actor_out, g_out, rtol=1e-3, atol=1e-7)
    torch.testing.assert_close(upd.g_values, g_val, rtol=1e-3, atol=1e-8)
    scale = lambda t: float(t.abs().max())
    torch.testing.assert_close(upd.actor_grads, ga, rtol=0.0, atol=1e-4 * scale(ga))
    torch.testing.assert_close(upd.critic_grads, gc, rtol=0.0, atol=1e-4 * scale(gc))
    # Adam's first step moves every parameter by about lr; both paths must agree on the sign and size
    torch.testing.assert_close(rb.actor_params - ap0, ap1 - ap0, rtol=0.0, atol=0.05 * 3e-4)
    torch.testing.assert_close(rb.critic_params - cp0, cp1 - cp0, rtol=0.0, atol=0.05 * 1e-3)
