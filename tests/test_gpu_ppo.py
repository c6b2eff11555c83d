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
    # the inverse-CDF comparison u < cumsum can flip when u is within an ulp of a boundary
    same = h(a) == a_h
    assert same.mean() > 0.9995, same.mean()
    np.testing.assert_allclose(h(lp)[same], lp_h[same], rtol=1e-5, atol=1e-6)
    assert set(np.unique(h(a))) <= {0.0, 1.0, 2.0, 3.0}


def test_sample_gaussian(mrl, orc, ctx):
    rng = np.random.default_rng(1)
    n, A = 4096, 6
    out = np.concatenate([rng.normal(size=(n, A)), rng.uniform(-6, 3, (n, A))], 1).astype(np.float32)
    a_h, lp_h = np.zeros((n, A), np.float32), np.zeros(n, np.float32)
    orc.orc_sample_gaussian(out, n, A, 4242, a_h, lp_h)
    a, lp = torch.zeros(n * A, device="cuda"), torch.zeros(n, device="cuda")
    mrl.ppo.sample_continuous_actions(ctx, d(out.reshape(-1)), a, lp, 4242)
    ctx.synchronize()
    np.testing.assert_allclose(h(a).reshape(n, A), a_h, rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(h(lp), lp_h, rtol=1e-4, atol=1e-3)


@pytest.mark.parametrize("T,N", [(1, 1), (7, 65), (512, 4096)])
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
    flip = ((gg == 0).all(1) != (g_h == 0).all(1))     # ratio within an ulp of the clip boundary
    assert flip.mean() < 1e-3
    np.testing.assert_allclose(gg[~flip], g_h[~flip], rtol=2e-5, atol=1e-9)
    np.testing.assert_allclose(h(kl), kl_h, rtol=1e-5, atol=1e-6)
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
    flip = ((gg == 0).all(1) != (g_h == 0).all(1))
    assert flip.mean() < 1e-3
    np.testing.assert_allclose(gg[~flip], g_h[~flip], rtol=1e-4, atol=1e-9)
    np.testing.assert_allclose(h(kl), kl_h, rtol=1e-3, atol=1e-6)
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
    same = r_actions == a_h
    assert same.mean() > 0.995, same.mean()
    np.testing.assert_allclose(r_logp[same], lp_h[same], rtol=1e-4, atol=1e-5)
