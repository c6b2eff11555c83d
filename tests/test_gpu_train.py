"""End to end: the agents' train_gpu loop (rollout -> GAE -> epochs of minibatch updates, all on
the device) actually learns.  CartPole is the reference's own smoke environment for PPO
(examples/cartpole PPO scripts): random play averages about 22 steps per episode."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


def test_discrete_agent_learns_cartpole(mrl):
    ctx = mrl.DeviceContext("cuda:0")
    agent = mrl.DeepPPOAgent(obs_dim=4, num_actions=2, hidden_dim=64, rollout_len=128, n_envs=512,
                             gpu_minibatch_size=2048, num_epochs=4, target_kl=0.0, anneal_lr=False,
                             entropy_coef=0.01, init_seed=1)
    m = agent.train_gpu(ctx, mrl.CartPoleEnv, num_episodes=10**9, max_rollouts=40, seed=3)
    assert m.rollouts == 40 and m.total_steps == 40 * 128 * 512
    early = float(np.mean(m.episode_rewards[:500]))
    late = float(np.mean(m.episode_rewards[-500:]))
    print("cartpole mean return: first 500 episodes %.1f, last 500 episodes %.1f" % (early, late), flush=True)
    assert early < 40.0            # starts near random play
    assert late > 4.0 * early      # and has clearly learned to balance
    assert torch.isfinite(agent.actor.params).all() and torch.isfinite(agent.critic.params).all()
    assert agent.actor.optimizer.t == 40 * 4 * (128 * 512 // 2048)


def test_continuous_agent_improves_pendulum(mrl):
    ctx = mrl.DeviceContext("cuda:0")
    agent = mrl.DeepPPOContinuousAgent(obs_dim=3, action_dim=1, hidden_dim=64, rollout_len=200, n_envs=1024,
                                       gpu_minibatch_size=4096, num_epochs=10, target_kl=0.0, anneal_lr=False,
                                       actor_lr=3e-4, critic_lr=1e-3, init_seed=2)
    m = agent.train_gpu(ctx, mrl.PendulumV2, num_episodes=10**9, max_rollouts=40, seed=5)
    # every episode lasts exactly 200 steps: 1024 episodes per rollout
    assert all(s == 200.0 for s in m.episode_steps[:100])
    early = float(np.mean(m.episode_rewards[:1024]))
    late = float(np.mean(m.episode_rewards[-1024:]))
    print("pendulum mean return: first rollout %.1f, last rollout %.1f" % (early, late), flush=True)
    assert early < -900.0          # random torques: about -1200
    assert late > early + 200.0    # swing-up cost goes down
    assert torch.isfinite(agent.actor.params).all()
    # the log_std clamp holds
    ls = agent.actor.params[-1:]
    assert (ls >= -5.0).all() and (ls <= 2.0).all()


def test_continuous_agent_runs_on_the_continuous_lunar_lander(mrl):
    """The continuous-action LunarLander overload behind the continuous agent: the fused collection
    kernel (hidden width 256), GAE and the update run and keep every buffer finite."""
    ctx = mrl.DeviceContext("cuda:0")
    agent = mrl.DeepPPOContinuousAgent(obs_dim=8, action_dim=2, hidden_dim=256, rollout_len=64, n_envs=512,
                                       gpu_minibatch_size=4096, num_epochs=2, target_kl=0.0, init_seed=3)
    m = agent.train_gpu(ctx, mrl.LunarLanderV2Continuous, num_episodes=10**9, max_rollouts=3, seed=2)
    assert mrl.ppo.rollout_fused(agent.rb.descriptor())
    assert m.rollouts == 3 and m.total_steps == 3 * 64 * 512
    assert len(m.episode_rewards) > 0 and all(np.isfinite(m.episode_rewards))
    assert torch.isfinite(agent.actor.params).all() and torch.isfinite(agent.critic.params).all()
    assert torch.isfinite(agent.rb.states).all()
    got = agent.evaluate_gpu(ctx, mrl.LunarLanderV2Continuous, num_episodes=64, max_steps=400)
    assert np.isfinite(got) and got < 0.0     # three rollouts do not make a pilot


@pytest.mark.parametrize("env_name,obs_dim,action_dim", [("BipedalWalkerV2", 24, 4), ("HalfCheetahPlanarV2", 17, 6)])
def test_continuous_agent_runs_on_the_walkers(mrl, env_name, obs_dim, action_dim):
    """The walkers behind the continuous agent with the reference's 256-wide nets: the fused collection
    kernel, GAE and the update run over several rollouts and keep every buffer finite; the default KL
    early stop is on."""
    ctx = mrl.DeviceContext("cuda:0")
    E = getattr(mrl, env_name)
    agent = mrl.DeepPPOContinuousAgent(obs_dim=obs_dim, action_dim=action_dim, hidden_dim=256, rollout_len=96,
                                       n_envs=400, gpu_minibatch_size=4096, num_epochs=3, init_seed=5)
    m = agent.train_gpu(ctx, E, num_episodes=10**9, max_rollouts=4, seed=1)
    assert mrl.ppo.rollout_fused(agent.rb.descriptor())
    assert m.rollouts == 4 and m.total_steps == 4 * 96 * 400
    assert all(np.isfinite(m.episode_rewards)) and all(1 <= n <= 2000 for n in m.episode_steps)
    if env_name == "BipedalWalkerV2":
        assert len(m.episode_rewards) > 100        # an untrained walker falls within a few dozen steps
    assert torch.isfinite(agent.actor.params).all() and torch.isfinite(agent.critic.params).all()
    assert torch.isfinite(agent.rb.states).all() and torch.isfinite(agent.rb.r_log_probs).all()
    assert agent.actor.optimizer.t > 0


def test_observation_noise_enters_the_rollout(mrl, orc):
    """obs_noise_std > 0 (ppo_continuous.mojo:2557-2564, :2705-2713): the policy sees noisy
    observations from the first step on, the env rows stay clean, and the stored observation of step
    0 is the reset observation plus the oracle's noise for the initial seed 42."""
    ctx = mrl.DeviceContext("cuda:0")
    N, T, std = 256, 8, 0.05
    agent = mrl.DeepPPOContinuousAgent(obs_dim=3, action_dim=1, hidden_dim=64, rollout_len=T, n_envs=N,
                                       gpu_minibatch_size=512, num_epochs=1, target_kl=0.0, obs_noise_std=std, init_seed=4)
    assert (agent.num_epochs, agent.entropy_coef, agent.action_scale, agent.action_bias) == (1, 0.01, 1.0, 0.0)
    assert mrl.DeepPPOContinuousAgent(3, 1).target_kl == 0.02 and mrl.DeepPPOContinuousAgent(3, 1).num_epochs == 10
    m = agent.train_gpu(ctx, mrl.PendulumV2, num_episodes=10**9, max_rollouts=1, seed=6)
    assert m.rollouts == 1
    s0 = torch.zeros(N * 8, device="cuda")
    mrl.PendulumV2.reset_kernel_gpu(ctx, s0, 6)
    ctx.synchronize()
    want = s0.view(N, 8)[:, :3].cpu().numpy().copy()
    orc.orc_add_obs_noise(want, N, 3, std, 42)
    np.testing.assert_array_equal(agent.rb.r_obs[:N * 3].cpu().numpy().reshape(N, 3), want)
    # later steps: stored observation = clean observation of the row + noise of that scale
    rows = agent.rb.states.view(N, 8).cpu().numpy()
    last = agent.rb.obs.cpu().numpy().reshape(N, 3)
    z = (last - rows[:, :3]) / std
    assert 0.7 < z.std() < 1.3 and abs(z.mean()) < 0.2
    assert np.abs(np.hypot(rows[:, 0], rows[:, 1]) - 1.0).max() < 1e-5      # the rows themselves carry no noise


class _SignEnv:
    """A host env with the reference's CPU interface: the observation is a random point, the reward is
    1 when the action names the sign of its first entry, an episode lasts `length` steps."""

    def __init__(self, seed, length=8, continuous=False):
        self.rng, self.length, self.continuous = np.random.default_rng(seed), length, continuous
        self.t, self.obs, self.log = 0, None, []          # log: (action, reward, done) of every step

    def _draw(self):
        self.obs = self.rng.uniform(-1, 1, 3).astype(np.float32)
        return self.obs.tolist()

    def reset_obs_list(self):
        self.t = 0
        return self._draw()

    def _step(self, good, action):
        self.t += 1
        done = self.t >= self.length
        self.log.append((action, 1.0 if good else 0.0, done))
        return self._draw(), 1.0 if good else 0.0, done

    def step_obs(self, action):
        assert isinstance(action, int) and not self.continuous
        return self._step((action == 1) == (self.obs[0] > 0), action)

    def step_continuous_vec(self, action):
        assert self.continuous and len(action) == 2 and all(-1.0 <= a <= 1.0 for a in action)
        return self._step((action[0] > 0) == (self.obs[0] > 0), list(action))


@pytest.mark.parametrize("continuous", [False, True])
def test_train_gpu_cpu_env_steps_host_envs_and_learns(mrl, continuous):
    """train_gpu_cpu_env: the envs are the caller's host objects; the rollout buffers hold what they
    reported, the metrics list their episodes in completion order, and the policy learns the task."""
    ctx = mrl.DeviceContext("cuda:0")
    N, T, L = 16, 32, 8
    if continuous:
        agent = mrl.DeepPPOContinuousAgent(3, 2, hidden_dim=64, rollout_len=T, n_envs=N, gpu_minibatch_size=128,
                                           num_epochs=4, actor_lr=3e-3, critic_lr=3e-3, entropy_coef=0.0,
                                           anneal_lr=False, target_kl=0.0, normalize_rewards=False)
    else:
        agent = mrl.DeepPPOAgent(3, 2, hidden_dim=64, rollout_len=T, n_envs=N, gpu_minibatch_size=128,
                                 num_epochs=4, actor_lr=3e-3, critic_lr=3e-3, entropy_coef=0.0,
                                 anneal_lr=False, target_kl=0.0)
    envs = [_SignEnv(100 + i, L, continuous) for i in range(N)]
    with pytest.raises(ValueError):
        agent.train_gpu_cpu_env(ctx, envs[:-1], 10)
    m = agent.train_gpu_cpu_env(ctx, envs, num_episodes=10 ** 9, max_rollouts=1)
    # one rollout: T steps of every env, in the buffers exactly as the envs saw them
    assert m.rollouts == 1 and m.total_steps == N * T and all(len(e.log) == T for e in envs)
    rb = agent.rb
    want_r = np.array([[e.log[t][1] for e in envs] for t in range(T)], np.float32)
    want_d = np.array([[float(e.log[t][2]) for e in envs] for t in range(T)], np.float32)
    np.testing.assert_array_equal(rb.r_rewards.cpu().numpy().reshape(T, N), want_r)
    np.testing.assert_array_equal(rb.r_dones.cpu().numpy().reshape(T, N), want_d)
    acts = rb.r_actions.cpu().numpy().reshape(T, N, -1)
    for t in range(T):
        for i, e in enumerate(envs):
            if continuous:   # the envs get the clipped action, the buffer keeps the raw one
                np.testing.assert_allclose(np.clip(acts[t, i], -1, 1), e.log[t][0], rtol=0, atol=0)
            else:
                assert int(acts[t, i, 0]) == e.log[t][0]
    assert len(m.episode_rewards) == N * T // L and m.episode_steps == [L] * (N * T // L)
    first = float(np.mean(m.episode_rewards))
    # keep training: the returns go up from about L / 2 towards L
    m2 = agent.train_gpu_cpu_env(ctx, envs, num_episodes=10 ** 9, max_rollouts=25)
    last = float(np.mean(m2.episode_rewards[-64:]))
    print("sign env, continuous=%s: mean return %.2f -> %.2f of %d" % (continuous, first, last, L), flush=True)
    assert first < 0.7 * L and last > 0.85 * L
    # the episode target inside a rollout ends the call without an update for that rollout
    t_before = agent.actor.optimizer.t
    seen = [len(e.log) for e in envs]
    m3 = agent.train_gpu_cpu_env(ctx, envs, num_episodes=5)
    assert m3.rollouts == 0 and len(m3.episode_rewards) >= 5 and agent.actor.optimizer.t == t_before
    # ... after the rollout's steps have all been taken: the reference tests the episode target behind its
    # `for t in range(rollout_len)` loop, not inside it (ppo.mojo:3290, :3454-3456), so every env has been
    # stepped T more times and every episode that ended on the way is in the metrics
    assert [len(e.log) - n for e, n in zip(envs, seen)] == [T] * N and m3.total_steps == N * T
    assert len(m3.episode_rewards) == N * T // L
