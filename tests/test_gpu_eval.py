"""evaluate_gpu and the checkpoint round trip of the PPO agents on the device.

evaluate_gpu is checked against the reference's literal sequence per step (actor forward ->
sample or deterministic action -> step_kernel_gpu -> host accounting -> selective_reset_kernel_gpu
-> observation from the state row, deep_agents/ppo/ppo_continuous.mojo:880-940) issued call by
call from here; each of those calls has its own oracle test."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ctx(mrl):
    return mrl.DeviceContext("cuda:0")


def test_greedy_actions(mrl, ctx):
    g = torch.Generator(device="cuda").manual_seed(1)
    n, A = 1000, 4
    logits = torch.rand(n * A, device="cuda", generator=g)
    lv = logits.view(n, A)
    lv[::7, 2] = lv[::7, 0]            # ties: the first of the equal maxima wins
    lv[::7, 0] += 0.0
    lv[5::11] = 0.25                   # a row of equal logits -> action 0
    acts = torch.full((n,), -1.0, device="cuda")
    mrl.ppo.greedy_actions(ctx, logits, acts, n, False)
    ctx.synchronize()
    want = np.argmax(lv.cpu().numpy(), axis=1).astype(np.float32)   # numpy: first maximum
    assert np.array_equal(acts.cpu().numpy(), want)
    out = torch.rand(n * 2 * 3, device="cuda", generator=g)
    mean = torch.zeros(n * 3, device="cuda")
    mrl.ppo.greedy_actions(ctx, out, mean, n, True)
    ctx.synchronize()
    assert torch.equal(mean.view(n, 3), out.view(n, 6)[:, :3])


def _by_hand(mrl, ctx, agent, env, num_episodes, max_steps, stochastic):
    N = agent.n_envs
    aw = env.ACTION_DIM if agent.continuous else 1
    dev = "cuda"
    states = torch.zeros(N * env.STATE_SIZE, device=dev)
    obs = torch.zeros(N * env.OBS_DIM, device=dev)
    actions, logp = torch.zeros(N * aw, device=dev), torch.zeros(N, device=dev)
    out = torch.zeros(N * agent.actor.model.OUT_DIM, device=dev)
    rewards, dones = torch.zeros(N, device=dev), torch.zeros(N, device=dev)
    env.reset_kernel_gpu(ctx, states, 0)
    obs.copy_(states.view(N, env.STATE_SIZE)[:, :env.OBS_DIM].reshape(-1))
    current, finished, step = np.zeros(N), [], 0
    while len(finished) < num_episodes and step < max_steps:
        agent.actor.model.forward_gpu_no_cache_ws(ctx, out, obs, agent.actor.params)
        if not stochastic:
            mrl.ppo.greedy_actions(ctx, out, actions, N, agent.continuous)
        elif agent.continuous:
            mrl.ppo.sample_continuous_actions(ctx, out, actions, logp, step * 2654435761)
        else:
            mrl.ppo.sample_actions(ctx, out, actions, logp, step * 2654435761)
        env.step_kernel_gpu(ctx, states, actions, rewards, dones, obs, step)
        ctx.synchronize()
        r, d = rewards.cpu().numpy().astype(np.float64), dones.cpu().numpy()
        for i in range(N):
            current[i] += r[i]
            if d[i] > 0:
                finished.append(current[i])
                current[i] = 0.0
                if len(finished) >= num_episodes:
                    break
        env.selective_reset_kernel_gpu(ctx, states, dones, step)
        obs.copy_(states.view(N, env.STATE_SIZE)[:, :env.OBS_DIM].reshape(-1))
        step += 1
    return (sum(finished) / len(finished)) if finished else 0.0, len(finished)


@pytest.mark.parametrize("stochastic", [True, False])
def test_evaluate_gpu_continuous_equals_the_reference_sequence(mrl, ctx, stochastic):
    print("case pendulum stochastic", stochastic, flush=True)
    agent = mrl.DeepPPOContinuousAgent(obs_dim=3, action_dim=1, hidden_dim=64, n_envs=64, init_seed=4)
    agent.build_networks(ctx)
    # 64 envs, every episode lasts 200 steps: 100 episodes = all of round one + envs 0..35 of round two
    got = agent.evaluate_gpu(ctx, mrl.PendulumV2, num_episodes=100, max_steps=450, stochastic=stochastic,
                             steps_per_readback=48)
    want, cnt = _by_hand(mrl, ctx, agent, mrl.PendulumV2, 100, 450, stochastic)
    assert cnt == 100
    assert got == want and -2000.0 < got < -200.0
    # the step limit ends the evaluation before any episode does
    assert agent.evaluate_gpu(ctx, mrl.PendulumV2, num_episodes=10, max_steps=150) == 0.0


@pytest.mark.parametrize("stochastic", [True, False])
def test_evaluate_gpu_discrete(mrl, ctx, stochastic):
    print("case cartpole stochastic", stochastic, flush=True)
    agent = mrl.DeepPPOAgent(obs_dim=4, num_actions=2, hidden_dim=64, n_envs=96, init_seed=6)
    agent.build_networks(ctx)
    got = agent.evaluate_gpu(ctx, mrl.CartPoleEnv, num_episodes=150, max_steps=400, stochastic=stochastic,
                             steps_per_readback=7)
    want, cnt = _by_hand(mrl, ctx, agent, mrl.CartPoleEnv, 150, 400, stochastic)
    assert cnt == 150 and got == want
    assert 5.0 < got < 200.0    # an untrained policy keeps the pole up for a few dozen steps at best


def test_checkpoint_round_trip_on_device(mrl, ctx, tmp_path):
    path = str(tmp_path / "agent.ckpt")
    a = mrl.DeepPPOAgent(obs_dim=4, num_actions=2, hidden_dim=64, rollout_len=32, n_envs=256, gpu_minibatch_size=1024,
                         num_epochs=2, target_kl=0.0, init_seed=1, checkpoint_every=100, checkpoint_path=path)
    a.train_gpu(ctx, mrl.CartPoleEnv, num_episodes=10**9, max_rollouts=2, seed=3)
    # the auto-checkpoint fired at the end of a rollout (more than 100 episodes finish in the first one)
    saved = open(path).read()
    assert saved.startswith("# mojo-rl checkpoint v1\n# type: ppo_agent\n")
    a.save_checkpoint(path)
    b = mrl.DeepPPOAgent(obs_dim=4, num_actions=2, hidden_dim=64, n_envs=256, init_seed=9)
    b.load_checkpoint(path, ctx)
    for x, y in ((a.actor, b.actor), (a.critic, b.critic)):
        assert torch.equal(x.params, y.params) and torch.equal(x.optimizer_state, y.optimizer_state)
        assert float(x.optimizer_state.abs().sum()) > 0.0
    assert a.evaluate_gpu(ctx, mrl.CartPoleEnv, 50, 300) == b.evaluate_gpu(ctx, mrl.CartPoleEnv, 50, 300)
    with pytest.raises(ValueError):
        mrl.DeepPPOAgent(obs_dim=4, num_actions=2).load_checkpoint(path)   # no networks yet and no context

    cpath = str(tmp_path / "cont.ckpt")
    c = mrl.DeepPPOContinuousAgent(obs_dim=3, action_dim=1, hidden_dim=64, rollout_len=16, n_envs=128,
                                   gpu_minibatch_size=1024, num_epochs=1, target_kl=0.0, init_seed=2)
    c.train_gpu(ctx, mrl.PendulumV2, num_episodes=10**9, max_rollouts=1, seed=1)
    assert c.train_step_count == 16 * 128
    c.save_checkpoint(cpath)
    e = mrl.DeepPPOContinuousAgent(obs_dim=3, action_dim=1, hidden_dim=64, n_envs=128, init_seed=7)
    e.load_checkpoint(cpath, ctx)
    assert e.train_step_count == 16 * 128
    for x, y in ((c.actor, e.actor), (c.critic, e.critic)):
        assert torch.equal(x.params, y.params) and torch.equal(x.optimizer_state, y.optimizer_state)
    # a network on its own
    npath = str(tmp_path / "net.ckpt")
    c.actor.save_checkpoint(npath)
    e.actor.params.zero_()
    e.actor.load_checkpoint(npath)
    assert torch.equal(c.actor.params, e.actor.params)
